"""A routed feed-forward: a mixture of small feed-forward layers (experts) of
which every token uses a few.

Router: z = Wr n in float32; scores s = softmax(z) over all router outputs;
the `top` outputs with the largest s + correction are chosen (the correction
moves the choice only) and their weights are their scores s, as they are, not
renormalized. The first `experts` router outputs are real experts,
y = Wdown act(Wup n) without biases; the last `identity` outputs stand for
experts that pass their input through. The result is the weighted sum of the
chosen experts' outputs, added in the order of the choice.

Parameters: width, hidden (an expert's), experts, identity, top, activation
("relu2": the square of max(z, 0); "swiglu": a gated expert, y = Wdown
(silu(Wgate n) * (Wup n)), whose gate matrix is named by `expert_gate`),
scoring ("softmax" over all router outputs, or "sigmoid" of each output by
itself), weigh ("output": a chosen expert's result is multiplied by its
weight; "input": the expert reads its input times its weight and the results
are added as they are), `group_count` and `group_keep` (the router outputs form
group_count equal groups of neighbours; a group's score is the sum of its two
largest score + correction, and only outputs of the group_keep best groups can
be chosen: an output of another group never is, however low the scores
inside the kept groups lie), `normalize` (the
chosen scores are divided by their sum + 1e-20), `route_scale` (a factor on the
weights), `shared` (the PartSpec of a feed-forward that every token uses; its
result is added, multiplied by sigmoid(Wsg n), one number a token, with Wsg the
tensor `shared_gate`), and the tensors' names: `router`, `correction` (None:
no correction), `expert_up` / `expert_down` as patterns with `{e}` for the
expert's number.

The experts' matrices lie stacked, [experts, out, in]. A step sorts its (token,
choice) entries by expert on the device and runs the two products over tiles of
one expert's rows each; the grids are sized by a bound the host knows, so
nothing comes back to the host and a step of this part can be captured.
"""
from __future__ import annotations

from typing import Dict, Optional

import torch

from ..config.plan import PartSpec
from ..kernels import ops
from ..weights.loader import TensorDecl
from .base import Declared, RowsToCombine, StepContext
from .linear import Linear, place_matrix, place_projection, place_vector
from .registry import part_class, register_part


class RoutedExperts:
    role = "feed_forward"
    graph_safe = True     # launches kernels only: a step made of such parts can be captured

    @staticmethod
    def _names(spec: PartSpec) -> Dict[str, str]:
        names = dict(router="router", correction="correction", expert_up="e{e}.up", expert_down="e{e}.down",
                     expert_gate="e{e}.gate", shared_gate="shared.sg")
        names.update(spec.get("names") or {})
        return {k: (None if v is None else f"{spec.prefix}.{v}") for k, v in names.items()}

    @classmethod
    def declare(cls, spec: PartSpec) -> Declared:
        n = cls._names(spec)
        E, F, X, I = spec["width"], spec["hidden"], spec["experts"], spec.get("identity", 0)
        out: Declared = {n["router"]: (TensorDecl((X + I, E)), "matrix")}
        if n["correction"] is not None:
            out[n["correction"]] = (TensorDecl((X + I,), "vector"), "bias")
        for e in range(X):
            if spec.get("activation", "relu2") == "swiglu":
                out[n["expert_gate"].format(e=e)] = (TensorDecl((F, E)), "matrix")
            out[n["expert_up"].format(e=e)] = (TensorDecl((F, E)), "matrix")
            out[n["expert_down"].format(e=e)] = (TensorDecl((E, F)), "matrix")
        if spec.get("shared") is not None:
            out.update(part_class("feed_forward", spec["shared"].kind).declare(spec["shared"]))
            out[n["shared_gate"]] = (TensorDecl((1, E)), "matrix")
        return out

    def __init__(self, spec: PartSpec, tensors: Dict[str, torch.Tensor], device: torch.device,
                 engine_dtype: torch.dtype):
        n = self._names(spec)
        self.width, self.hidden = spec["width"], spec["hidden"]
        self.experts, self.identity, self.top = spec["experts"], int(spec.get("identity", 0)), spec["top"]
        self.activation = spec.get("activation", "relu2")
        self.gated = self.activation == "swiglu"
        if not self.gated and (self.activation not in ops.MOE_EPILOGUES or self.activation in (None, "none")):
            raise ValueError(f"the experts' activation {self.activation!r} is not one the product's epilogue knows")
        self.scoring = spec.get("scoring", "softmax")
        if self.scoring not in ops.MOE_SCORINGS:
            raise ValueError(f"the router's scoring {self.scoring!r} is none of {sorted(ops.MOE_SCORINGS)}")
        self.weigh = spec.get("weigh", "output")
        if self.weigh not in ("output", "input"):
            raise ValueError(f"weigh is 'output' or 'input', got {self.weigh!r}")
        if self.weigh == "input" and (not self.gated or self.identity):
            # w act(W n) = act(W (w n)) holds for no activation here but the gated one's kernel, which takes w itself
            raise ValueError("experts that read their input times their weight are the gated ones, without pass-through experts")
        if not 1 <= self.top <= self.experts + self.identity:
            raise ValueError(f"{self.top} of {self.experts + self.identity} experts cannot be chosen")
        # bfloat16 x bfloat16 products are exact in float32 and the sums are float32: the router runs in 32 bits
        # on the matrix cores too; its input is the norm's output in the engine's dtype
        self.n_router = self.experts + self.identity
        self.group_count, self.group_keep = int(spec.get("group_count") or 1), int(spec.get("group_keep") or 1)
        if self.group_count > 1 and (self.n_router % self.group_count or not 1 <= self.group_keep <= self.group_count
                                     or self.group_keep * (self.n_router // self.group_count) < self.top):
            raise ValueError(f"{self.n_router} router outputs in {self.group_count} groups of which {self.group_keep} "
                             f"stay cannot give {self.top} choices")
        self.normalize, self.route_scale = bool(spec.get("normalize")), float(spec.get("route_scale", 1.0))
        router = tensors[n["router"]]
        self.shared = None
        if spec.get("shared") is not None:
            if self.top > 0 and spec["shared"].get("scratch_tag") is None:
                raise ValueError("a feed-forward inside this one keeps its scratch under a tag of its own (scratch_tag)")
            self.shared = part_class("feed_forward", spec["shared"].kind)(spec["shared"], tensors, device, engine_dtype)
            # the shared expert's gate is one more row of the router's matrix: the same dot products, one launch
            gate = tensors[n["shared_gate"]].reshape(1, self.width)
            if gate.dtype != router.dtype:
                router, gate = router.to(torch.float32), gate.to(torch.float32)
            router = torch.cat([router, gate], dim=0)
        self.router = Linear(place_projection(router, engine_dtype, device))
        if self.shared is not None and self.shared.in_dtype != self.router.in_dtype:
            raise ValueError("the shared expert and the router read their input in one dtype")
        self.correction = None if n["correction"] is None else place_vector(tensors[n["correction"]], device)
        ups = [tensors[n["expert_up"].format(e=e)] for e in range(self.experts)]
        downs = [tensors[n["expert_down"].format(e=e)] for e in range(self.experts)]
        gates = [tensors[n["expert_gate"].format(e=e)] for e in range(self.experts)] if self.gated else []
        if self.experts:
            up, down = torch.stack(ups), torch.stack(downs)
            gate = torch.stack(gates) if self.gated else None
            # The bfloat16 products walk K in steps of 8: a hidden width that is no multiple of 8 is filled up
            # with hidden units of zero weight (act(0) = 0 goes through zero columns of the way back).
            fill = (-self.hidden) % 8
            if fill and engine_dtype != torch.float32:
                up = torch.cat([up, up.new_zeros(self.experts, fill, self.width)], dim=1)
                down = torch.cat([down, down.new_zeros(self.experts, self.width, fill)], dim=2)
                if self.gated:
                    gate = torch.cat([gate, gate.new_zeros(self.experts, fill, self.width)], dim=1)
            if self.gated:
                # an expert's gate rows, then its up rows: one product makes both, a launch behind it gates
                up = torch.cat([gate.to(up.dtype), up], dim=1)
            if engine_dtype != torch.float32 and (self.width % 8 or self.router.in_dtype == torch.float32):
                up, down = up.to(torch.float32), down.to(torch.float32)      # such a width runs in float32 throughout
            self.up = place_matrix(up, engine_dtype, device)
            self.down = place_matrix(down, engine_dtype, device)
        else:
            self.up = self.down = None

    @property
    def in_dtype(self) -> torch.dtype:
        return self.router.in_dtype

    @property
    def forward_rows(self):
        """Everything but the weighted sum over a token's experts: for a block whose next launch (a norm on
        this part's result) makes that sum itself. None where the result is more than that sum."""
        return None if self.shared is not None else self._rows

    def _rows(self, ctx: StepContext, n: torch.Tensor, shared_out: Optional[list] = None) -> RowsToCombine:
        T, top, X = n.shape[0], self.top, self.experts
        ws = ctx.workspace
        rules = dict(scoring=self.scoring, n_router=self.n_router, groups=self.group_count, keep=self.group_keep,
                     normalize=self.normalize, scale=self.route_scale)
        if self.shared is not None:
            # first, while the scratch it shares with the experts' products is free
            stream, ctx.stream = ctx.stream, None          # (its result is weighed before it is added anywhere)
            try:
                shared_out.append(self.shared.forward(ctx, n))
            finally:
                ctx.stream = stream
        z = self.router(ctx, n, torch.float32, "router_logits")
        if shared_out is not None:
            shared_out.append(z)
        choice = ws.get("moe_choice", (T, top), torch.int32)
        weight = ws.get("moe_weight", (T, top), torch.float32)
        entries = T * top
        slot_of_entry = ws.get("moe_slot_of_entry", (entries,), torch.int32)
        y = ws.get("moe_y", (entries, self.width), torch.float32)
        if X:
            rows = ops.moe_tile_rows(entries, X, self.up.dtype)
            tiles = ws.get("moe_tiles", (ops.moe_max_tiles(entries, X, rows), 3), torch.int32)
            entry_of_slot = ws.get("moe_entry_of_slot", (entries,), torch.int32)
            if T <= ops.moe_route_plan_tokens():      # a decode step: choice and plan in one launch
                ops.moe_route_plan(z, self.correction, choice, weight, top, X, rows, slot_of_entry, entry_of_slot, tiles,
                                   **rules)
            else:
                ops.moe_route(z, self.correction, choice, weight, top, **rules)
                ops.moe_plan(choice, X, rows, slot_of_entry, entry_of_slot, tiles)
            if self.gated:
                both = ws.get("moe_gate_up", (entries, self.up.shape[1]), torch.float32, alias="mixer_in")
                ops.moe_gemm(n, self.up, both, tiles, rows, entry_of_slot, gather_div=top)
                hidden = ws.get("moe_hidden", (entries, self.up.shape[1] // 2), self.down.dtype)
                ops.moe_gated(both, weight.view(-1) if self.weigh == "input" else None, entry_of_slot, hidden)
            else:
                hidden = ws.get("moe_hidden", (entries, self.up.shape[1]), self.up.dtype, alias="mixer_in")
                ops.moe_gemm(n, self.up, hidden, tiles, rows, entry_of_slot, gather_div=top, epilogue=self.activation)
            ops.moe_gemm(hidden, self.down, y, tiles, rows)
        else:
            ops.moe_route(z, self.correction, choice, weight, top, **rules)
        return RowsToCombine(y, n, choice, None if self.weigh == "input" else weight, slot_of_entry, X)

    def forward(self, ctx: StepContext, n: torch.Tensor) -> torch.Tensor:
        extra: list = []
        r = self._rows(ctx, n, extra if self.shared is not None else None)
        out = ctx.workspace.get("ffn_out", (n.shape[0], self.width), torch.float32)
        ops.moe_combine(r.y, r.h, r.choice, r.weight, r.slot_of_entry, r.n_experts, out)
        if self.shared is not None:
            y, z = extra
            ops.gated_row_add(out, y, z, self.n_router)
        return out


register_part("feed_forward", "routed_experts", RoutedExperts)
