"""Retention: linear attention with a fixed decay a head, no softmax and no
denominator.

q = Wq h and k = Wk h are [heads, dim], v = Wv h is [heads, vdim], no biases.
q and k are rotated by position (whatever rotation the position part names),
k is then multiplied by dim^(-1/2). Per head, with a state S [dim, vdim]:

    S <- decay_h S + k v^T,    o = S^T q.

Each head's o is divided by its root mean square (no weight); the heads side
by side are multiplied by silu(Wg h) and go through the output projection. A
request's state is S, float32. Angles, the state and every sum of the
recurrence are float32 whatever the engine's dtype.

Parameters: width, heads, dim, vdim, decay (one number a head), position, eps, names.
"""
from __future__ import annotations

from typing import Dict

import torch

from ..cache.pages import FixedArray, FixedSpec
from ..config.plan import PartSpec
from ..kernels import ops
from ..weights.loader import TensorDecl
from .base import Declared, StepContext
from .linear import Linear, place_projection, place_vector
from .registry import part_class, register_part

_DEFAULT_NAMES = dict(q="q", k="k", v="v", g="g", o="o")


class Retention:
    role = "mixer"
    graph_safe = True     # launches kernels only: a step made of such parts can be captured

    @staticmethod
    def _names(spec: PartSpec) -> Dict[str, str]:
        names = dict(_DEFAULT_NAMES)
        names.update(spec.get("names") or {})
        return {k: f"{spec.prefix}.{v}" for k, v in names.items()}

    @classmethod
    def declare(cls, spec: PartSpec) -> Declared:
        n = cls._names(spec)
        E, H, d, dv = spec["width"], spec["heads"], spec["dim"], spec["vdim"]
        return {
            n["q"]: (TensorDecl((H * d, E)), "matrix"),
            n["k"]: (TensorDecl((H * d, E)), "matrix"),
            n["v"]: (TensorDecl((H * dv, E)), "matrix"),
            n["g"]: (TensorDecl((H * dv, E)), "matrix"),
            n["o"]: (TensorDecl((E, H * dv)), "matrix"),
        }

    def __init__(self, spec: PartSpec, tensors: Dict[str, torch.Tensor], device: torch.device,
                 engine_dtype: torch.dtype):
        n = self._names(spec)
        self.width, self.heads, self.dim, self.vdim = spec["width"], spec["heads"], spec["dim"], spec["vdim"]
        self.eps = float(spec["eps"])
        decay = [float(x) for x in spec["decay"]]
        if len(decay) != self.heads:
            raise ValueError(f"{len(decay)} decays for {self.heads} heads")
        if self.dim > ops.DECAY_SCAN_MAX_DIM:
            raise ValueError(f"the recurrence kernel takes up to {ops.DECAY_SCAN_MAX_DIM} state rows a head, got {self.dim}")
        self.decay = place_vector(torch.tensor(decay, dtype=torch.float64).to(torch.float32), device)
        ws = [tensors[n[x]] for x in ("q", "k", "v", "g")]
        if len({w.dtype for w in ws}) > 1:
            ws = [w.to(torch.float32) for w in ws]
        # one projection for q | k | v | g: the same dot products, one launch
        self.proj = Linear(place_projection(torch.cat(ws, dim=0), engine_dtype, device))
        self.out = Linear(place_projection(tensors[n["o"]], engine_dtype, device))
        pos = spec.get("position") or PartSpec("none")
        self.position = part_class("position", pos.kind)(pos, device)
        if self.position.rotary_dim > self.dim:
            raise ValueError("the rotated part of a head cannot be wider than the head")

    @property
    def in_dtype(self) -> torch.dtype:
        return self.proj.in_dtype

    def cache_spec(self, page_size: int) -> FixedSpec:
        return FixedSpec(arrays=(FixedArray("state", (self.heads, self.dim, self.vdim), "float32", 0.0),))

    def forward(self, ctx: StepContext, site: int, owns_cache: bool, h: torch.Tensor) -> torch.Tensor:
        if not owns_cache:
            raise ValueError("a recurrence's state cannot be read from another layer")
        T, H, d, dv = h.shape[0], self.heads, self.dim, self.vdim
        rows = self.proj(ctx, h, torch.float32, "retention_rows", alias="mixer_in")      # q | k | v | g
        # q and k heads rotated where they lie; the keys carry dim^(-1/2)
        ops.head_prepare(rows, 0, 2 * H, d, inv_freq=self.position.inv_freq,
                         interleaved=bool(getattr(self.position, "interleaved", False)), positions=ctx.positions,
                         n_first=H, scale_first=1.0, scale_rest=float(d) ** -0.5)
        o = ctx.workspace.get("retention_o", (T, H * dv), torch.float32)
        chunk_tokens, max_chunks = ops.decay_scan_chunks(ctx.max_seg_len, dim=d, blocks=ctx.n_rows * H * -(-dv // 8))
        chunk_state = chunk_decay = None
        if chunk_tokens:
            n_state, n_decay = ops.decay_scan_scratch(ctx.n_rows, max_chunks, H, d, dv, chunk_tokens)
            chunk_state = ctx.workspace.get("scan_chunk_state", (n_state,), torch.float32)
            chunk_decay = ctx.workspace.get("scan_chunk_decay", (n_decay,), torch.float32)
        ops.decay_scan(rows, 0, 1, rows, H * d, 1, rows, 2 * H * d, ctx.fixed_arrays(site)["state"], ctx.seg_start,
                       ctx.seg_len, ctx.slot, o, H, d, dv, decay_const=self.decay, chunk_tokens=chunk_tokens,
                       max_chunks=max_chunks, chunk_state=chunk_state, chunk_decay=chunk_decay)
        gated = ctx.workspace.get("retention_gated", (T, H * dv), self.out.in_dtype, alias="mixer_mid")
        ops.gated_group_norm(o, rows, 2 * H * d + H * dv, None, H, self.eps, gated, gate_first=False)
        return self.out(ctx, gated, torch.float32, "mixer_out", sliced_ok=True, into=ctx.stream)


register_part("mixer", "retention", Retention)
