"""Dense SwiGLU feed-forward: f = W2 ( silu(W1 n) * (W3 n) ), SiLU on the gate
(/root/reference/crates/imparo-model/src/lfm2/workflow_cpu.rs:298-316).

PolyNorm feed-forward: f = Wdown act(Wup n) with act(z) = a N(z) + b N(z^2) +
c N(z^3) + e, powers taken element by element and N dividing a token's vector
of hidden values by its root mean square (in float32); a, b, c, e are four
numbers of the layer."""
from __future__ import annotations

from typing import Dict

import torch

from ..config.plan import PartSpec
from ..kernels import ops
from ..weights.loader import TensorDecl
from .base import Declared, StepContext
from .linear import Linear, place_matrix, place_projection, place_vector
from .registry import register_part

_DEFAULT_NAMES = dict(gate="gate_proj", up="up_proj", down="down_proj")


class SwiGlu:
    role = "feed_forward"
    graph_safe = True     # launches kernels only: a step made of such parts can be captured

    @staticmethod
    def _names(spec: PartSpec) -> Dict[str, str]:
        names = dict(_DEFAULT_NAMES)
        names.update(spec.get("names") or {})
        return {k: f"{spec.prefix}.{v}" for k, v in names.items()}

    @classmethod
    def declare(cls, spec: PartSpec) -> Declared:
        n = cls._names(spec)
        sfx = spec.get("weight_suffix", ".weight")
        E, F = spec["width"], spec["hidden"]
        return {
            n["gate"] + sfx: (TensorDecl((F, E)), "matrix"),
            n["up"] + sfx: (TensorDecl((F, E)), "matrix"),
            n["down"] + sfx: (TensorDecl((E, F)), "matrix"),
        }

    def __init__(self, spec: PartSpec, tensors: Dict[str, torch.Tensor], device: torch.device,
                 engine_dtype: torch.dtype):
        n = self._names(spec)
        sfx = spec.get("weight_suffix", ".weight")          # what a checkpoint appends to a matrix's name
        self.width, self.hidden = spec["width"], spec["hidden"]
        # a second feed-forward inside another part keeps its scratch under names of its own
        self.tag = spec.get("scratch_tag") or ""
        gate, up = tensors[n["gate"] + sfx], tensors[n["up"] + sfx]
        if gate.dtype != up.dtype:
            gate, up = gate.to(torch.float32), up.to(torch.float32)
        down = tensors[n["down"] + sfx]
        # The bfloat16 kernels walk K in steps of 8. A hidden width that is no multiple of 8 is
        # filled up with hidden units whose weights are zero: silu(0) * 0 = 0 goes through zero
        # columns of the way back, so every sum is the one it was.
        fill = (-self.hidden) % 8
        if fill and engine_dtype != torch.float32 and down.dtype != torch.float32:
            gate = torch.cat([gate, gate.new_zeros(fill, self.width)])
            up = torch.cat([up, up.new_zeros(fill, self.width)])
            down = torch.cat([down, down.new_zeros(self.width, fill)], dim=1)
        # gate and up as one projection with alternating rows (g0, u0, g1, u1, ...): the same dot
        # products, one launch, and the GEMM's epilogue applies silu(gate) * up before it stores
        fused = torch.stack([gate, up], dim=1).reshape(2 * gate.shape[0], self.width)
        self.gate_up = Linear(place_projection(fused, engine_dtype, device))
        self.down = Linear(place_matrix(down, engine_dtype, device))

    @property
    def in_dtype(self) -> torch.dtype:
        return self.gate_up.in_dtype

    def forward(self, ctx: StepContext, n: torch.Tensor) -> torch.Tensor:
        # the gated hidden may lie where the mixer's input projection lay: that is dead by now
        g = self.gate_up(ctx, n, self.down.in_dtype, self.tag + "gated", swiglu=True, alias="mixer_in")
        # the result is a delta for the residual stream, whose next norm adds slices: it may come sliced
        return self.down(ctx, g, torch.float32, self.tag + "ffn_out", sliced_ok=True, into=ctx.stream)


    def can_emit(self) -> bool:
        return not self.tag

    def emit(self, program) -> None:
        """Appends `forward` to a native step program."""
        from ..kernels.program import SwigluDesc
        program.swiglu(SwigluDesc(program.linear(self.gate_up), program.linear(self.down)))


class PolyNormFfn:
    role = "feed_forward"
    graph_safe = True     # launches kernels only: a step made of such parts can be captured

    @staticmethod
    def _names(spec: PartSpec) -> Dict[str, str]:
        names = dict(up="up", down="down", act="act")
        names.update(spec.get("names") or {})
        return {k: f"{spec.prefix}.{v}" for k, v in names.items()}

    @classmethod
    def declare(cls, spec: PartSpec) -> Declared:
        n = cls._names(spec)
        E, F = spec["width"], spec["hidden"]
        return {
            n["up"]: (TensorDecl((F, E)), "matrix"),
            n["down"]: (TensorDecl((E, F)), "matrix"),
            n["act"]: (TensorDecl((4,), "vector"), "wide"),
        }

    def __init__(self, spec: PartSpec, tensors: Dict[str, torch.Tensor], device: torch.device,
                 engine_dtype: torch.dtype):
        n = self._names(spec)
        self.width, self.hidden = spec["width"], spec["hidden"]
        self.eps = float(spec["eps"])
        up, down = tensors[n["up"]], tensors[n["down"]]
        # a hidden width that is no multiple of 8 is filled up with units of zero weight on the way back
        # (the bfloat16 kernels walk K in steps of 8); the norms divide by the true width
        fill = (-self.hidden) % 8
        if fill and engine_dtype != torch.float32 and down.dtype != torch.float32:
            up = torch.cat([up, up.new_zeros(fill, self.width)])
            down = torch.cat([down, down.new_zeros(self.width, fill)], dim=1)
        self.up = Linear(place_projection(up, engine_dtype, device))
        self.down = Linear(place_matrix(down, engine_dtype, device))
        self.coef = place_vector(tensors[n["act"]], device)

    @property
    def in_dtype(self) -> torch.dtype:
        return self.up.in_dtype

    def forward(self, ctx: StepContext, n: torch.Tensor) -> torch.Tensor:
        z = self.up(ctx, n, torch.float32, "ffn_hidden", alias="mixer_in")
        g = ctx.workspace.get("ffn_act", tuple(z.shape), self.down.in_dtype, alias="mixer_mid")
        ops.poly_norm(z, self.coef, self.eps, g, width=self.hidden)
        return self.down(ctx, g, torch.float32, "ffn_out", sliced_ok=True, into=ctx.stream)


class ClampedGlu:
    """A gated unit with bounds: g = min(Wgate n, limit), u = clamp(Wup n, -limit, limit),
    f = Wdown (g sigmoid(alpha g) (u + 1)). Parameters: width, hidden, limit, alpha (1.702 unless
    given), names, weight_suffix."""
    role = "feed_forward"
    graph_safe = True     # launches kernels only: a step made of such parts can be captured
    _names = staticmethod(SwiGlu._names)

    @classmethod
    def declare(cls, spec: PartSpec) -> Declared:
        return SwiGlu.declare.__func__(cls, spec)

    def __init__(self, spec: PartSpec, tensors: Dict[str, torch.Tensor], device: torch.device,
                 engine_dtype: torch.dtype):
        n = self._names(spec)
        sfx = spec.get("weight_suffix", ".weight")
        self.width, self.hidden = spec["width"], spec["hidden"]
        self.limit = float(spec["limit"])
        self.alpha = float(spec.get("alpha", 1.702))
        if not self.limit > 0:
            raise ValueError(f"the bound of a clamped unit is positive, got {self.limit}")
        gate, up, down = tensors[n["gate"] + sfx], tensors[n["up"] + sfx], tensors[n["down"] + sfx]
        if gate.dtype != up.dtype:
            gate, up = gate.to(torch.float32), up.to(torch.float32)
        # one projection for gate | up (gate rows first); the activation reads both halves of its float32 rows.
        # The bfloat16 kernels walk K in steps of 8: a hidden width that is none gets columns of zero weight on the
        # way back, and the activation fills the hidden rows up with zeros.
        self.fill = (-self.hidden) % 8 if engine_dtype != torch.float32 and down.dtype != torch.float32 else 0
        if self.fill:
            down = torch.cat([down, down.new_zeros(self.width, self.fill)], dim=1)
        self.gate_up = Linear(place_projection(torch.cat([gate, up], dim=0), engine_dtype, device))
        self.down = Linear(place_matrix(down, engine_dtype, device))

    @property
    def in_dtype(self) -> torch.dtype:
        return self.gate_up.in_dtype

    def forward(self, ctx: StepContext, n: torch.Tensor) -> torch.Tensor:
        gu = self.gate_up(ctx, n, torch.float32, "gate_up", alias="mixer_in")
        g = ctx.workspace.get("gated", (n.shape[0], self.hidden + self.fill), self.down.in_dtype, alias="mixer_mid")
        ops.clamped_glu(gu, g, self.hidden, self.limit, self.alpha)
        return self.down(ctx, g, torch.float32, "ffn_out", sliced_ok=True, into=ctx.stream)


register_part("feed_forward", "swiglu", SwiGlu)
register_part("feed_forward", "clamped_glu", ClampedGlu)
register_part("feed_forward", "poly_norm", PolyNormFfn)
