"""What a parallel block multiplies a sublayer's result by and what it adds behind both sublayers.

`sigmoid_gate` (role "gate"): a sublayer's result is multiplied element by
element by sigmoid(W h + b), h being the sublayer's own input. The part holds
W and b; the block that owns it runs the gates of its sublayers as one
projection.

`token_side` (role "side"): a per-layer input from the token itself. With e
the layer's `dim` columns of a second embedding table, taken at the token,
g = gelu_tanh(W_gate x) * e, y = W_proj g, and x += y / rms(y) * w: the
part returns y and the norm it goes through, and whoever reads the stream next
applies that norm and adds, in the launch of its own norm.
"""
from __future__ import annotations

from typing import Dict

import torch

from ..config.plan import PartSpec
from ..kernels import ops
from ..weights.loader import TensorDecl
from .base import Declared, StepContext
from .linear import Linear, place_matrix, place_projection, place_vector
from .registry import register_part


class SigmoidGate:
    role = "gate"
    graph_safe = True

    @classmethod
    def declare(cls, spec: PartSpec) -> Declared:
        E = spec["width"]
        return {spec["weight"]: (TensorDecl((E, E)), "matrix"), spec["bias"]: (TensorDecl((E,), "vector"), "bias")}

    def __init__(self, spec: PartSpec, tensors: Dict[str, torch.Tensor], device: torch.device,
                 engine_dtype: torch.dtype):
        self.width = spec["width"]
        self.weight = place_projection(tensors[spec["weight"]], engine_dtype, device)
        self.bias = place_vector(tensors[spec["bias"]], device)

    @staticmethod
    def together(gates) -> Linear:
        """The gates of a block's sublayers as one projection: their outputs side by side."""
        weights = [g.weight for g in gates]
        if len({w.dtype for w in weights}) > 1:
            weights = [w.to(torch.float32) for w in weights]
        return Linear(torch.cat(weights, dim=0), torch.cat([g.bias for g in gates]))


class TokenSide:
    role = "side"
    graph_safe = True

    @classmethod
    def declare(cls, spec: PartSpec) -> Declared:
        E, d = spec["width"], spec["dim"]
        p = spec.prefix
        return {
            spec["table"]: (TensorDecl((spec["vocab"], spec["table_width"])), "matrix"),
            f"{p}.gate": (TensorDecl((d, E)), "matrix"),
            f"{p}.proj": (TensorDecl((E, d)), "matrix"),
            f"{p}.norm": (TensorDecl((E,), "vector"), "norm"),
        }

    def __init__(self, spec: PartSpec, tensors: Dict[str, torch.Tensor], device: torch.device,
                 engine_dtype: torch.dtype):
        p = spec.prefix
        self.width, self.dim, self.eps = spec["width"], spec["dim"], float(spec["eps"])
        offset = int(spec.get("offset", 0))
        # the layer keeps its own columns of the table only
        self.table = place_matrix(tensors[spec["table"]][:, offset:offset + self.dim].contiguous(), engine_dtype, device)
        self.gate = Linear(place_projection(tensors[f"{p}.gate"], engine_dtype, device))
        proj = tensors[f"{p}.proj"]
        # the bfloat16 products walk their inner size in steps of 8: a narrower side input is filled up with
        # columns of zero weight, and the gated rows end in as many zeros
        fill = (-self.dim) % 8 if engine_dtype != torch.float32 and proj.dtype != torch.float32 else 0
        if fill:
            proj = torch.cat([proj, proj.new_zeros(proj.shape[0], fill)], dim=1)
        self.proj = Linear(place_matrix(proj, engine_dtype, device))
        self.norm = place_vector(tensors[f"{p}.norm"], device)

    @property
    def in_dtype(self) -> torch.dtype:
        """The dtype in which this part reads the stream."""
        return self.gate.in_dtype

    def as_post(self):
        return self.norm, self.eps

    def forward(self, ctx: StepContext, x: torch.Tensor) -> torch.Tensor:
        """`x`: the stream in `in_dtype`. Returns y float32 [tokens, width], to go through `as_post()` and be added."""
        if ctx.token_ids is None:
            raise ValueError("a per-layer token input needs the step's token ids")
        T = x.shape[0]
        z = self.gate(ctx, x, torch.float32, "side_gate")
        g = ctx.workspace.get("side_gated", (T, self.proj.in_features), self.proj.in_dtype)
        ops.side_gate(z, self.table, 0, ctx.token_ids, g)
        return self.proj(ctx, g, torch.float32, "side_out")


register_part("gate", "sigmoid_gate", SigmoidGate)
register_part("side", "token_side", TokenSide)
