"""Token embedding (a row gather; `scale` multiplies the row in float32, 1 in the reference:
/root/reference/crates/imparo-model/src/cpu_support.rs:327-342) and the output
head (logits = W h for the rows that want logits, no bias, no softcap:
/root/reference/crates/imparo-model/src/cpu_support.rs:451-466).

`tensor` names the table outright where a checkpoint does not call it
`<prefix>.weight`. The sinusoidal embedding adds a position vector to the
gathered row: entry 2i is sin(p * base^(-2i/width)), entry 2i+1 the cosine of
the same angle, angles in float32. `norm` (the spec of a norm part) norms the
gathered rows before they become the stream."""
from __future__ import annotations

from typing import Dict

import numpy as np
import torch

from ..config.plan import PartSpec
from ..kernels import ops
from ..weights.loader import TensorDecl
from .base import Declared, StepContext
from .linear import Linear, place_matrix, place_projection
from .registry import part_class, register_part


def _table_name(spec: PartSpec) -> str:
    return spec.get("tensor") or f"{spec.prefix}.weight"


class Embedding:
    role = "embedding"
    graph_safe = True     # launches kernels only: a step made of such parts can be captured

    @staticmethod
    def declare(spec: PartSpec) -> Declared:
        out = {_table_name(spec): (TensorDecl((spec["vocab"], spec["width"])), "matrix")}
        norm = spec.get("norm")
        if norm is not None:
            out.update(part_class("norm", norm.kind).declare(norm))
        return out

    def __init__(self, spec: PartSpec, tensors: Dict[str, torch.Tensor], device: torch.device,
                 engine_dtype: torch.dtype, placed: Dict[str, torch.Tensor]):
        name = _table_name(spec)
        if name not in placed:     # a tied head shares this very tensor
            placed[name] = place_matrix(tensors[name], engine_dtype, device)
        self.table = placed[name]
        self.vocab, self.width = spec["vocab"], spec["width"]
        self.scale = float(spec.get("scale", 1.0))
        norm = spec.get("norm")
        self.norm = None if norm is None else part_class("norm", norm.kind)(norm, tensors, device, engine_dtype)
        if self.norm is not None and getattr(self.norm, "groups", 1) != 1:
            raise ValueError("the norm on the embedding's rows does not cut them into groups")

    def forward(self, ctx: StepContext, token_ids: torch.Tensor, name: str = "residual") -> torch.Tensor:
        """The rows of the stream, float32, in the workspace buffer `name` (a caller that needs the
        embedding's output twice, once to keep, asks twice: the same launches, the same bits)."""
        x = ctx.workspace.get(name, (token_ids.shape[0], self.width), torch.float32)
        if self.norm is None:
            return ops.embed_gather(self.table, token_ids, x, self.scale)
        raw = ctx.workspace.get("embedding_rows", (token_ids.shape[0], self.width), torch.float32)
        ops.embed_gather(self.table, token_ids, raw, self.scale)
        return ops.rms_norm(raw, self.norm.weight, self.norm.eps, x)

    def can_emit(self) -> bool:
        return self.scale == 1.0 and self.norm is None     # the step program's gather has neither

    def emit(self, program) -> None:
        """Appends `forward` to a native step program."""
        program.embedding(self.table, self.vocab, self.width)


class SinusoidEmbedding(Embedding):
    """The table's row plus the sinusoidal vector of the token's position."""

    def __init__(self, spec: PartSpec, tensors: Dict[str, torch.Tensor], device: torch.device,
                 engine_dtype: torch.dtype, placed: Dict[str, torch.Tensor]):
        super().__init__(spec, tensors, device, engine_dtype, placed)
        base = float(spec.get("base") or 10000.0)
        i = np.arange((self.width + 1) // 2, dtype=np.float32)
        expo = (np.float32(-2.0) * i / np.float32(self.width)).astype(np.float32)
        self.inv_freq = torch.from_numpy(np.power(np.float32(base), expo).astype(np.float32)).to(device)

    def forward(self, ctx: StepContext, token_ids: torch.Tensor) -> torch.Tensor:
        x = ctx.workspace.get("residual", (token_ids.shape[0], self.width), torch.float32)
        return ops.embed_sinusoid(self.table, token_ids, ctx.positions, self.inv_freq, x)


class LinearHead:
    role = "head"
    graph_safe = True     # launches kernels only: a step made of such parts can be captured

    @staticmethod
    def declare(spec: PartSpec) -> Declared:
        return {_table_name(spec): (TensorDecl((spec["vocab"], spec["width"])), "matrix")}

    def __init__(self, spec: PartSpec, tensors: Dict[str, torch.Tensor], device: torch.device,
                 engine_dtype: torch.dtype, placed: Dict[str, torch.Tensor]):
        name = _table_name(spec)
        if name not in placed:
            placed[name] = place_projection(tensors[name], engine_dtype, device)
        self.proj = Linear(placed[name])
        self.vocab = spec["vocab"]

    @property
    def in_dtype(self) -> torch.dtype:
        return self.proj.in_dtype

    def forward(self, ctx: StepContext, h: torch.Tensor) -> torch.Tensor:
        return self.proj(ctx, h, torch.float32, "logits")

    def emit_projection(self) -> Linear:
        """What `forward` computes, for a native step program: this projection, float32 out."""
        return self.proj


register_part("embedding", "embedding", Embedding)
register_part("embedding", "sinusoid_embedding", SinusoidEmbedding)
register_part("head", "linear_head", LinearHead)
