"""A gated linear recurrence with a matrix of state a head (HGRN2).

q = silu(W_q h) and the forget gate f = lower + (1 - lower) sigmoid(W_f h + b)
are [heads, dim], v = W_v h is [heads, vdim]. Per head the state S [dim, vdim]
moves as S <- diag(f) S + (1 - f) v^T (what the gate forgets is what it lets
in: there is no key), and the head's result is S^T q. Each head's result is
divided by its root mean square over vdim and multiplied by a weight that all
heads share; the heads side by side go through the output projection. The
state is float32, starts at zero and is carried from token to token per
request; gates and sums of the recurrence are float32 whatever the engine's
dtype.

Parameters: width, heads, dim, vdim, eps (of the head norm), names.
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
from .registry import register_part

_DEFAULT_NAMES = dict(q="q", f="f", f_bias="f.b", lower="lower", v="v", norm="norm", o="o")


class Hgrn2:
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
        E, H, dk, dv = spec["width"], spec["heads"], spec["dim"], spec["vdim"]
        return {
            n["q"]: (TensorDecl((H * dk, E)), "matrix"),
            n["f"]: (TensorDecl((H * dk, E)), "matrix"),
            n["f_bias"]: (TensorDecl((H * dk,), "vector"), "bias"),
            n["lower"]: (TensorDecl((H * dk,), "vector"), "unit"),
            n["v"]: (TensorDecl((H * dv, E)), "matrix"),
            n["norm"]: (TensorDecl((dv,), "vector"), "norm"),
            n["o"]: (TensorDecl((E, H * dv)), "matrix"),
        }

    def __init__(self, spec: PartSpec, tensors: Dict[str, torch.Tensor], device: torch.device,
                 engine_dtype: torch.dtype):
        n = self._names(spec)
        self.width, self.heads, self.dim, self.vdim = spec["width"], spec["heads"], spec["dim"], spec["vdim"]
        self.eps = float(spec["eps"])
        if self.dim > ops.HGRN2_MAX_DIM:
            raise ValueError(f"the recurrence kernel takes up to {ops.HGRN2_MAX_DIM} state rows a head, got {self.dim}")
        H, dk, dv = self.heads, self.dim, self.vdim
        ws = [tensors[n[x]] for x in ("q", "f", "v")]
        if len({w.dtype for w in ws}) > 1:
            ws = [w.to(torch.float32) for w in ws]
        # one projection for zq | zf | v: the same dot products, one launch; the gate's bias rides in it
        bias = torch.cat([torch.zeros(H * dk), tensors[n["f_bias"]].to(torch.float32).cpu(), torch.zeros(H * dv)])
        self.proj = Linear(place_projection(torch.cat(ws, dim=0), engine_dtype, device), place_vector(bias, device))
        self.lower = place_vector(tensors[n["lower"]], device)
        self.norm = place_vector(tensors[n["norm"]].to(torch.float32).repeat(H), device)
        self.out = Linear(place_projection(tensors[n["o"]], engine_dtype, device))

    @property
    def in_dtype(self) -> torch.dtype:
        return self.proj.in_dtype

    def cache_spec(self, page_size: int) -> FixedSpec:
        return FixedSpec(arrays=(FixedArray("state", (self.heads, self.dim, self.vdim), "float32", 0.0),))

    def forward(self, ctx: StepContext, site: int, owns_cache: bool, h: torch.Tensor) -> torch.Tensor:
        if not owns_cache:
            raise ValueError("a recurrence's state cannot be read from another layer")
        T, H, dk, dv = h.shape[0], self.heads, self.dim, self.vdim
        rows = self.proj(ctx, h, torch.float32, "hgrn2_rows", alias="mixer_in")
        o = ctx.workspace.get("hgrn2_out", (T, H * dv), torch.float32)
        chunk_tokens, max_chunks = ops.hgrn2_chunks(ctx.max_seg_len)
        chunk_state = chunk_decay = None
        if chunk_tokens:
            # a long portion: its chunks side by side, each from the state that a pass over the chunks' ends leaves it
            chunk_state = ctx.workspace.get("hgrn2_chunk_state", (ctx.seg_start.shape[0] * max_chunks * H * dk * dv,), torch.float32)
            chunk_decay = ctx.workspace.get("hgrn2_chunk_decay", (ctx.seg_start.shape[0] * max_chunks * H * dk,), torch.float32)
        ops.hgrn2_scan(rows, 0, H * dk, 2 * H * dk, self.lower, ctx.fixed_arrays(site)["state"], ctx.seg_start,
                       ctx.seg_len, ctx.slot, o, H, dk, dv, chunk_tokens, max_chunks, chunk_state, chunk_decay)
        normed = ctx.workspace.get("hgrn2_normed", (T, H * dv), self.out.in_dtype, alias="mixer_mid")
        ops.group_rms_norm(o, self.norm, H, self.eps, normed)
        return self.out(ctx, normed, torch.float32, "mixer_out", sliced_ok=True)


register_part("mixer", "hgrn2", Hgrn2)
