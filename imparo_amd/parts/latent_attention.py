"""Attention over a cached latent.

Keys and values are not projected from the layer's input directly: c =
RMSnorm(W_dkv h)[:kv_rank] is a small latent a token, the unrotated part of
head n's key is W_uk[n] c and its value W_uv[n] c; the last `rot_dim` outputs
of W_dkv, rotated by position, are one more key part that every head shares.
A head's query is [dim unrotated | rot_dim rotated] and a score is
(q_unrotated . k_unrotated + q_rotated . k_rotated) * scale. Queries come
from the input directly (`q`) or, with `q_rank`, through a normed latent of
their own (`dq`, `dq.norm`, `uq`).

Only [c | rotated key part] is cached, one row a position for all heads, and
the kernels never make a key or a value: q_unrotated . (W_uk c) =
(W_uk^T q_unrotated) . c, so a query carries W_uk^T q_unrotated next to its
rotated part and a score is one dot product with a cached row; the softmax
weights sum the cached latents, and W_uv is applied to that sum, once a query
instead of once a key.

Kernels: under a bfloat16 engine, with pages of at least 32 positions and a
latent of up to 256 numbers in steps of 8, attention runs on the matrix cores,
16 or 32 heads of one token a wave (all heads read the same rows over the same
range of keys); the cache then keeps the latents a second time, transposed
inside a page (`latent_t` [kv_rank, PAGE]), which is what the second product
reads 8 positions at a time. Otherwise one wave a (token, head) walks the rows.
Both per-head products run on the matrix cores where their inner sizes are
multiples of 8.

Parameters: width, heads, dim, rot_dim, vdim, kv_rank, q_rank (None: queries
projected directly), scale, window (a query at position i sees positions
i - window + 1 .. i; None: all before it), eps (of the latents' norms),
position (a rotation of pairs over the first `rotary_dim` of the rot_dim
part, in halves or in neighbours as the position part says), names.
"""
from __future__ import annotations

from typing import Dict, Optional

import torch

from ..cache.pages import PAGE, PagedArray, PagedSpec
from ..config.plan import PartSpec
from ..kernels import ops
from ..weights.loader import TensorDecl
from .base import Declared, StepContext
from .linear import Linear, place_matrix, place_projection, place_vector
from .registry import part_class, register_part

_DEFAULT_NAMES = dict(q="q", dq="dq", dq_norm="dq.norm", uq="uq", dkv="dkv", dkv_norm="dkv.norm", uk="uk", uv="uv", o="o")


class LatentAttention:
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
        E, H, dn, dr, dv, r = (spec["width"], spec["heads"], spec["dim"], spec["rot_dim"], spec["vdim"], spec["kv_rank"])
        qr = spec.get("q_rank")
        out: Declared = {}
        if qr:
            out[n["dq"]] = (TensorDecl((qr, E)), "matrix")
            out[n["dq_norm"]] = (TensorDecl((qr,), "vector"), "norm")
            out[n["uq"]] = (TensorDecl((H * (dn + dr), qr)), "matrix")
        else:
            out[n["q"]] = (TensorDecl((H * (dn + dr), E)), "matrix")
        out[n["dkv"]] = (TensorDecl((r + dr, E)), "matrix")
        out[n["dkv_norm"]] = (TensorDecl((r,), "vector"), "norm")
        out[n["uk"]] = (TensorDecl((H * dn, r)), "matrix")
        out[n["uv"]] = (TensorDecl((H * dv, r)), "matrix")
        out[n["o"]] = (TensorDecl((E, H * dv)), "matrix")
        return out

    def __init__(self, spec: PartSpec, tensors: Dict[str, torch.Tensor], device: torch.device,
                 engine_dtype: torch.dtype):
        n = self._names(spec)
        self.engine_dtype = engine_dtype
        self.width, self.heads, self.dim, self.rot_dim = spec["width"], spec["heads"], spec["dim"], spec["rot_dim"]
        self.vdim, self.rank = spec["vdim"], spec["kv_rank"]
        self.q_rank: Optional[int] = spec.get("q_rank") or None
        self.scale = float(spec["scale"])
        self.window: Optional[int] = spec.get("window")
        self.eps = float(spec["eps"])
        self.row_dim = self.rank + self.rot_dim
        self.tiles = False        # whether the matrix-core kernel runs (cache_spec decides, with the page size)
        if self.row_dim > ops.ATTENTION_MAX_HEAD_DIM:
            raise ValueError(f"a cached row of {self.row_dim} numbers (kv_rank + rot_dim) passes the attention "
                             f"kernel's {ops.ATTENTION_MAX_HEAD_DIM}")
        H, dn, dv, r = self.heads, self.dim, self.vdim, self.rank
        if self.q_rank:
            self.q_down = Linear(place_projection(tensors[n["dq"]], engine_dtype, device))
            self.q_norm = place_vector(tensors[n["dq_norm"]], device)
            self.q_up = Linear(place_projection(tensors[n["uq"]], engine_dtype, device))
        else:
            self.q_down, self.q_norm = None, None
            self.q_up = Linear(place_projection(tensors[n["q"]], engine_dtype, device))
        self.kv_down = Linear(place_projection(tensors[n["dkv"]], engine_dtype, device))
        self.kv_norm = place_vector(tensors[n["dkv_norm"]], device)
        # the two up-projections head by head, laid [heads, in, out] as the small product reads them:
        # W_uk[h] is [dim, rank] and maps dim -> rank as its transpose; W_uv[h] is [vdim, rank] and maps rank -> vdim
        # (the matrix-core form of that product wants them [heads, out, in], where it takes the sizes)
        uk, uv = tensors[n["uk"]].reshape(H, dn, r), tensors[n["uv"]].reshape(H, dv, r)
        self.absorb_tiles = ops.head_gemm_tiles_takes(engine_dtype, dn)
        self.values_tiles = ops.head_gemm_tiles_takes(engine_dtype, r)
        self.w_absorb = (uk.transpose(1, 2) if self.absorb_tiles else uk).to(device=device, dtype=engine_dtype).contiguous()
        self.w_values = (uv if self.values_tiles else uv.transpose(1, 2)).to(device=device, dtype=engine_dtype).contiguous()
        self.out = Linear(place_projection(tensors[n["o"]], engine_dtype, device))
        pos = spec.get("position") or PartSpec("none")
        self.position = part_class("position", pos.kind)(pos, device)
        if self.position.rotary_dim > self.rot_dim:
            raise ValueError("the rotation cannot be wider than the rotated part of a head")

    @property
    def in_dtype(self) -> torch.dtype:
        return self.kv_down.in_dtype

    def cache_spec(self, page_size: int) -> PagedSpec:
        """One row [latent | rotated key part] a position, shared by all heads."""
        self.tiles = ops.attention_latent_tiles_takes(self.engine_dtype, self.row_dim, self.rank, page_size)
        arrays = (PagedArray("latent", (PAGE, self.row_dim)),)
        if self.tiles:
            # the latents once more, transposed inside a page: the matrix-core kernel's second product reads
            # 8 positions of one number of the latent in one load
            arrays += (PagedArray("latent_t", (self.rank, PAGE)),)
        return PagedSpec(arrays, self.window)

    def forward(self, ctx: StepContext, site: int, owns_cache: bool, h: torch.Tensor) -> torch.Tensor:
        T, H = h.shape[0], self.heads
        ws = ctx.workspace
        if self.q_down is not None:
            cq_raw = self.q_down(ctx, h, torch.float32, "latent_q_down")
            cq = ws.get("latent_q_normed", (T, self.q_rank), self.q_up.in_dtype)
            ops.rms_norm(cq_raw, self.q_norm, self.eps, cq)
            q_rows = self.q_up(ctx, cq, torch.float32, "latent_q_rows", alias="mixer_in")
        else:
            q_rows = self.q_up(ctx, h, torch.float32, "latent_q_rows", alias="mixer_in")
        kv_rows = self.kv_down(ctx, h, torch.float32, "latent_kv_rows")
        arrays, table = ctx.paged(site)
        cache = arrays["latent"]
        q_plain = ws.get("latent_q_plain", (T, H, self.dim), ctx.dtype)
        q_full = ws.get("latent_q_full", (T, H, self.row_dim), ctx.dtype)
        ops.latent_store(q_rows, kv_rows, self.kv_norm, self.eps, self.position.inv_freq,
                         bool(getattr(self.position, "interleaved", False)), ctx.positions, ctx.row_of_token,
                         table if owns_cache else None, ctx.page_size, cache if owns_cache else None,
                         q_plain, q_full, H, self.dim, self.rot_dim, self.rank,
                         cache_t=arrays["latent_t"] if self.tiles and owns_cache else None)
        # columns 0 .. rank of every head's query
        (ops.head_gemm_tiles if self.absorb_tiles else ops.head_gemm)(q_plain, self.w_absorb, q_full)
        mixed = ws.get("latent_mixed", (T, H * self.rank), ctx.dtype, alias="mixer_mid")
        if self.tiles:
            n_splits, split_keys = ops.attention_latent_tiles_split(T, H, ctx.max_context)
            part_o = part_ml = None
            if n_splits > 1:
                part_o = ws.get("latent_part_o", (T * H * n_splits * self.rank,), torch.float32)
                part_ml = ws.get("latent_part_ml", (T * H * n_splits * 2,), torch.float32)
            ops.attention_latent_tiles(q_full, cache, arrays["latent_t"], mixed, ctx.positions, ctx.row_of_token, table,
                                       self.scale, self.window, n_splits, split_keys, part_o, part_ml)
        else:
            ops.attention_latent(q_full, cache, mixed, ctx.positions, ctx.row_of_token, table, self.rank, self.scale,
                                 self.window)
        o = ws.get("latent_values", (T, H, self.vdim), self.out.in_dtype)
        (ops.head_gemm_tiles if self.values_tiles else ops.head_gemm)(mixed.view(T, H, self.rank), self.w_values, o)
        return self.out(ctx, o.view(T, H * self.vdim), torch.float32, "mixer_out", sliced_ok=True)


register_part("mixer", "latent_attention", LatentAttention)
