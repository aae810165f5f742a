"""The gated delta rule: a recurrence that corrects what its state predicts.

q = Wq h and k = Wk h are [kv_heads, dim], v = Wv h is [heads, vdim]; head h
reads q and k of head h // (heads / kv_heads). Each of q, k, v goes through a
causal convolution per channel (`taps` wide, no bias, the last tap the current
token's, zeros before the start) and SiLU; q and k are then made unit vectors
per head, x / sqrt(sum x^2 + 1e-6), and q is multiplied by dim^(-1/2).
b = sigmoid(Wb h) and the decay g = exp(-exp(A_log) softplus(Wa h + dt_bias))
are one number a head. Per head, with a state S [dim, vdim]:

    S <- g S;   u = b (v - S^T k);   S <- S + k u^T;   o = S^T q

(in that order: a token's result already holds what the token wrote). Each head's o is divided by its
root mean square, multiplied by a weight that all heads share and by
silu(Wg h); the heads side by side go through the output projection. A
request's state is S, float32, and the convs' last taps - 1 inputs. Gates,
decays, unit vectors, the state and every sum of the recurrence are float32
whatever the engine's dtype.

Parameters: width, heads, kv_heads, dim, vdim, taps, eps, names.
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

_DEFAULT_NAMES = dict(q="q", k="k", v="v", q_conv="q.conv", k_conv="k.conv", v_conv="v.conv", b="b", a="a",
                      A_log="A_log", dt_bias="dt_bias", g="g", norm="norm", o="o")
UNIT_EPS = 1e-6          # inside the root that makes q and k unit vectors


class GatedDelta:
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
        E, H, Hk, dk, dv, L = spec["width"], spec["heads"], spec["kv_heads"], spec["dim"], spec["vdim"], spec["taps"]
        return {
            n["q"]: (TensorDecl((Hk * dk, E)), "matrix"),
            n["k"]: (TensorDecl((Hk * dk, E)), "matrix"),
            n["v"]: (TensorDecl((H * dv, E)), "matrix"),
            n["q_conv"]: (TensorDecl((Hk * dk, L), "vector"), "conv"),
            n["k_conv"]: (TensorDecl((Hk * dk, L), "vector"), "conv"),
            n["v_conv"]: (TensorDecl((H * dv, L), "vector"), "conv"),
            n["b"]: (TensorDecl((H, E)), "matrix"),
            n["a"]: (TensorDecl((H, E)), "matrix"),
            n["A_log"]: (TensorDecl((H,), "vector"), "wide"),
            n["dt_bias"]: (TensorDecl((H,), "vector"), "bias"),
            n["g"]: (TensorDecl((H * dv, E)), "matrix"),
            n["norm"]: (TensorDecl((dv,), "vector"), "norm"),
            n["o"]: (TensorDecl((E, H * dv)), "matrix"),
        }

    def __init__(self, spec: PartSpec, tensors: Dict[str, torch.Tensor], device: torch.device,
                 engine_dtype: torch.dtype):
        n = self._names(spec)
        self.width, self.heads, self.kv_heads = spec["width"], spec["heads"], spec["kv_heads"]
        self.dim, self.vdim, self.taps = spec["dim"], spec["vdim"], spec["taps"]
        self.eps = float(spec["eps"])
        if self.heads % self.kv_heads:
            raise ValueError(f"{self.heads} heads cannot share {self.kv_heads} query/key heads evenly")
        if not 1 <= self.taps <= 64:
            raise ValueError(f"the conv kernels take 1 to 64 taps, got {self.taps}")
        if self.dim > ops.DECAY_SCAN_MAX_DIM:
            raise ValueError(f"the recurrence kernel takes up to {ops.DECAY_SCAN_MAX_DIM} state rows a head, got {self.dim}")
        H, Hk, dk, dv = self.heads, self.kv_heads, self.dim, self.vdim
        self.conv_channels = 2 * Hk * dk + H * dv
        ws = [tensors[n[x]] for x in ("q", "k", "v", "b", "a", "g")]
        if len({w.dtype for w in ws}) > 1:
            ws = [w.to(torch.float32) for w in ws]
        # one projection for q | k | v | b | a | g: the same dot products, one launch
        self.proj = Linear(place_projection(torch.cat(ws, dim=0), engine_dtype, device))
        self.conv_weight = place_vector(torch.cat([tensors[n[x]].to(torch.float32).reshape(-1, self.taps)
                                                   for x in ("q_conv", "k_conv", "v_conv")], dim=0), device)
        self.dt_bias = place_vector(tensors[n["dt_bias"]], device)
        self.rate = place_vector(torch.exp(tensors[n["A_log"]].to(torch.float32)), device)
        self.norm = place_vector(tensors[n["norm"]].to(torch.float32).repeat(H), device)
        self.out = Linear(place_projection(tensors[n["o"]], engine_dtype, device))

    @property
    def in_dtype(self) -> torch.dtype:
        return self.proj.in_dtype

    def cache_spec(self, page_size: int) -> FixedSpec:
        arrays = (FixedArray("state", (self.heads, self.dim, self.vdim), "float32", 0.0),)
        if self.taps > 1:
            arrays += (FixedArray("conv", (self.taps - 1, self.conv_channels), "float32", 0.0),)
        return FixedSpec(arrays=arrays)

    def forward(self, ctx: StepContext, site: int, owns_cache: bool, h: torch.Tensor) -> torch.Tensor:
        if not owns_cache:
            raise ValueError("a recurrence's state cannot be read from another layer")
        T, H, Hk, dk, dv, C = h.shape[0], self.heads, self.kv_heads, self.dim, self.vdim, self.conv_channels
        state = ctx.fixed_arrays(site)
        rows = self.proj(ctx, h, torch.float32, "delta_rows", alias="mixer_in")     # q k v | b | a | g
        qkv = ctx.workspace.get("delta_qkv", (T, C), torch.float32)
        ops.causal_conv(rows, C, self.conv_weight, None, state.get("conv"), ctx.row_of_token, ctx.seg_start,
                        ctx.seg_len, ctx.slot, qkv, silu=True, single_tokens=ctx.max_seg_len == 1)
        # q and k heads as unit vectors; the queries carry dim^(-1/2)
        ops.head_prepare(qkv, 0, 2 * Hk, dk, unit=True, unit_eps=UNIT_EPS, n_first=Hk, scale_first=float(dk) ** -0.5)
        o = ctx.workspace.get("delta_o", (T, H * dv), torch.float32)
        # a long portion: the rule in chunks (a triangle solved a chunk, side by side; then the chunks in order)
        chunk_tokens, max_chunks = ops.decay_scan_chunks(ctx.max_seg_len, delta=True, dim=dk)
        chunk_state = chunk_decay = None
        if chunk_tokens:
            n_state, n_decay = ops.decay_scan_scratch(ctx.n_rows, max_chunks, H, dk, dv, chunk_tokens)
            chunk_state = ctx.workspace.get("scan_chunk_state", (n_state,), torch.float32)
            chunk_decay = ctx.workspace.get("scan_chunk_decay", (n_decay,), torch.float32)
        ops.decay_scan(qkv, 0, H // Hk, qkv, Hk * dk, H // Hk, qkv, 2 * Hk * dk, state["state"], ctx.seg_start,
                       ctx.seg_len, ctx.slot, o, H, dk, dv, step=rows, step_off=C + H, step_bias=self.dt_bias,
                       rate=self.rate, beta=rows, beta_off=C, chunk_tokens=chunk_tokens, max_chunks=max_chunks,
                       chunk_state=chunk_state, chunk_decay=chunk_decay)
        gated = ctx.workspace.get("delta_gated", (T, H * dv), self.out.in_dtype, alias="mixer_mid")
        ops.gated_group_norm(o, rows, C + 2 * H, self.norm, H, self.eps, gated, gate_first=False)
        return self.out(ctx, gated, torch.float32, "mixer_out", sliced_ok=True, into=ctx.stream)


register_part("mixer", "gated_delta", GatedDelta)
