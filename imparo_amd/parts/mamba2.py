"""A state-space mixer with one decay a head (Mamba-2, state-space duality).

[z | x | B | C | dt] = Win h with inner = heads * vdim, B and C of groups *
state each and one dt a head. x, B and C together go through a causal
convolution per channel (`taps` wide, the last tap the current token's, zeros
before the start, with a bias) and SiLU. dt = softplus(dt + dt_bias), no bound.
Per head h, whose B and C are those of group h // (heads / groups), with a
state S [state, vdim]:

    S <- exp(-exp(A_log_h) dt) S + dt B x_h^T,    y_h = S^T C + D_h x_h.

The heads side by side are multiplied by silu(z), divided by their root mean
square in `norm_groups` equal parts of the row, multiplied by a weight, and go
through the output projection. A request's state is S, float32, and the conv's
last taps - 1 inputs. Steps, decays, exponentials, the state and every sum of
the recurrence are float32 whatever the engine's dtype.

Parameters: width, heads, vdim, state, groups, taps, norm_groups, eps, names.
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

_DEFAULT_NAMES = {"in": "in", "conv": "conv", "conv_bias": "conv.b", "dt_bias": "dt_bias", "A_log": "A_log",
                  "D": "D", "norm": "norm", "o": "o"}


class Mamba2:
    role = "mixer"
    graph_safe = True     # launches kernels only: a step made of such parts can be captured

    @staticmethod
    def _names(spec: PartSpec) -> Dict[str, str]:
        names = dict(_DEFAULT_NAMES)
        names.update(spec.get("names") or {})
        return {k: f"{spec.prefix}.{v}" for k, v in names.items()}

    @staticmethod
    def _sizes(spec: PartSpec):
        H, P, N, G = spec["heads"], spec["vdim"], spec["state"], int(spec.get("groups") or 1)
        return H, P, N, G, H * P, H * P + 2 * G * N

    @classmethod
    def declare(cls, spec: PartSpec) -> Declared:
        n = cls._names(spec)
        E, L = spec["width"], spec["taps"]
        H, P, N, G, inner, conv = cls._sizes(spec)
        return {
            n["in"]: (TensorDecl((inner + conv + H, E)), "matrix"),
            n["conv"]: (TensorDecl((conv, L), "vector"), "conv"),
            n["conv_bias"]: (TensorDecl((conv,), "vector"), "bias"),
            n["dt_bias"]: (TensorDecl((H,), "vector"), "bias"),
            n["A_log"]: (TensorDecl((H,), "vector"), "wide"),
            n["D"]: (TensorDecl((H,), "vector"), "norm"),
            n["norm"]: (TensorDecl((inner,), "vector"), "norm"),
            n["o"]: (TensorDecl((E, inner)), "matrix"),
        }

    def __init__(self, spec: PartSpec, tensors: Dict[str, torch.Tensor], device: torch.device,
                 engine_dtype: torch.dtype):
        n = self._names(spec)
        self.width, self.taps = spec["width"], spec["taps"]
        self.heads, self.vdim, self.n_state, self.groups, self.inner, self.conv_channels = self._sizes(spec)
        self.norm_groups = int(spec.get("norm_groups") or 1)
        self.eps = float(spec["eps"])
        if self.heads % self.groups:
            raise ValueError(f"{self.heads} heads cannot share {self.groups} groups of B and C evenly")
        if self.inner % self.norm_groups:
            raise ValueError(f"a row of {self.inner} values cannot be normed in {self.norm_groups} equal parts")
        if not 1 <= self.taps <= 64:
            raise ValueError(f"the conv kernels take 1 to 64 taps, got {self.taps}")
        if self.n_state > ops.DECAY_SCAN_MAX_DIM:
            raise ValueError(f"the recurrence kernel takes up to {ops.DECAY_SCAN_MAX_DIM} state rows a head, got {self.n_state}")
        self.in_proj = Linear(place_projection(tensors[n["in"]], engine_dtype, device))
        out = tensors[n["o"]]
        # the bfloat16 products walk K in steps of 8: an inner size that is none runs its way back in float32
        self.out_proj = Linear(place_projection(out, engine_dtype, device))
        self.conv_weight = place_vector(tensors[n["conv"]].reshape(self.conv_channels, self.taps), device)
        self.conv_bias = place_vector(tensors[n["conv_bias"]], device)
        self.dt_bias = place_vector(tensors[n["dt_bias"]], device)
        self.rate = place_vector(torch.exp(tensors[n["A_log"]].to(torch.float32)), device)
        self.D = place_vector(tensors[n["D"]], device)
        self.norm = place_vector(tensors[n["norm"]], device)

    @property
    def in_dtype(self) -> torch.dtype:
        return self.in_proj.in_dtype

    def cache_spec(self, page_size: int) -> FixedSpec:
        arrays = (FixedArray("state", (self.heads, self.n_state, self.vdim), "float32", 0.0),)
        if self.taps > 1:
            arrays += (FixedArray("conv", (self.taps - 1, self.conv_channels), "float32", 0.0),)
        return FixedSpec(arrays=arrays)

    def forward(self, ctx: StepContext, site: int, owns_cache: bool, h: torch.Tensor) -> torch.Tensor:
        if not owns_cache:
            raise ValueError("a recurrence's state cannot be read from another layer")
        T, H, P, N, G = h.shape[0], self.heads, self.vdim, self.n_state, self.groups
        inner, C = self.inner, self.conv_channels
        state = ctx.fixed_arrays(site)
        rows = self.in_proj(ctx, h, torch.float32, "ssd_rows", alias="mixer_in")        # z | x B C | dt
        xbc = ctx.workspace.get("ssd_xbc", (T, C), torch.float32)
        ops.causal_conv(rows, C, self.conv_weight, self.conv_bias, state.get("conv"), ctx.row_of_token, ctx.seg_start,
                        ctx.seg_len, ctx.slot, xbc, silu=True, single_tokens=ctx.max_seg_len == 1, u_off=inner)
        y = ctx.workspace.get("ssd_y", (T, inner), torch.float32)
        chunk_tokens, max_chunks = ops.decay_scan_chunks(ctx.max_seg_len, dim=N, blocks=ctx.n_rows * H * -(-P // 8))
        chunk_state = chunk_decay = None
        if chunk_tokens:
            n_state, n_decay = ops.decay_scan_scratch(ctx.n_rows, max_chunks, H, N, P, chunk_tokens)
            chunk_state = ctx.workspace.get("scan_chunk_state", (n_state,), torch.float32)
            chunk_decay = ctx.workspace.get("scan_chunk_decay", (n_decay,), torch.float32)
        ops.decay_scan(xbc, inner + G * N, H // G, xbc, inner, H // G, xbc, 0, state["state"], ctx.seg_start, ctx.seg_len,
                       ctx.slot, y, H, N, P, step=rows, step_off=inner + C, step_bias=self.dt_bias, rate=self.rate,
                       v_times_step=True, skip=self.D, chunk_tokens=chunk_tokens, max_chunks=max_chunks,
                       chunk_state=chunk_state, chunk_decay=chunk_decay)
        gated = ctx.workspace.get("ssd_gated", (T, inner), self.out_proj.in_dtype, alias="mixer_mid")
        ops.gated_group_norm(y, rows, 0, self.norm, self.norm_groups, self.eps, gated, gate_first=True)
        return self.out_proj(ctx, gated, torch.float32, "mixer_out", sliced_ok=True, into=ctx.stream)


register_part("mixer", "mamba2", Mamba2)
