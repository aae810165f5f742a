"""Grouped-query attention over the paged cache.

q = Wq h, k = Wk h, v = Wv h (one fused projection), per-head RMS norm of q
and k, rotation, k and v appended to the cache at the tokens' positions before
attention of the same batch, causal softmax attention bounded by position,
then the output projection
(/root/reference/crates/imparo-model/src/lfm2/workflow_cpu.rs:203-250,
/root/reference/crates/imparo-model/src/cpu_support.rs:361-445).

Parameters beyond the sizes: `value_dim` (a head's values where they are not
head_dim wide), `window` (a query at position i sees positions i - window + 1 .. i), `keep_window` (what the cache keeps, where a layer that reads this
layer's cache looks further back than this layer itself; None: everything),
`shared_kv` (the layer has no key and value projections: it is run with
another layer's cache, `LayerCall.cache_of`, and brings queries only),
`weight_suffix` and `names` (how the checkpoint calls the tensors),
`chunk` (instead of a window: a query at position i sees j <= i only in its
own chunk, floor(i / chunk) = floor(j / chunk), chunks counted from position 0
whatever way a prompt was cut), `bias` (q, k, v and the output projection carry
biases, the tensor's name with `bias_suffix`, added in the projection),
`conv_taps` (a causal convolution per channel on q, k and v right behind the
projection, before head norm and rotation: y_t = sum_j w[:, j] u_(t - taps + 1 + j),
no bias, zeros before the start, tensors `<name>.conv`; the last taps - 1
projected rows of a request are state beside its pages),
`exact_weights` (the softmax weights keep float32's precision through the
product with the values: the matrix-core kernels then send what rounding a
weight to bfloat16 took off through a second product; the wave kernel, which
takes every other shape, keeps its weights in float32 anyway)."""
from __future__ import annotations

from typing import Dict, Optional

import torch

from ..cache.pages import FixedArray, PagedSpec, kv_spec, with_fixed_arrays
from ..config.plan import PartSpec
from ..kernels import ops
from ..weights.loader import TensorDecl
from .base import Declared, StepContext
from .linear import Linear, place_matrix, place_projection, place_vector
from .registry import part_class, register_part

_DEFAULT_NAMES = dict(q="q_proj", k="k_proj", v="v_proj", o="o_proj", q_norm="q_norm", k_norm="k_norm")


class Attention:
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
        sfx = spec.get("weight_suffix", ".weight")
        E, H, Hk, D = spec["width"], spec["heads"], spec["kv_heads"], spec["head_dim"]
        Dv = spec.get("value_dim") or D
        shared = bool(spec.get("shared_kv"))
        out: Declared = {n["q"] + sfx: (TensorDecl((H * D, E)), "matrix"),
                         n["o"] + sfx: (TensorDecl((E, H * Dv)), "matrix")}
        if not shared:
            out[n["k"] + sfx] = (TensorDecl((Hk * D, E)), "matrix")
            out[n["v"] + sfx] = (TensorDecl((Hk * Dv, E)), "matrix")
        if spec.get("qk_norm") is not None:
            out[n["q_norm"] + sfx] = (TensorDecl((D,), "vector"), "norm")
            if not shared:
                out[n["k_norm"] + sfx] = (TensorDecl((D,), "vector"), "norm")
        sides = ("q",) if shared else ("q", "k", "v")
        rows = dict(q=H * D, k=Hk * D, v=Hk * Dv)
        if spec.get("bias"):
            bsfx = spec.get("bias_suffix", ".bias")
            for x in sides:
                out[n[x] + bsfx] = (TensorDecl((rows[x],), "vector"), "bias")
            out[n["o"] + bsfx] = (TensorDecl((E,), "vector"), "bias")
        if spec.get("conv_taps"):
            for x in sides:
                out[n[x] + spec.get("conv_suffix", ".conv")] = (TensorDecl((rows[x], spec["conv_taps"]), "vector"), "conv")
        return out

    def __init__(self, spec: PartSpec, tensors: Dict[str, torch.Tensor], device: torch.device,
                 engine_dtype: torch.dtype):
        n = self._names(spec)
        sfx = spec.get("weight_suffix", ".weight")
        self.engine_dtype = engine_dtype
        self.v_transposed = False        # decided with the cache's page size, in cache_spec
        self.width, self.heads, self.kv_heads, self.head_dim = (spec["width"], spec["heads"], spec["kv_heads"],
                                                                spec["head_dim"])
        self.value_dim = int(spec.get("value_dim") or self.head_dim)
        self.shared_kv = bool(spec.get("shared_kv"))
        self.exact_weights = bool(spec.get("exact_weights"))
        if self.heads % self.kv_heads:
            raise ValueError(f"{self.heads} heads cannot share {self.kv_heads} kv heads evenly")
        self.scale = float(spec["scale"])
        self.window: Optional[int] = spec.get("window")
        self.keep_window: Optional[int] = spec.params["keep_window"] if "keep_window" in spec.params else self.window
        self.chunk: Optional[int] = spec.get("chunk")
        if self.chunk is not None:
            if self.window is not None or self.keep_window is not None or self.chunk < 1:
                raise ValueError("a layer sees a window or its own chunk (of at least one position), not both")
            self.window = -int(self.chunk)        # as the kernels take it: a negative window is a chunk of that size
        sides = ("q",) if self.shared_kv else ("q", "k", "v")
        ws = [tensors[n[x] + sfx] for x in sides]
        if len({w.dtype for w in ws}) > 1:
            ws = [w.to(torch.float32) for w in ws]
        bias = out_bias = None
        if spec.get("bias"):
            bsfx = spec.get("bias_suffix", ".bias")
            bias = place_vector(torch.cat([tensors[n[x] + bsfx].to(torch.float32) for x in sides]), device)
            out_bias = place_vector(tensors[n["o"] + bsfx], device)
        # one projection for q | k | v: the same dot products, one launch
        self.qkv = Linear(place_projection(torch.cat(ws, dim=0), engine_dtype, device), bias)
        self.conv_taps = int(spec.get("conv_taps") or 0)
        self.conv_weight = None
        if self.conv_taps:
            if self.conv_taps > 64:
                raise ValueError(f"the conv kernels take at most 64 taps, got {self.conv_taps}")
            csfx = spec.get("conv_suffix", ".conv")
            self.conv_weight = place_vector(torch.cat([tensors[n[x] + csfx].to(torch.float32).reshape(-1, self.conv_taps)
                                                       for x in sides], dim=0), device)
        out = tensors[n["o"] + sfx]
        # The attention kernels write their result in the cache's dtype and the bfloat16 products walk K in steps
        # of 8: where heads x value size is no multiple of 8 the output projection gets columns of zero weight and
        # the attention rows end in as many zeros.
        self.out_fill = (-self.heads * self.value_dim) % 8 if engine_dtype != torch.float32 and out.dtype != torch.float32 else 0
        if self.out_fill:
            out = torch.cat([out, out.new_zeros(out.shape[0], self.out_fill)], dim=1)
        self.out = Linear(place_matrix(out, engine_dtype, device), out_bias)
        norm = spec.get("qk_norm")
        if norm is not None:
            # the kernels that norm a head know one norm: RMS with a weight per dimension, no offset
            if getattr(norm, "kind", "rms_norm") != "rms_norm":
                raise ValueError(f"this attention mixer norms q and k per head with an RMS norm; the plan names "
                                 f"{norm.kind!r} (another norm on the heads is another mixer, with kernels of its own)")
            self.norm_eps = float(norm["eps"])
            self.q_norm = place_vector(tensors[n["q_norm"] + sfx], device)
            # a layer without keys of its own hands the kernels its query weight in the key weight's place
            self.k_norm = self.q_norm if self.shared_kv else place_vector(tensors[n["k_norm"] + sfx], device)
        else:
            self.norm_eps, self.q_norm, self.k_norm = 0.0, None, None
        pos = spec.get("position") or PartSpec("none")
        self.position = part_class("position", pos.kind)(pos, device)
        if self.position.rotary_dim > self.head_dim:
            raise ValueError("the rotated part of a head cannot be wider than the head")

    @property
    def in_dtype(self) -> torch.dtype:
        return self.qkv.in_dtype

    def cache_spec(self, page_size: int) -> PagedSpec:
        """Keys and values per position, laid out as this mixer's kernels read
        them: where the matrix-core kernels apply (bfloat16, pages of at least
        16, head sizes up to 128), V is kept transposed inside a page."""
        self.v_transposed = (self.value_dim == self.head_dim
                             and ops.mfma_attention_supported(self.engine_dtype, page_size, self.head_dim))
        spec = kv_spec(self.kv_heads, self.head_dim, self.keep_window, self.v_transposed, self.value_dim, self.chunk)
        if self.conv_taps > 1:
            spec = with_fixed_arrays(spec, (FixedArray("conv", (self.conv_taps - 1, self.qkv.out_features), "float32", 0.0),))
        return spec

    def _portion_tiles(self, ctx: StepContext) -> int:
        """Tiles of queries that the portions of this batch make, as the prompt kernel counts them."""
        key = ("attention portion tiles", ops.prefill_tile())
        if key not in ctx.memo:
            tile = ops.prefill_tile()
            ctx.memo[key] = sum((int(n) + tile - 1) // tile for n in ctx.host_seg_len if n > 1)
        return ctx.memo[key]

    def _decode_parts(self, ctx: StepContext):
        """Room for the partial results of the single-token rows' splits."""
        split = ops.decode_split()
        n_splits = (ctx.max_context + split - 1) // split
        part_o = ctx.workspace.get("attn_part_o", (ctx.n_single_rows * self.heads * n_splits * self.head_dim,),
                                   torch.float32)
        part_ml = ctx.workspace.get("attn_part_ml", (ctx.n_single_rows * self.heads * n_splits * 2,), torch.float32)
        return part_o, part_ml

    def forward(self, ctx: StepContext, site: int, owns_cache: bool, h: torch.Tensor) -> torch.Tensor:
        T = h.shape[0]
        if self.shared_kv and owns_cache:
            raise ValueError("a layer without key and value projections must be run with another layer's cache")
        qkv = self.qkv(ctx, h, torch.float32, "qkv", alias="mixer_in")
        if self.conv_taps:
            if not owns_cache:
                raise ValueError("a conv's history cannot be read from another layer")
            mixed = ctx.workspace.get("qkv_conv", tuple(qkv.shape), torch.float32)
            history = ctx.fixed_arrays(site)["conv"] if self.conv_taps > 1 else None
            qkv = ops.causal_conv(qkv, qkv.shape[1], self.conv_weight, None, history, ctx.row_of_token, ctx.seg_start,
                                  ctx.seg_len, ctx.slot, mixed, silu=False, single_tokens=ctx.max_seg_len == 1)
        k_cache, v_cache, table = ctx.kv(site)
        vt = self.v_transposed
        inv_freq = self.position.inv_freq
        interleaved = bool(getattr(self.position, "interleaved", False))
        Dv = self.value_dim
        if (vt and owns_cache and not self.exact_weights and ctx.single_rows is not None and ctx.n_single_rows == T and not ctx.n_portion_rows
                and ops.attention_decode_qkv_pays(T, ctx.max_context)
                and ops.attention_decode_qkv_takes(self.head_dim, 0 if inv_freq is None else inv_freq.shape[0])):
            # every row brings one token: head norm, rotation and the write of the new key and value ride
            # in the attention launch (the new key is weighed in from registers)
            o = ctx.workspace.get("attn_out", (T, self.heads * self.head_dim), ctx.dtype, alias="mixer_mid")
            part_o, part_ml = self._decode_parts(ctx)
            ops.attention_decode_qkv(qkv, self.q_norm, self.k_norm, self.norm_eps, inv_freq, k_cache, v_cache, o,
                                     part_o, part_ml, ctx.single_rows, ctx.n_single_rows, ctx.seg_start,
                                     ctx.positions, table, self.heads, self.scale, self.window, ctx.max_context,
                                     interleaved=interleaved)
            return self.out(ctx, o, torch.float32, "mixer_out", sliced_ok=True, into=ctx.stream)
        q = ctx.workspace.get("q", (T, self.heads, self.head_dim), ctx.dtype)
        ops.qk_norm_rope_store(qkv, self.q_norm, self.k_norm, self.norm_eps, inv_freq,
                               ctx.positions, ctx.row_of_token, table if owns_cache else None, ctx.page_size,
                               q, k_cache if owns_cache else None, v_cache if owns_cache else None,
                               self.heads, 0 if self.shared_kv else self.kv_heads, self.head_dim, v_transposed=vt,
                               interleaved=interleaved, value_dim=Dv)
        o = ctx.workspace.get("attn_out", (T, self.heads * Dv + self.out_fill), ctx.dtype, alias="mixer_mid")
        if vt and ctx.single_rows is not None:
            # matrix-core kernels: single tokens split over their keys, portions tiled over their queries
            if ctx.n_single_rows:
                part_o, part_ml = self._decode_parts(ctx)
                ops.attention_decode(q, k_cache, v_cache, o, part_o, part_ml, ctx.single_rows, ctx.n_single_rows,
                                     ctx.seg_start, ctx.positions, table, self.scale, self.window, ctx.max_context,
                                     exact=self.exact_weights)
            if ctx.n_portion_rows:
                # few queries over long contexts: each block's keys in parts, merged by a second launch
                n_tiles = self._portion_tiles(ctx)
                # (the bound on the contexts that the launch itself sees: what its block table can hold)
                parts = ops.attention_prefill_splits(n_tiles, self.heads, self.kv_heads, self.head_dim,
                                                     table.shape[1] * ctx.page_size)
                part_o = part_ml = None
                if parts > 1:
                    part_o = ctx.workspace.get("attn_prefill_part_o", (T * self.heads * parts * self.head_dim,),
                                               torch.float32)
                    part_ml = ctx.workspace.get("attn_prefill_part_ml", (T * self.heads * parts * 2,), torch.float32)
                ops.attention_prefill(q, k_cache, v_cache, o, ctx.portion_rows, ctx.n_portion_rows,
                                      n_tiles, ctx.seg_start, ctx.seg_len, ctx.positions, table,
                                      self.scale, self.window, part_o, part_ml, parts, exact=self.exact_weights)
        else:
            ops.attention(q, k_cache, v_cache, o, ctx.positions, ctx.row_of_token, table, self.scale, self.window,
                          v_transposed=vt)
        if o.dtype != self.out.in_dtype:
            raise ValueError("the output projection's weight dtype differs from the attention output's")
        # a delta for the residual stream: the next norm adds slices, so it may come sliced
        return self.out(ctx, o, torch.float32, "mixer_out", sliced_ok=True, into=ctx.stream)


    def can_emit(self) -> bool:
        # the step program's attention has one head size, keys and values of its own, and the matrix-core kernels
        return (self.value_dim == self.head_dim and not self.shared_kv and not self.exact_weights
                and not self.out_fill and not self.conv_taps and self.chunk is None)

    def emit(self, program, site: int, owns_cache: bool) -> None:
        """Appends `forward` to a native step program."""
        from ..kernels.program import AttentionDesc
        arrays = program.storage.paged[site]
        k_cache, v_cache = arrays["k"], arrays["v"]
        inv_freq = self.position.inv_freq
        program.attention(AttentionDesc(
            program.linear(self.qkv), program.linear(self.out),
            program._hold(self.q_norm, "q norm weight", torch.float32),
            program._hold(self.k_norm, "k norm weight", torch.float32), self.norm_eps,
            program._hold(inv_freq, "inverse frequencies", torch.float32), 0 if inv_freq is None else inv_freq.shape[0],
            int(bool(getattr(self.position, "interleaved", False))), self.heads, self.kv_heads, self.head_dim,
            self.scale, int(self.window or 0), program._hold(k_cache, "k cache"), program._hold(v_cache, "v cache"),
            k_cache.shape[0], int(self.v_transposed), program.group_of_site[site], int(owns_cache)))


register_part("mixer", "attention", Attention)
