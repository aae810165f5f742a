"""Python faces of the gfx950 kernels.

Each function checks on the host what its kernel assumes (device, dtype,
contiguity, shapes, index ranges that the host knows), then launches on the
current stream. There is no CPU path: a tensor that is not on the GPU is an
error, and so is a missing kernel library.
"""
from __future__ import annotations

from typing import Optional

import ctypes

import torch

from .library import library

F32, BF16 = 0, 1
ATTENTION_MAX_HEAD_DIM = 576      # the wave attention kernel's longest key row
HGRN2_MAX_DIM = 512               # state rows a head of the gated linear recurrence
_CODES = {torch.float32: F32, torch.bfloat16: BF16}


class KernelArgumentError(ValueError):
    pass


def _code(t: torch.Tensor, what: str) -> int:
    if t.dtype not in _CODES:
        raise KernelArgumentError(f"{what} has dtype {t.dtype}; kernels take float32 or bfloat16")
    return _CODES[t.dtype]


def _dev(t: Optional[torch.Tensor], what: str, dtype=None, shape=None) -> int:
    """Checks a tensor and returns its device address (0 for None)."""
    if t is None:
        return 0
    if not isinstance(t, torch.Tensor):
        raise KernelArgumentError(f"{what} is not a tensor")
    if t.device.type != "cuda":
        raise KernelArgumentError(f"{what} is on {t.device}; the kernels run on the GPU only")
    if not t.is_contiguous():
        raise KernelArgumentError(f"{what} is not contiguous")
    if dtype is not None and t.dtype != dtype:
        raise KernelArgumentError(f"{what} has dtype {t.dtype}, expected {dtype}")
    if shape is not None and tuple(t.shape) != tuple(shape):
        raise KernelArgumentError(f"{what} has shape {list(t.shape)}, expected {list(shape)}")
    return t.data_ptr()


_launch_stream: Optional[int] = None


class on_current_stream:
    """For a run of launches that all go to the stream that is current now (a
    step's hundred kernels, also under graph capture): looks the stream up once
    instead of once per launch, which costs more host time than the launch."""

    def __enter__(self):
        global _launch_stream
        self._before = _launch_stream
        _launch_stream = torch.cuda.current_stream().cuda_stream
        return self

    def __exit__(self, *exc):
        global _launch_stream
        _launch_stream = self._before
        return False


def _stream() -> int:
    if _launch_stream is not None:
        return _launch_stream
    return torch.cuda.current_stream().cuda_stream


def _check(status: int, name: str) -> None:
    if status == 0:
        return
    why = {1: "an argument was refused (size or pointer the kernel cannot take)",
           2: "the launch failed"}.get(status, f"status {status}")
    raise KernelArgumentError(f"{name}: {why}")


def load_code() -> None:
    """Loads every kernel file's code onto the current device (the runtime would do so at each
    file's first launch, which a stream under graph capture cannot)."""
    _check(library().imparo_load_code(), "load_code")


def embed_gather(table: torch.Tensor, ids: torch.Tensor, out: torch.Tensor, scale: float = 1.0) -> torch.Tensor:
    """out[t] = table[ids[t]] * scale in float32."""
    vocab, width = table.shape
    n = ids.shape[0]
    _check(library().imparo_embed_gather_scaled(
        _dev(table, "embedding table"), _code(table, "embedding table"),
        _dev(ids, "token ids", torch.int32, (n,)), _dev(out, "embedding output", torch.float32, (n, width)),
        n, width, vocab, float(scale), _stream()), "embed_gather")
    return out


def place_tokens(ids: torch.Tensor, dst: torch.Tensor, src: torch.Tensor, src_index: torch.Tensor,
                 vocab: int) -> torch.Tensor:
    """ids[dst[i]] = src[src_index[i]]: token ids that the step before sampled and that were
    not read back. The caller has checked the indices on the host (they come from there)."""
    n = dst.shape[0]
    _check(library().imparo_place_tokens(
        _dev(ids, "token ids", torch.int32), _dev(dst, "places", torch.int32, (n,)),
        _dev(src, "sampled tokens", torch.int32), _dev(src_index, "indices of sampled tokens", torch.int32, (n,)),
        n, vocab, _stream()), "place_tokens")
    return ids


def rms_norm(x: torch.Tensor, weight: torch.Tensor, eps: float, out: torch.Tensor,
             delta: Optional[torch.Tensor] = None, rows: Optional[torch.Tensor] = None,
             write_back: bool = False) -> torch.Tensor:
    """out[i] = norm(x[src] (+ delta[src])) * weight, src = rows[i] or i.
    `delta` is shaped like x, or [slices, *x.shape]: slices are added in order.
    write_back stores x + delta into x (only without rows)."""
    width = x.shape[-1]
    n_out = out.shape[0]
    if rows is None and n_out != x.shape[0]:
        raise KernelArgumentError(f"rms_norm: out has {n_out} rows, x has {x.shape[0]}")
    if rows is not None and rows.shape[0] != n_out:
        raise KernelArgumentError("rms_norm: one source row index per output row is needed")
    if write_back and (rows is not None or delta is None):
        raise KernelArgumentError("rms_norm: write_back needs a delta and no row selection")
    n_delta = 0
    if delta is not None:
        n_delta = delta.shape[0] if delta.dim() == x.dim() + 1 else 1
        want = (n_delta,) + tuple(x.shape) if delta.dim() == x.dim() + 1 else tuple(x.shape)
        _dev(delta, "rms_norm delta", torch.float32, want)
    _check(library().imparo_rms_norm(
        _dev(x, "rms_norm x", torch.float32), _dev(delta, "rms_norm delta", torch.float32), n_delta, x.shape[0],
        _dev(rows, "rms_norm rows", torch.int32), _dev(weight, "rms_norm weight", torch.float32, (width,)),
        _dev(out, "rms_norm out", None, (n_out, width)), _code(out, "rms_norm out"),
        n_out, width, float(eps), int(write_back), _stream()), "rms_norm")
    return out


def gemm_slices(m: int, n: int, k: int, dtype: torch.dtype) -> int:
    """Into how many slices of K this product may be cut when its consumer adds the slices (1: none)."""
    return int(library().imparo_gemm_slices(m, n, k, _CODES.get(dtype, -1)))


def gemm_adds(m: int, n: int, k: int, dtype: torch.dtype) -> bool:
    """Whether `gemm(..., add=True)` is taken for this shape (many rows on the tile kernel, K in one piece)."""
    return bool(library().imparo_gemm_adds(m, n, k, _CODES.get(dtype, -1)))


def gemm(x: torch.Tensor, w: torch.Tensor, out: torch.Tensor, bias: Optional[torch.Tensor] = None,
         swiglu: bool = False, variant: int = 0, add: bool = False) -> torch.Tensor:
    """out[m, n] = x[m, k] . w[n, k]^T (+ bias[n]); x and w share a dtype; float32
    accumulate. With `swiglu` the rows of w alternate gate and up and out is
    [m, n/2] = silu(gate) * up. An `out` of shape [slices, m, n] (slices =
    gemm_slices(...)) receives the sums over slices of K, to be added by the consumer.
    With `add` (float32 out, where gemm_adds(...) says so) the product is added to what `out` holds.
    `variant` other than 0 names the kernel (tests and measurements only; see imparo_gemm_variant)."""
    m, k = x.shape
    n, kw = w.shape
    if kw != k:
        raise KernelArgumentError(f"gemm: x has {k} columns but the weight has {kw}")
    if x.dtype != w.dtype:
        raise KernelArgumentError(f"gemm: x is {x.dtype} but the weight is {w.dtype}")
    if x.dtype == torch.bfloat16 and k % 8 != 0:
        raise KernelArgumentError(f"gemm: the bfloat16 kernels need the inner size to be a multiple of 8, got {k}")
    if swiglu and n % 2:
        raise KernelArgumentError("gemm: a gate/up weight has an even number of rows")
    slices = 1
    if out.dim() == 3:
        slices = out.shape[0]
        if (slices != gemm_slices(m, n, k, x.dtype) and not variant) or swiglu or out.dtype != torch.float32:
            raise KernelArgumentError(f"gemm: this product cannot be cut into {slices} slices of K")
        _dev(out, "gemm out", torch.float32, (slices, m, n))
    else:
        _dev(out, "gemm out", None, (m, n // 2 if swiglu else n))
    if add and (swiglu or slices != 1 or variant or out.dtype != torch.float32 or not gemm_adds(m, n, k, x.dtype)):
        raise KernelArgumentError("gemm: this product cannot be added to what its output holds")
    args = (_dev(x, "gemm x"), _dev(w, "gemm weight"), _dev(bias, "gemm bias", torch.float32, (n,)),
            out.data_ptr(), _code(x, "gemm x"), _code(out, "gemm out"), m, n, k, 2 if add else int(swiglu), slices)
    if variant:
        _check(library().imparo_gemm_variant(*args, int(variant), _stream()), "gemm")
    else:
        _check(library().imparo_gemm(*args, _stream()), "gemm")
    return out


def qk_norm_rope_store(qkv: torch.Tensor, q_weight: Optional[torch.Tensor], k_weight: Optional[torch.Tensor],
                       eps: float, inv_freq: Optional[torch.Tensor], positions: torch.Tensor,
                       row_of_token: torch.Tensor, block_table: Optional[torch.Tensor], page_size: int,
                       q_out: torch.Tensor, k_cache: Optional[torch.Tensor], v_cache: Optional[torch.Tensor],
                       heads: int, kv_heads: int, head_dim: int, v_transposed: bool = False,
                       interleaved: bool = False, value_dim: Optional[int] = None) -> torch.Tensor:
    """`inv_freq` [n] turns pair i by position * inv_freq[i]: pair i is dims (i, i + n), or with
    `interleaved` dims (2i, 2i + 1). `value_dim`: the size of a head's values where it is not
    head_dim (the row then ends in kv_heads units of that size). kv_heads 0: rows of queries only."""
    n = qkv.shape[0]
    value_dim = head_dim if value_dim is None else int(value_dim)
    row_width = (heads + kv_heads) * head_dim + kv_heads * value_dim
    write_kv = k_cache is not None
    n_freq = 0 if inv_freq is None else inv_freq.shape[0]
    n_pages = 0
    table_stride = 0
    if write_kv:
        n_pages = k_cache.shape[0]
        _dev(k_cache, "k cache", q_out.dtype, (n_pages, kv_heads, page_size, head_dim))
        _dev(v_cache, "v cache", q_out.dtype, (n_pages, kv_heads, value_dim, page_size) if v_transposed
             else (n_pages, kv_heads, page_size, value_dim))
        if block_table is None or block_table.dim() != 2:
            raise KernelArgumentError("qk_norm_rope_store: a [rows, pages] block table is needed to write the cache")
        table_stride = block_table.shape[1]
    _check(library().imparo_qk_norm_rope_store_dv(
        _dev(qkv, "qkv", torch.float32, (n, row_width)),
        _dev(q_weight, "q norm weight", torch.float32, (head_dim,)),
        _dev(k_weight, "k norm weight", torch.float32, (head_dim,)), float(eps),
        _dev(inv_freq, "inverse frequencies", torch.float32), n_freq, int(interleaved),
        _dev(positions, "positions", torch.int32, (n,)), _dev(row_of_token, "row_of_token", torch.int32, (n,)),
        _dev(block_table, "block table", torch.int32), table_stride, page_size,
        _dev(q_out, "q out", None, (n, heads, head_dim)), _dev(k_cache, "k cache"), _dev(v_cache, "v cache"),
        _code(q_out, "q out"), int(write_kv), n, heads, kv_heads, head_dim, value_dim, n_pages, int(v_transposed),
        _stream()), "qk_norm_rope_store")
    return q_out


def attention(q: torch.Tensor, k_cache: torch.Tensor, v_cache: torch.Tensor, out: torch.Tensor,
              positions: torch.Tensor, row_of_token: torch.Tensor, block_table: torch.Tensor,
              scale: float, window: Optional[int], v_transposed: bool = False) -> torch.Tensor:
    """The general kernel: any page size, head sizes up to 512 (values of a size of their own
    are read off the value cache's shape), float32 or bfloat16; one wave per (token, head). `out`
    may be wider than heads x value size: the rest of a row is written as zeros."""
    n, heads, head_dim = q.shape
    n_pages, kv_heads, page_size, hd = k_cache.shape
    value_dim = v_cache.shape[2] if v_transposed else v_cache.shape[3]
    if hd != head_dim:
        raise KernelArgumentError(f"attention: q has head size {head_dim}, the cache {hd}")
    if heads % kv_heads != 0:
        raise KernelArgumentError(f"attention: {heads} heads cannot share {kv_heads} kv heads evenly")
    if out.dim() != 2 or out.shape[0] != n or out.shape[1] < heads * value_dim:
        raise KernelArgumentError(f"attention: out is {list(out.shape)}; [{n}, at least {heads * value_dim}] is needed")
    _check(library().imparo_attention_dv(
        _dev(q, "q"), _dev(k_cache, "k cache", q.dtype),
        _dev(v_cache, "v cache", q.dtype, (n_pages, kv_heads, value_dim, page_size) if v_transposed
             else (n_pages, kv_heads, page_size, value_dim)),
        _dev(out, "attention out", q.dtype), _code(q, "q"),
        _dev(positions, "positions", torch.int32, (n,)), _dev(row_of_token, "row_of_token", torch.int32, (n,)),
        _dev(block_table, "block table", torch.int32), block_table.shape[1], page_size,
        n, heads, kv_heads, head_dim, value_dim, out.shape[1], n_pages, float(scale), int(window or 0),
        int(v_transposed), _stream()), "attention")
    return out


def decode_split() -> int:
    """Keys per split of the matrix-core decode kernel: its partial results hold one entry per split."""
    return int(library().imparo_attention_decode_split())


def prefill_tile() -> int:
    """Queries per tile that `attention_prefill`'s n_tiles counts."""
    return int(library().imparo_attention_prefill_tile())


def mfma_attention_supported(dtype: torch.dtype, page_size: int, head_dim: int) -> bool:
    return (dtype == torch.bfloat16 and page_size >= 16 and page_size & (page_size - 1) == 0
            and head_dim % 16 == 0 and head_dim <= 128)


def _check_mfma(q, k_cache, v_cache, out):
    n, heads, head_dim = q.shape
    n_pages, kv_heads, page_size, hd = k_cache.shape
    if not mfma_attention_supported(q.dtype, page_size, head_dim) or hd != head_dim:
        raise KernelArgumentError(f"the matrix-core attention kernels take bfloat16, pages of a power of two >= 16 and "
                                  f"head sizes in steps of 16 up to 128; got {q.dtype}, pages of {page_size}, "
                                  f"head size {head_dim}")
    if heads % kv_heads != 0:
        raise KernelArgumentError(f"attention: {heads} heads cannot share {kv_heads} kv heads evenly")
    _dev(k_cache, "k cache", torch.bfloat16)
    _dev(v_cache, "v cache", torch.bfloat16, (n_pages, kv_heads, head_dim, page_size))
    _dev(out, "attention out", torch.bfloat16, (n, heads * head_dim))
    return n, heads, head_dim, n_pages, kv_heads, page_size


def attention_decode(q, k_cache, v_cache, out, part_o, part_ml, rows, n_rows: int, seg_start, positions,
                     block_table, scale: float, window: Optional[int], max_context: int,
                     exact: bool = False) -> torch.Tensor:
    """Split-KV attention for rows that bring one token each. `rows` lists
    them (indices into seg_start); `max_context` bounds every row's position + 1.
    `exact`: the softmax weights keep float32's precision through the product with the values."""
    n, heads, head_dim, n_pages, kv_heads, page_size = _check_mfma(q, k_cache, v_cache, out)
    split = decode_split()
    n_splits = max(1, (max_context + split - 1) // split)
    if part_o.numel() < n_rows * heads * n_splits * head_dim or part_ml.numel() < n_rows * heads * n_splits * 2:
        raise KernelArgumentError("attention_decode: the scratch for partial results is too small")
    _check((library().imparo_attention_decode_exact if exact else library().imparo_attention_decode)(
        _dev(q, "q"), k_cache.data_ptr(), v_cache.data_ptr(), out.data_ptr(),
        _dev(part_o, "partial outputs", torch.float32), _dev(part_ml, "partial sums", torch.float32),
        _dev(rows, "decode rows", torch.int32), n_rows, _dev(seg_start, "seg_start", torch.int32),
        _dev(positions, "positions", torch.int32, (n,)), _dev(block_table, "block table", torch.int32),
        block_table.shape[1], page_size, heads, kv_heads, head_dim, n_pages, float(scale), int(window or 0),
        n_splits, _stream()), "attention_decode")
    return out


def attention_decode_qkv_takes(head_dim: int, n_freq: int) -> bool:
    """Whether attention_decode_qkv takes heads of this size with this many rotated pairs."""
    return bool(library().imparo_attention_decode_qkv_takes(int(head_dim), int(n_freq)))


def attention_decode_qkv_pays(n_rows: int, max_context: int) -> bool:
    """Whether the one launch is the faster way for a step of this many rows whose longest context is `max_context`."""
    n_splits = max(1, -(-int(max_context) // decode_split()))
    return bool(library().imparo_attention_decode_qkv_pays(int(n_rows), n_splits))


def attention_decode_qkv(qkv, q_weight, k_weight, eps: float, inv_freq, k_cache, v_cache, out, part_o, part_ml,
                         rows, n_rows: int, seg_start, positions, block_table, heads: int, scale: float,
                         window: Optional[int], max_context: int, interleaved: bool = False,
                         write_kv: bool = True) -> torch.Tensor:
    """qk_norm_rope_store and attention_decode in one launch less, for a step whose rows all bring one
    token: `qkv` is the fused projection's float32 rows; the new keys and values are weighed in from
    registers and, with `write_kv`, written into their pages (V pages transposed)."""
    n_pages, kv_heads, page_size, head_dim = k_cache.shape
    n = qkv.shape[0]
    _dev(qkv, "qkv", torch.float32, (n, (heads + 2 * kv_heads) * head_dim))
    _dev(out, "attention out", torch.bfloat16)
    if out.numel() != n * heads * head_dim:
        raise KernelArgumentError("attention_decode_qkv: the output does not match the rows")
    if k_cache.dtype != torch.bfloat16 or v_cache.dtype != torch.bfloat16 or tuple(v_cache.shape) != (n_pages, kv_heads, head_dim, page_size):
        raise KernelArgumentError("attention_decode_qkv: bfloat16 caches, V pages transposed")
    n_freq = 0 if inv_freq is None else inv_freq.shape[0]
    if not attention_decode_qkv_takes(head_dim, n_freq):
        raise KernelArgumentError(f"attention_decode_qkv: heads of {head_dim} with {n_freq} rotated pairs are not taken")
    split = decode_split()
    n_splits = max(1, (max_context + split - 1) // split)
    if part_o.numel() < n_rows * heads * n_splits * head_dim or part_ml.numel() < n_rows * heads * n_splits * 2:
        raise KernelArgumentError("attention_decode_qkv: the scratch for partial results is too small")
    _check(library().imparo_attention_decode_qkv(
        qkv.data_ptr(), _dev(q_weight, "q norm weight", torch.float32, (head_dim,)),
        _dev(k_weight, "k norm weight", torch.float32, (head_dim,)), float(eps),
        _dev(inv_freq, "inv_freq", torch.float32), n_freq, int(bool(interleaved)), k_cache.data_ptr(),
        v_cache.data_ptr(), int(bool(write_kv)), out.data_ptr(), _dev(part_o, "partial outputs", torch.float32),
        _dev(part_ml, "partial sums", torch.float32), _dev(rows, "decode rows", torch.int32), n_rows,
        _dev(seg_start, "seg_start", torch.int32), _dev(positions, "positions", torch.int32, (n,)),
        _dev(block_table, "block table", torch.int32), block_table.shape[1], page_size, heads, kv_heads, head_dim,
        n_pages, float(scale), int(window or 0), n_splits, _stream()), "attention_decode_qkv")
    return out


def attention_prefill_splits(n_tiles: int, heads: int, kv_heads: int, head_dim: int, max_context: int) -> int:
    """Into how many parts the keys of a launch of prompt portions are cut (1: none): few queries
    over long contexts would leave most of the chip idle."""
    return int(library().imparo_attention_prefill_splits(n_tiles, heads, kv_heads, head_dim, max_context))


def attention_prefill(q, k_cache, v_cache, out, rows, n_rows: int, n_tiles: int, seg_start, seg_len, positions,
                      block_table, scale: float, window: Optional[int], part_o: Optional[torch.Tensor] = None,
                      part_ml: Optional[torch.Tensor] = None, n_splits: int = 1, exact: bool = False) -> torch.Tensor:
    """Tiled attention for rows that bring a portion of a prompt. `n_tiles` is
    the sum over the listed rows of ceil(seg_len / prefill_tile()). With `n_splits` > 1
    (attention_prefill_splits) each block's keys are walked in that many parts,
    merged by a second launch: `part_o` [n, heads, n_splits, head_dim] and
    `part_ml` [n, heads, n_splits, 2] float32 hold the parts."""
    n, heads, head_dim, n_pages, kv_heads, page_size = _check_mfma(q, k_cache, v_cache, out)
    if n_splits > 1:
        if part_o is None or part_ml is None:
            raise KernelArgumentError("attention_prefill: parts of the keys need buffers for their results")
        _dev(part_o, "part_o", torch.float32)
        _dev(part_ml, "part_ml", torch.float32)
        if part_o.numel() < n * heads * n_splits * head_dim or part_ml.numel() < n * heads * n_splits * 2:
            raise KernelArgumentError("attention_prefill: the buffers for the parts are too small")
    _check((library().imparo_attention_prefill_exact if exact else library().imparo_attention_prefill)(
        _dev(q, "q"), k_cache.data_ptr(), v_cache.data_ptr(), out.data_ptr(),
        part_o.data_ptr() if n_splits > 1 else None, part_ml.data_ptr() if n_splits > 1 else None, int(n_splits),
        _dev(rows, "prefill rows", torch.int32), n_rows, n_tiles, _dev(seg_start, "seg_start", torch.int32),
        _dev(seg_len, "seg_len", torch.int32), _dev(positions, "positions", torch.int32, (n,)),
        _dev(block_table, "block table", torch.int32), block_table.shape[1], page_size, heads, kv_heads, head_dim,
        n_pages, float(scale), int(window or 0), _stream()), "attention_prefill")
    return out


def short_conv(bcx: torch.Tensor, weight: torch.Tensor, bias: Optional[torch.Tensor], state: torch.Tensor,
               row_of_token: torch.Tensor, seg_start: torch.Tensor, seg_len: torch.Tensor, slot: torch.Tensor,
               out: torch.Tensor, single_tokens: bool = False) -> torch.Tensor:
    """Gated short convolution of every request's segment, then the state
    update; the two launches are ordered by the stream. `single_tokens`: the
    caller knows that every request brings exactly one token; output and
    update then share one launch."""
    n, three_w = bcx.shape
    width, taps = weight.shape
    if three_w != 3 * width:
        raise KernelArgumentError(f"short_conv: rows of {three_w} values do not hold B, C and x of width {width}")
    n_slots = state.shape[0]
    n_rows = seg_start.shape[0]
    lib = library()
    if single_tokens:
        if n != n_rows:
            raise KernelArgumentError("short_conv: single_tokens needs one token per request")
        _check(lib.imparo_short_conv_decode(
            _dev(bcx, "bcx", torch.float32), _dev(weight, "conv weight", torch.float32),
            _dev(bias, "conv bias", torch.float32, (width,)),
            _dev(state, "conv state", torch.float32, (n_slots, taps - 1, width)),
            _dev(slot, "slot", torch.int32, (n_rows,)), _dev(out, "conv out", None, (n, width)), _code(out, "conv out"),
            n_rows, width, taps, n_slots, _stream()), "short_conv_decode")
        return out
    _check(lib.imparo_short_conv(
        _dev(bcx, "bcx", torch.float32), _dev(weight, "conv weight", torch.float32),
        _dev(bias, "conv bias", torch.float32, (width,)),
        _dev(state, "conv state", torch.float32, (n_slots, taps - 1, width)),
        _dev(row_of_token, "row_of_token", torch.int32, (n,)), _dev(seg_start, "seg_start", torch.int32, (n_rows,)),
        _dev(slot, "slot", torch.int32, (n_rows,)), _dev(out, "conv out", None, (n, width)), _code(out, "conv out"),
        n, width, taps, n_slots, n_rows, _stream()), "short_conv")
    _check(lib.imparo_short_conv_state(
        bcx.data_ptr(), state.data_ptr(), seg_start.data_ptr(), _dev(seg_len, "seg_len", torch.int32, (n_rows,)),
        slot.data_ptr(), n_rows, n, width, taps, n_slots, _stream()), "short_conv_state")
    return out


def in_proj_conv_decode_supported(x_rows: int, weight: torch.Tensor) -> bool:
    """The fused launch takes a bfloat16 projection and at most 16 rows."""
    return weight.dtype == torch.bfloat16 and 0 < x_rows <= 16 and weight.shape[0] % 24 == 0 and weight.shape[1] % 8 == 0


def in_proj_conv_decode(x: torch.Tensor, in_weight: torch.Tensor, in_bias: Optional[torch.Tensor],
                        conv_weight: torch.Tensor, conv_bias: Optional[torch.Tensor], state: torch.Tensor,
                        slot: torch.Tensor, out: torch.Tensor) -> torch.Tensor:
    """For rows of one token each: [B | C | x] = x . in_weight^T (+ bias), then the gated short
    convolution against each row's state, which is shifted; one launch."""
    m, k = x.shape
    three_e, kw = in_weight.shape
    width, taps = conv_weight.shape
    if three_e != 3 * width or kw != k:
        raise KernelArgumentError(f"in_proj_conv_decode: a [{three_e}, {kw}] projection does not feed a conv of "
                                  f"width {width} from rows of {k}")
    if not in_proj_conv_decode_supported(m, in_weight) or x.dtype != torch.bfloat16:
        raise KernelArgumentError("in_proj_conv_decode: takes 1 to 16 bfloat16 rows and a bfloat16 projection whose "
                                  "width is a multiple of 8")
    n_slots = state.shape[0]
    _check(library().imparo_in_proj_conv_decode(
        _dev(x, "x", torch.bfloat16), _dev(in_weight, "in_proj weight", torch.bfloat16),
        _dev(in_bias, "in_proj bias", torch.float32, (three_e,)), _dev(conv_weight, "conv weight", torch.float32),
        _dev(conv_bias, "conv bias", torch.float32, (width,)),
        _dev(state, "conv state", torch.float32, (n_slots, taps - 1, width)),
        _dev(slot, "slot", torch.int32, (m,)), _dev(out, "conv out", None, (m, width)), _code(out, "conv out"),
        m, width, k, taps, n_slots, _stream()), "in_proj_conv_decode")
    return out


def rows_parts(n: int) -> int:
    """Partial sums of squares that `rows_gemm(..., into=...)` leaves for a weight of n rows."""
    return int(library().imparo_rows_parts(int(n)))


def rows_gemm(x: torch.Tensor, w: torch.Tensor, out: Optional[torch.Tensor] = None, bias: Optional[torch.Tensor] = None,
              swiglu: bool = False, ssq_in: Optional[torch.Tensor] = None, eps: float = 0.0,
              into: Optional[torch.Tensor] = None, ssq_out: Optional[torch.Tensor] = None,
              weighted_out: Optional[torch.Tensor] = None, weighted_by: Optional[torch.Tensor] = None) -> torch.Tensor:
    """Products of a step of at most 16 rows with a norm of the residual stream folded in. x [m, k] and
    w [n, k] bfloat16. With `ssq_in` [parts, 16] and `eps`, x is the stream times a norm's weight and row
    r's result is multiplied by rsqrt(sum_p ssq_in[p][r] / k + eps). Stored to `out` ([m, n], or [m, n/2]
    with `swiglu`), or added to `into` [m, n] float32 in place; then `ssq_out` [rows_parts(n), 16] receives
    the partial sums of squares of the new rows and, with `weighted_by` [n], `weighted_out` [m, n]
    bfloat16 the new rows times it."""
    m, k = x.shape
    n, kw = w.shape
    if kw != k or x.dtype != torch.bfloat16 or w.dtype != torch.bfloat16 or not 0 < m <= 16 or k % 8:
        raise KernelArgumentError("rows_gemm: 1 to 16 bfloat16 rows, a bfloat16 weight over the same inner size, "
                                  "a multiple of 8")
    n_parts = 0
    if ssq_in is not None:
        n_parts = ssq_in.shape[0]
        _dev(ssq_in, "sums of squares", torch.float32, (n_parts, 16))
    if into is not None:
        if out is not None or swiglu or ssq_out is None:
            raise KernelArgumentError("rows_gemm: adding to the stream stores nothing else and leaves sums of squares")
        _dev(into, "stream", torch.float32, (m, n))
        _dev(ssq_out, "sums of squares out", torch.float32, (rows_parts(n), 16))
        epilogue, y, code = 2, None, F32
    else:
        if out is None:
            raise KernelArgumentError("rows_gemm: an output is needed")
        _dev(out, "rows_gemm out", None, (m, n // 2 if swiglu else n))
        epilogue, y, code = int(swiglu), out, _code(out, "rows_gemm out")
    _check(library().imparo_rows_gemm(
        _dev(x, "x"), _dev(ssq_in, "sums of squares"), n_parts, float(eps), _dev(w, "weight"),
        _dev(bias, "bias", torch.float32, (n,)), _dev(y, "out"), code, _dev(into, "stream"), _dev(ssq_out, "ssq out"),
        _dev(weighted_out, "weighted out", torch.bfloat16, (m, n)), _dev(weighted_by, "weighted by", torch.float32, (n,)),
        m, n, k, epilogue, _stream()), "rows_gemm")
    return into if into is not None else out


def argmax_rows(logits: torch.Tensor, out: torch.Tensor) -> torch.Tensor:
    n, vocab = logits.shape
    _check(library().imparo_argmax_rows(_dev(logits, "logits", torch.float32), _dev(out, "picks", torch.int32, (n,)),
                                        n, vocab, _stream()), "argmax_rows")
    return out


def sample_rows(logits: torch.Tensor, temperature: torch.Tensor, uniform: torch.Tensor,
                out: torch.Tensor) -> torch.Tensor:
    n, vocab = logits.shape
    _check(library().imparo_sample_rows(
        _dev(logits, "logits", torch.float32), _dev(temperature, "temperature", torch.float32, (n,)),
        _dev(uniform, "uniform", torch.float32, (n,)), _dev(out, "picks", torch.int32, (n,)),
        n, vocab, _stream()), "sample_rows")
    return out


def fill_f32(t: torch.Tensor, value: float) -> torch.Tensor:
    _check(library().imparo_fill_f32(_dev(t, "fill target", torch.float32), float(value), t.numel(), _stream()),
           "fill_f32")
    return t


def fill_sites(base: torch.Tensor, per_slot: torch.Tensor, value: torch.Tensor, slot: int) -> None:
    """Sets one slot's row of every fixed-state site in one launch: site i's row is per_slot[i]
    float32 values at address base[i] + slot * per_slot[i] * 4 and becomes value[i] everywhere."""
    n = base.shape[0]
    _check(library().imparo_fill_sites(_dev(base, "site addresses", torch.int64, (n,)),
                                       _dev(per_slot, "site row sizes", torch.int64, (n,)),
                                       _dev(value, "site values", torch.float32, (n,)), n, int(slot), _stream()),
           "fill_sites")


# ------------------------------------------------------------------ grouped norm, token shift, sinusoid, polynomial
def embed_sinusoid(table: torch.Tensor, ids: torch.Tensor, positions: torch.Tensor, inv_freq: torch.Tensor,
                   out: torch.Tensor) -> torch.Tensor:
    """out[t] = table[ids[t]] + the sinusoidal vector of positions[t]: entry 2i is sin(pos * inv_freq[i]),
    entry 2i + 1 the cosine of the same angle."""
    vocab, width = table.shape
    n = ids.shape[0]
    _check(library().imparo_embed_sinusoid(
        _dev(table, "embedding table"), _code(table, "embedding table"), _dev(ids, "token ids", torch.int32, (n,)),
        _dev(positions, "positions", torch.int32, (n,)), _dev(inv_freq, "inverse frequencies", torch.float32, ((width + 1) // 2,)),
        _dev(out, "embedding output", torch.float32, (n, width)), n, width, vocab, _stream()), "embed_sinusoid")
    return out


def group_rms_norm(x: torch.Tensor, weight: torch.Tensor, groups: int, eps: float, out: torch.Tensor,
                   delta: Optional[torch.Tensor] = None, rows: Optional[torch.Tensor] = None, write_back: bool = False,
                   shift_mix: Optional[torch.Tensor] = None, shift_state: Optional[torch.Tensor] = None,
                   slot: Optional[torch.Tensor] = None) -> torch.Tensor:
    """`rms_norm` with the row in `groups` equal consecutive parts, each divided by its own root mean square.
    With `shift_mix` [width], for rows of one token each (row i's request in slot[i]): out = h + (prev - h) *
    mix, where prev = shift_state[slot[i]] is replaced by h, the normed row."""
    width = x.shape[-1]
    n_out = out.shape[0]
    if groups < 1 or width % groups:
        raise KernelArgumentError(f"group_rms_norm: {width} values do not make {groups} equal parts")
    if rows is None and n_out != x.shape[0]:
        raise KernelArgumentError(f"group_rms_norm: out has {n_out} rows, x has {x.shape[0]}")
    if rows is not None and rows.shape[0] != n_out:
        raise KernelArgumentError("group_rms_norm: one source row index per output row is needed")
    if write_back and (rows is not None or delta is None):
        raise KernelArgumentError("group_rms_norm: write_back needs a delta and no row selection")
    n_delta = 0
    if delta is not None:
        n_delta = delta.shape[0] if delta.dim() == x.dim() + 1 else 1
        want = (n_delta,) + tuple(x.shape) if delta.dim() == x.dim() + 1 else tuple(x.shape)
        _dev(delta, "group_rms_norm delta", torch.float32, want)
    if shift_mix is not None:
        if rows is not None or shift_state is None or slot is None or shift_state.dim() != 2:
            raise KernelArgumentError("group_rms_norm: a token shift needs its state, the rows' slots and no row selection")
        _dev(shift_state, "shift state", torch.float32, (shift_state.shape[0], width))
        _dev(slot, "slot", torch.int32, (n_out,))
    _check(library().imparo_group_rms_norm(
        _dev(x, "group_rms_norm x", torch.float32), _dev(delta, "group_rms_norm delta", torch.float32), n_delta, x.shape[0],
        _dev(rows, "group_rms_norm rows", torch.int32), _dev(weight, "group_rms_norm weight", torch.float32, (width,)),
        _dev(out, "group_rms_norm out", None, (n_out, width)), _code(out, "group_rms_norm out"), n_out, width, int(groups),
        float(eps), int(write_back), _dev(shift_mix, "shift mix", torch.float32, (width,)),
        _dev(shift_state, "shift state", torch.float32), _dev(slot, "slot", torch.int32), _stream()), "group_rms_norm")
    return out


def token_shift(h: torch.Tensor, mix: torch.Tensor, state: torch.Tensor, row_of_token: torch.Tensor,
                seg_start: torch.Tensor, seg_len: torch.Tensor, slot: torch.Tensor, out: torch.Tensor) -> torch.Tensor:
    """out[t] = h[t] + (prev - h[t]) * mix: prev is the row before inside a request's segment and the request's
    state at the segment's first token; the state then becomes the segment's last row of h."""
    n, width = h.shape
    n_rows = seg_start.shape[0]
    _check(library().imparo_token_shift(
        _dev(h, "normed rows", torch.float32), _dev(mix, "shift mix", torch.float32, (width,)),
        _dev(state, "shift state", torch.float32, (state.shape[0], width)),
        _dev(row_of_token, "row_of_token", torch.int32, (n,)), _dev(seg_start, "seg_start", torch.int32, (n_rows,)),
        _dev(seg_len, "seg_len", torch.int32, (n_rows,)), _dev(slot, "slot", torch.int32, (n_rows,)),
        _dev(out, "shifted rows", None, (n, width)), _code(out, "shifted rows"), n, n_rows, width, _stream()), "token_shift")
    return out


def poly_norm(z: torch.Tensor, coef: torch.Tensor, eps: float, out: torch.Tensor, width: Optional[int] = None) -> torch.Tensor:
    """out = a N(z) + b N(z^2) + c N(z^3) + e over the first `width` values of every row of z (default: all),
    N(v) = v / sqrt(mean(v^2) + eps); coef = [a, b, c, e] on the device. Columns of out beyond `width` become zero."""
    n, z_ld = z.shape
    width = z_ld if width is None else int(width)
    if out.shape[0] != n or out.dim() != 2 or out.shape[1] < width or width > z_ld:
        raise KernelArgumentError("poly_norm: the output does not match the rows")
    _check(library().imparo_poly_norm(
        _dev(z, "poly_norm z", torch.float32), z_ld, _dev(coef, "poly_norm coefficients", torch.float32, (4,)),
        _dev(out, "poly_norm out"), _code(out, "poly_norm out"), out.shape[1], n, width, float(eps), _stream()), "poly_norm")
    return out


# ------------------------------------------------------------------ selective state-space mixer
def causal_conv(u: torch.Tensor, channels: int, weight: torch.Tensor, bias: Optional[torch.Tensor],
                state: Optional[torch.Tensor], row_of_token: torch.Tensor, seg_start: torch.Tensor, seg_len: torch.Tensor,
                slot: torch.Tensor, out: torch.Tensor, silu: bool = True, single_tokens: bool = False,
                u_off: int = 0) -> torch.Tensor:
    """Causal per-channel convolution of each request's segment over `channels` columns of u (float32 rows)
    from column `u_off` on, continued from the request's history, which is advanced: state [slots, taps - 1,
    channels] (None with one tap). The last tap is the current token's."""
    n, u_ld = u.shape
    ch, taps = weight.shape
    n_rows = seg_start.shape[0]
    if ch != channels or u_off < 0 or u_ld < u_off + channels:
        raise KernelArgumentError(f"causal_conv: a [{ch}, {taps}] filter does not fit {channels} channels of rows of {u_ld}")
    if taps > 1:
        if state is None:
            raise KernelArgumentError("causal_conv: a filter of more than one tap needs a history")
        _dev(state, "conv history", torch.float32, (state.shape[0], taps - 1, channels))
    _check(library().imparo_causal_conv(
        _dev(u, "conv input", torch.float32) + 4 * int(u_off), u_ld, _dev(weight, "conv weight", torch.float32),
        _dev(bias, "conv bias", torch.float32, (channels,)), _dev(state, "conv history", torch.float32) if taps > 1 else 0,
        _dev(row_of_token, "row_of_token", torch.int32, (n,)), _dev(seg_start, "seg_start", torch.int32, (n_rows,)),
        _dev(seg_len, "seg_len", torch.int32, (n_rows,)), _dev(slot, "slot", torch.int32, (n_rows,)),
        _dev(out, "conv out", None, (n, channels)), _code(out, "conv out"), n, n_rows, channels, taps, int(silu),
        int(single_tokens), _stream()), "causal_conv")
    return out


def selective_scan_chunk() -> int:
    """Tokens per chunk when `selective_scan` walks long segments in chunks side by side."""
    return int(library().imparo_selective_scan_chunk())


def selective_scan_scratch(n_rows: int, n_chunks: int, channels: int, n_state: int) -> int:
    """Floats of scratch that `selective_scan` needs for `n_chunks` > 1."""
    return n_rows * (n_chunks * channels * (n_state + 1) + channels * n_state)


def selective_scan(dt_raw: torch.Tensor, x: torch.Tensor, bc: torch.Tensor, z: torch.Tensor, z_ld: int, A: torch.Tensor,
                   D: torch.Tensor, state: torch.Tensor, seg_start: torch.Tensor, seg_len: torch.Tensor,
                   slot: torch.Tensor, out: torch.Tensor, scratch: Optional[torch.Tensor] = None,
                   n_chunks: int = 1) -> torch.Tensor:
    """The selective scan of every request's segment, continued from its state [slots, channels, n_state]
    (float32), which is advanced. dt_raw [tokens, channels] float32 before softplus (taken in place: the
    array holds the steps afterwards); x and out [tokens,
    channels] in one dtype; bc [tokens, 2 n_state] float32; z a float32 view whose rows lie z_ld apart.
    `n_chunks` > 1 (at least ceil(longest segment / selective_scan_chunk())): the chunks of a segment run
    side by side through `scratch` (selective_scan_scratch floats); the caller knows the longest segment."""
    n, channels = x.shape
    n_state = A.shape[1]
    n_rows = seg_start.shape[0]
    if z.dtype != torch.float32 or z.device != x.device or z_ld < channels:
        raise KernelArgumentError("selective_scan: z is float32 on the GPU, its rows at least `channels` apart")
    if n_chunks > 1 and (scratch is None or scratch.numel() < selective_scan_scratch(n_rows, n_chunks, channels, n_state)):
        raise KernelArgumentError("selective_scan: the scratch for the chunks' states is too small")
    _check(library().imparo_selective_scan(
        _dev(dt_raw, "dt", torch.float32, (n, channels)), _dev(x, "scan x"), _dev(bc, "B and C", torch.float32, (n, 2 * n_state)),
        z.data_ptr(), int(z_ld), _dev(A, "A", torch.float32, (channels, n_state)), _dev(D, "D", torch.float32, (channels,)),
        _dev(state, "scan state", torch.float32, (state.shape[0], channels, n_state)),
        _dev(seg_start, "seg_start", torch.int32, (n_rows,)), _dev(seg_len, "seg_len", torch.int32, (n_rows,)),
        _dev(slot, "slot", torch.int32, (n_rows,)), _dev(out, "scan out", x.dtype, (n, channels)), _code(x, "scan x"),
        _dev(scratch, "scan scratch", torch.float32) if n_chunks > 1 else 0, int(n_chunks),
        n, n_rows, channels, n_state, _stream()), "selective_scan")
    return out


# ------------------------------------------------------------------ differential attention
def diff_attention_split() -> int:
    """Keys per split of the differential attention kernel."""
    return int(library().imparo_diff_attention_split())


def diff_qkv_store(rows_in: torch.Tensor, positions: torch.Tensor, row_of_token: torch.Tensor,
                   block_table: Optional[torch.Tensor], page_size: int, q_out: torch.Tensor,
                   k_cache: Optional[torch.Tensor], v_cache: Optional[torch.Tensor], heads: int, kv_heads: int, dim: int,
                   vdim: int, temp_coef: float, temp_every: int) -> torch.Tensor:
    """From the fused projection's float32 rows [q | k | v | ...]: the queries times their position's
    temperature into q_out [tokens, heads, 2, dim]; keys and values into their pages (caches None: not written)."""
    n, ld = rows_in.shape
    write_kv = k_cache is not None
    n_pages, stride = 0, 0
    if write_kv:
        n_pages = k_cache.shape[0]
        _dev(k_cache, "k cache", q_out.dtype, (n_pages, 2 * kv_heads, page_size, dim))
        _dev(v_cache, "v cache", q_out.dtype, (n_pages, kv_heads, page_size, vdim))
        if block_table is None or block_table.dim() != 2:
            raise KernelArgumentError("diff_qkv_store: a [rows, pages] block table is needed to write the cache")
        stride = block_table.shape[1]
    _check(library().imparo_diff_qkv_store(
        _dev(rows_in, "projection rows", torch.float32), ld, _dev(positions, "positions", torch.int32, (n,)),
        _dev(row_of_token, "row_of_token", torch.int32, (n,)), _dev(block_table, "block table", torch.int32) if write_kv else 0,
        stride, page_size, _dev(q_out, "q out", None, (n, heads, 2, dim)), _dev(k_cache, "k cache"), _dev(v_cache, "v cache"),
        _code(q_out, "q out"), int(write_kv), n, heads, kv_heads, dim, vdim, n_pages, float(temp_coef), int(temp_every),
        _stream()), "diff_qkv_store")
    return q_out


def diff_attention(q: torch.Tensor, k_cache: torch.Tensor, v_cache: torch.Tensor, gate: Optional[torch.Tensor],
                   gate_ld: int, out: torch.Tensor, positions: torch.Tensor, row_of_token: torch.Tensor,
                   block_table: torch.Tensor, scale: float, window: Optional[int], lam: float, eps: float,
                   out_scale: float, part: Optional[torch.Tensor] = None, n_splits: int = 1,
                   seg_len: Optional[torch.Tensor] = None, below: int = 0) -> torch.Tensor:
    """Differential attention of every token over its request's cached keys (see imparo_diff_attention).
    `below` > 0: only the tokens of rows that bring fewer than that many tokens (`seg_len` per row)."""
    n, heads, two, dim = q.shape
    n_pages, kv2, page_size, kdim = k_cache.shape
    kv_heads, vdim = v_cache.shape[1], v_cache.shape[3]
    if two != 2 or kdim != dim or kv2 != 2 * kv_heads or heads % kv_heads:
        raise KernelArgumentError("diff_attention: queries [tokens, heads, 2, dim], keys [pages, 2 kv_heads, page, dim]")
    _dev(v_cache, "v cache", q.dtype, (n_pages, kv_heads, page_size, vdim))
    if n_splits > 1 and (part is None or part.numel() < n * heads * n_splits * (2 * vdim + 4)):
        raise KernelArgumentError("diff_attention: the scratch for partial results is too small")
    if gate is not None and (gate.dtype != torch.float32 or gate.device != q.device):
        raise KernelArgumentError("diff_attention: the gate's logits are float32 on the GPU")
    _check(library().imparo_diff_attention(
        _dev(q, "q"), _dev(k_cache, "k cache", q.dtype), v_cache.data_ptr(), 0 if gate is None else gate.data_ptr(),
        int(gate_ld), _dev(out, "attention out", q.dtype, (n, heads * vdim)), _dev(part, "partial results", torch.float32),
        _code(q, "q"), _dev(positions, "positions", torch.int32, (n,)), _dev(row_of_token, "row_of_token", torch.int32, (n,)),
        _dev(block_table, "block table", torch.int32), block_table.shape[1], page_size, n, heads, kv_heads, dim, vdim,
        n_pages, float(scale), int(window or 0), float(lam), float(eps), float(out_scale), int(n_splits),
        _dev(seg_len, "seg_len", torch.int32) if below > 0 else 0, int(below), _stream()), "diff_attention")
    return out


def diff_attention_tiles_takes(dtype: torch.dtype, page_size: int, dim: int, vdim: int) -> bool:
    """Whether the matrix-core kernel for portions takes these sizes."""
    return dtype == torch.bfloat16 and bool(library().imparo_diff_attention_tiles_takes(int(page_size), int(dim), int(vdim)))


def diff_attention_tiles(q: torch.Tensor, k_cache: torch.Tensor, v_cache: torch.Tensor, gate: Optional[torch.Tensor],
                         gate_ld: int, out: torch.Tensor, positions: torch.Tensor, seg_start: torch.Tensor,
                         seg_len: torch.Tensor, max_seg_len: int, block_table: torch.Tensor, scale: float,
                         window: Optional[int], lam: float, eps: float, out_scale: float, min_len: int = 1) -> torch.Tensor:
    """Differential attention on the matrix cores for the rows that bring at least `min_len` tokens (bfloat16;
    sizes as diff_attention_tiles_takes says); the other rows' outputs are left as they are."""
    n, heads, two, dim = q.shape
    n_pages, kv2, page_size, kdim = k_cache.shape
    kv_heads, vdim = v_cache.shape[1], v_cache.shape[3]
    n_rows = seg_start.shape[0]
    if two != 2 or kdim != dim or kv2 != 2 * kv_heads or heads % kv_heads:
        raise KernelArgumentError("diff_attention_tiles: queries [tokens, heads, 2, dim], keys [pages, 2 kv_heads, page, dim]")
    if not diff_attention_tiles_takes(q.dtype, page_size, dim, vdim):
        raise KernelArgumentError(f"diff_attention_tiles: bfloat16, pages of a multiple of 16, dim and vdim multiples of 4 "
                                  f"up to 128; got {q.dtype}, pages of {page_size}, {dim} and {vdim}")
    if gate is not None and (gate.dtype != torch.float32 or gate.device != q.device):
        raise KernelArgumentError("diff_attention_tiles: the gate's logits are float32 on the GPU")
    _check(library().imparo_diff_attention_tiles(
        _dev(q, "q", torch.bfloat16), _dev(k_cache, "k cache", torch.bfloat16),
        _dev(v_cache, "v cache", torch.bfloat16, (n_pages, kv_heads, page_size, vdim)), 0 if gate is None else gate.data_ptr(),
        int(gate_ld), _dev(out, "attention out", torch.bfloat16, (n, heads * vdim)), _dev(positions, "positions", torch.int32, (n,)),
        _dev(seg_start, "seg_start", torch.int32, (n_rows,)), _dev(seg_len, "seg_len", torch.int32, (n_rows,)),
        _dev(block_table, "block table", torch.int32), block_table.shape[1], page_size, n_rows, int(max_seg_len), heads,
        kv_heads, dim, vdim, n_pages, float(scale), int(window or 0), float(lam), float(eps), float(out_scale),
        int(min_len), _stream()), "diff_attention_tiles")
    return out


# ---------------------------------------------------------------- routed feed-forward, norm on a sublayer's result
MOE_EPILOGUES = {None: 0, "none": 0, "relu2": 1}
MOE_SCORINGS = {"softmax": 0, "sigmoid": 1}


def _route_rules(logits: torch.Tensor, n_router: Optional[int], groups: int, keep: int, normalize: bool, scale: float):
    """The router outputs among a token's logits and the rules of the choice, as the kernels take them."""
    r = logits.shape[1] if n_router is None else int(n_router)
    if not 1 <= r <= logits.shape[1]:
        raise KernelArgumentError(f"moe_route: {r} router outputs in rows of {logits.shape[1]} logits")
    groups = int(groups or 1)
    if groups < 1 or groups > 64 or r % groups or (groups > 1 and not 1 <= keep <= groups):
        raise KernelArgumentError(f"moe_route: {r} outputs in {groups} groups of which {keep} stay")
    return r, (logits.shape[1], groups, int(keep or 1), int(bool(normalize)), float(scale))


def moe_route(logits: torch.Tensor, correction: Optional[torch.Tensor], choice: torch.Tensor, weight: torch.Tensor,
              top: int, scoring: str = "softmax", n_router: Optional[int] = None, groups: int = 1, keep: int = 1,
              normalize: bool = False, scale: float = 1.0) -> None:
    """choice[t] = the `top` router outputs with the largest score + correction, weight[t] their scores (as
    they are); scores are softmax(logits[t]) or, with scoring "sigmoid", the sigmoid of each output.
    `n_router`: only the first so many columns of `logits` are router outputs. `groups` > 1: the outputs form
    that many equal groups of neighbours, a group scores the sum of its two largest score + correction, and
    only the `keep` best groups' outputs can be chosen. `normalize`: the chosen scores are divided by their
    sum (+ 1e-20); `scale` multiplies the weights at the end."""
    n = logits.shape[0]
    r, rules = _route_rules(logits, n_router, groups, keep, normalize, scale)
    _check(library().imparo_moe_route(
        _dev(logits, "router logits", torch.float32), _dev(correction, "router correction", torch.float32, (r,)),
        _dev(choice, "choice", torch.int32, (n, top)), _dev(weight, "choice weights", torch.float32, (n, top)),
        n, r, top, MOE_SCORINGS[scoring], *rules, _stream()), "moe_route")


def moe_gated(gu: torch.Tensor, weight: Optional[torch.Tensor], entry_of_slot: Optional[torch.Tensor],
              hidden: torch.Tensor) -> torch.Tensor:
    """hidden[slot, j] = silu(w g) * (w u) with g = gu[slot, j], u = gu[slot, half + j] and w the weight of the
    slot's entry (weight None: 1)."""
    n, two = gu.shape
    half = two // 2
    if two != 2 * half or tuple(hidden.shape) != (n, half):
        raise KernelArgumentError(f"moe_gated: gu is {tuple(gu.shape)}, hidden {tuple(hidden.shape)}")
    if weight is not None and (entry_of_slot is None or weight.numel() < n or entry_of_slot.numel() < n):
        raise KernelArgumentError("moe_gated: a weight and an entry per slot are needed")
    _check(library().imparo_moe_gated(
        _dev(gu, "gate and up products", torch.float32), _dev(weight, "choice weights", torch.float32),
        _dev(entry_of_slot, "entry_of_slot", torch.int32), _dev(hidden, "hidden"), _code(hidden, "hidden"),
        n, half, _stream()), "moe_gated")
    return hidden


def moe_route_plan_tokens() -> int:
    """The most tokens `moe_route_plan` takes."""
    return int(library().imparo_moe_route_plan_tokens())


def moe_route_plan(logits: torch.Tensor, correction: Optional[torch.Tensor], choice: torch.Tensor, weight: torch.Tensor,
                   top: int, n_experts: int, tile_rows: int, slot_of_entry: torch.Tensor, entry_of_slot: torch.Tensor,
                   tiles: torch.Tensor, scoring: str = "softmax", n_router: Optional[int] = None, groups: int = 1,
                   keep: int = 1, normalize: bool = False, scale: float = 1.0) -> None:
    """`moe_route` and `moe_plan` in one launch, for the few tokens of a decode step."""
    n = logits.shape[0]
    r, rules = _route_rules(logits, n_router, groups, keep, normalize, scale)
    _dev(slot_of_entry, "slot_of_entry", torch.int32, (n * top,))
    _dev(entry_of_slot, "entry_of_slot", torch.int32, (n * top,))
    _check(library().imparo_moe_route_plan(
        _dev(logits, "router logits", torch.float32), _dev(correction, "router correction", torch.float32, (r,)),
        _dev(choice, "choice", torch.int32, (n, top)), _dev(weight, "choice weights", torch.float32, (n, top)),
        n, r, top, MOE_SCORINGS[scoring], n_experts, tile_rows, slot_of_entry.data_ptr(), entry_of_slot.data_ptr(),
        _dev(tiles, "tiles", torch.int32), tiles.shape[0], *rules, _stream()), "moe_route_plan")


def moe_tile_rows(n_entries: int, n_experts: int, dtype: torch.dtype) -> int:
    return int(library().imparo_moe_tile_rows(int(n_entries), int(n_experts), 0 if dtype == torch.float32 else 1))


def moe_max_tiles(n_entries: int, n_experts: int, tile_rows: int) -> int:
    return int(library().imparo_moe_max_tiles(int(n_entries), int(n_experts), int(tile_rows)))


def moe_plan(choice: torch.Tensor, n_experts: int, tile_rows: int, slot_of_entry: torch.Tensor,
             entry_of_slot: torch.Tensor, tiles: torch.Tensor) -> None:
    n_entries = choice.numel()
    _dev(slot_of_entry, "slot_of_entry", torch.int32, (n_entries,))
    _dev(entry_of_slot, "entry_of_slot", torch.int32, (n_entries,))
    _check(library().imparo_moe_plan(
        _dev(choice, "choice", torch.int32), n_entries, n_experts, tile_rows, slot_of_entry.data_ptr(),
        entry_of_slot.data_ptr(), _dev(tiles, "tiles", torch.int32), tiles.shape[0], _stream()), "moe_plan")


def moe_gemm(a: torch.Tensor, w: torch.Tensor, out: torch.Tensor, tiles: torch.Tensor, tile_rows: int,
             entry_of_slot: Optional[torch.Tensor] = None, gather_div: int = 0, epilogue: Optional[str] = None) -> torch.Tensor:
    """out[slot] = epilogue(a[row(slot)] . w[expert of the slot's tile]^T); w is [experts, n, k]."""
    n_experts, n, k = w.shape
    if a.dim() != 2 or a.shape[1] != k or a.dtype != w.dtype:
        raise KernelArgumentError(f"moe_gemm: a is {tuple(a.shape)} {a.dtype}, the experts' matrices {tuple(w.shape)} {w.dtype}")
    if out.dim() != 2 or out.shape[1] != n:
        raise KernelArgumentError(f"moe_gemm: out is {tuple(out.shape)}, {n} columns are needed")
    if gather_div == 0 and a.shape[0] < out.shape[0]:
        raise KernelArgumentError("moe_gemm: fewer input rows than slots")
    if epilogue not in MOE_EPILOGUES:
        raise KernelArgumentError(f"moe_gemm: unknown epilogue {epilogue!r}")
    if tiles.dim() != 2 or tiles.shape[1] != 3:
        raise KernelArgumentError("moe_gemm: tiles is [max_tiles, 3]")
    _check(library().imparo_moe_gemm(
        _dev(a, "moe_gemm a"), a.stride(0), int(gather_div), _dev(entry_of_slot, "entry_of_slot", torch.int32),
        _dev(w, "experts' matrices"), _dev(out, "moe_gemm out"), _code(out, "moe_gemm out"), _code(w, "experts' matrices"),
        _dev(tiles, "tiles", torch.int32), tiles.shape[0], int(tile_rows), n, k, MOE_EPILOGUES[epilogue], _stream()),
        "moe_gemm")
    return out


def moe_combine(y: torch.Tensor, h: torch.Tensor, choice: torch.Tensor, weight: Optional[torch.Tensor],
                slot_of_entry: torch.Tensor, n_experts: int, out: torch.Tensor) -> torch.Tensor:
    """out[t] = the sum over a token's choices of weight * (its expert's row, or h[t] for an expert past the
    last real one); weight None: every weight is 1."""
    n, top = choice.shape
    width = h.shape[1]
    _check(library().imparo_moe_combine(
        _dev(y, "experts' results", torch.float32), _dev(h, "feed-forward input", None, (n, width)), _code(h, "input"),
        _dev(choice, "choice", torch.int32), _dev(weight, "choice weights", torch.float32, (n, top)),
        _dev(slot_of_entry, "slot_of_entry", torch.int32, (n * top,)), _dev(out, "combined", torch.float32, (n, width)),
        n, width, top, n_experts, _stream()), "moe_combine")
    return out


def post_norm_add(x: torch.Tensor, delta, w_post: torch.Tensor, eps_post: float,
                  w_next: Optional[torch.Tensor] = None, eps_next: float = 0.0, out: Optional[torch.Tensor] = None,
                  rows: Optional[torch.Tensor] = None) -> Optional[torch.Tensor]:
    """x += rms_norm(delta) * w_post (delta shaped like x, or [slices, *x.shape], added in order); with
    `w_next`, out = rms_norm(x) * w_next; with `out` and no `w_next`, out = the new x itself in out's dtype.
    With `rows` only those rows are taken, into out, and x stays.
    `delta` may be what a routed feed-forward left to be combined (an object with y, h, choice, weight,
    slot_of_entry, n_experts): the launch then makes moe_combine's sum itself."""
    n_x, width = x.shape
    n_out = n_x if rows is None else rows.shape[0]
    if not isinstance(delta, torch.Tensor):
        top = delta.choice.shape[1]
        if delta.weight is None:
            raise KernelArgumentError("post_norm_add: the experts' sum inside this launch needs the choice's weights")
        if (w_next is not None or out is not None) and (out is None or tuple(out.shape) != (n_out, width)):
            raise KernelArgumentError("post_norm_add: the next norm needs an output of one row per taken row")
        if out is None and rows is not None:
            raise KernelArgumentError("post_norm_add: a row selection without an output has no result")
        _check(library().imparo_post_norm_add_moe(
            _dev(x, "stream", torch.float32), _dev(delta.y, "experts' results", torch.float32),
            _dev(delta.h, "feed-forward input", None, (n_x, width)), _code(delta.h, "feed-forward input"),
            _dev(delta.choice, "choice", torch.int32, (n_x, top)), _dev(delta.weight, "choice weights", torch.float32, (n_x, top)),
            _dev(delta.slot_of_entry, "slot_of_entry", torch.int32, (n_x * top,)), top, int(delta.n_experts), n_x,
            _dev(rows, "rows", torch.int32), _dev(w_post, "post norm weight", torch.float32, (width,)), float(eps_post),
            _dev(w_next, "next norm weight", torch.float32, (width,)), float(eps_next),
            _dev(out, "normed"), _code(out, "normed") if out is not None else 0,
            n_out, width, _stream()), "post_norm_add")
        return out
    n_delta = delta.shape[0] if delta.dim() == 3 else 1
    _dev(delta, "sublayer result", torch.float32, ((n_delta, n_x, width) if delta.dim() == 3 else (n_x, width)))
    if w_next is not None or out is not None:
        if out is None or tuple(out.shape) != (n_out, width):
            raise KernelArgumentError("post_norm_add: the next norm needs an output of one row per taken row")
    elif rows is not None:
        raise KernelArgumentError("post_norm_add: a row selection without an output has no result")
    _check(library().imparo_post_norm_add(
        _dev(x, "stream", torch.float32), delta.data_ptr(), n_delta, n_x, _dev(rows, "rows", torch.int32),
        _dev(w_post, "post norm weight", torch.float32, (width,)), float(eps_post),
        _dev(w_next, "next norm weight", torch.float32, (width,)), float(eps_next),
        _dev(out, "normed"), _code(out, "normed") if out is not None else 0,
        n_out, width, _stream()), "post_norm_add")
    return out


# ---------------------------------------------------------------- attention over a cached latent
def latent_store(q_rows: torch.Tensor, kv_rows: torch.Tensor, norm_weight: torch.Tensor, eps: float,
                 inv_freq: Optional[torch.Tensor], interleaved: bool, positions: torch.Tensor, row_of_token: torch.Tensor,
                 block_table: Optional[torch.Tensor], page_size: int, cache: Optional[torch.Tensor], q_plain: torch.Tensor,
                 q_full: torch.Tensor, heads: int, dim: int, rot_dim: int, rank: int,
                 cache_t: Optional[torch.Tensor] = None) -> None:
    """The latent's norm, the rotation of the shared key part and of every head's rotated query part, the write
    of [latent | rotated key part] into the token's page, and the queries laid out for the absorbed products.
    `cache_t` [pages, rank, page]: the latent is written there once more, transposed inside the page."""
    n = q_rows.shape[0]
    n_freq = 0 if inv_freq is None else inv_freq.shape[0]
    n_pages = table_stride = 0
    if cache is not None:
        n_pages = cache.shape[0]
        _dev(cache, "latent cache", q_full.dtype, (n_pages, page_size, rank + rot_dim))
        if block_table is None or block_table.dim() != 2:
            raise KernelArgumentError("latent_store: a [rows, pages] block table is needed to write the cache")
        table_stride = block_table.shape[1]
        if cache_t is not None:
            _dev(cache_t, "transposed latents", q_full.dtype, (n_pages, rank, page_size))
    elif cache_t is not None:
        raise KernelArgumentError("latent_store: the transposed latents are written with the rows only")
    _check(library().imparo_latent_store(
        _dev(q_rows, "query rows", torch.float32, (n, heads * (dim + rot_dim))),
        _dev(kv_rows, "latent rows", torch.float32, (n, rank + rot_dim)),
        _dev(norm_weight, "latent norm weight", torch.float32, (rank,)), float(eps),
        _dev(inv_freq, "inverse frequencies", torch.float32), n_freq, int(interleaved),
        _dev(positions, "positions", torch.int32, (n,)), _dev(row_of_token, "row_of_token", torch.int32, (n,)),
        _dev(block_table, "block table", torch.int32), table_stride, page_size, n_pages, _dev(cache, "latent cache"),
        _dev(cache_t, "transposed latents"), _dev(q_plain, "unrotated queries", q_full.dtype, (n, heads, dim)),
        _dev(q_full, "queries", None, (n, heads, rank + rot_dim)), _code(q_full, "queries"),
        n, heads, dim, rot_dim, rank, _stream()), "latent_store")


def head_gemm(x: torch.Tensor, w: torch.Tensor, out: torch.Tensor, out_columns: Optional[int] = None) -> torch.Tensor:
    """out[t, h, :n] = W[h] x[t, h, :] with w [heads, k, n] (an up-projection of its own per head); x [tokens,
    heads, k]; out [tokens, heads, n], or wider rows a head of which the first n columns are written."""
    T, H, K = x.shape
    Hw, Kw, N = w.shape
    if (Hw, Kw) != (H, K) or x.dtype != w.dtype:
        raise KernelArgumentError(f"head_gemm: x is {tuple(x.shape)} {x.dtype}, the weights {tuple(w.shape)} {w.dtype}")
    if out.dim() != 3 or out.shape[0] != T or out.shape[1] != H or out.shape[2] < N:
        raise KernelArgumentError(f"head_gemm: out is {tuple(out.shape)}; [{T}, {H}, at least {N}] is needed")
    _check(library().imparo_head_gemm(
        _dev(x, "head_gemm x"), H * K, K, _dev(w, "head_gemm weights"), _code(x, "head_gemm x"),
        _dev(out, "head_gemm out"), _code(out, "head_gemm out"), H * out.shape[2], out.shape[2], T, H, K, N, _stream()),
        "head_gemm")
    return out


def head_gemm_tiles_takes(dtype: torch.dtype, k: int) -> bool:
    """Whether the matrix-core form of the per-head product takes inputs of this dtype and inner size."""
    return dtype == torch.bfloat16 and k >= 8 and k % 8 == 0


def head_gemm_tiles(x: torch.Tensor, w_t: torch.Tensor, out: torch.Tensor) -> torch.Tensor:
    """head_gemm on the matrix cores: x [tokens, heads, k] bfloat16, w_t [heads, n, k] bfloat16 (a head's matrix
    with the inner size running fastest); out [tokens, heads, at least n] bfloat16 or float32."""
    T, H, K = x.shape
    Hw, N, Kw = w_t.shape
    if (Hw, Kw) != (H, K) or not head_gemm_tiles_takes(x.dtype, K) or w_t.dtype != torch.bfloat16:
        raise KernelArgumentError(f"head_gemm_tiles: x is {tuple(x.shape)} {x.dtype}, the weights {tuple(w_t.shape)} {w_t.dtype}")
    if out.dim() != 3 or out.shape[0] != T or out.shape[1] != H or out.shape[2] < N:
        raise KernelArgumentError(f"head_gemm_tiles: out is {tuple(out.shape)}; [{T}, {H}, at least {N}] is needed")
    _check(library().imparo_head_gemm_tiles(
        _dev(x, "head_gemm x", torch.bfloat16), H * K, K, _dev(w_t, "head_gemm weights", torch.bfloat16),
        _dev(out, "head_gemm out"), _code(out, "head_gemm out"), H * out.shape[2], out.shape[2], T, H, K, N, _stream()),
        "head_gemm_tiles")
    return out


def attention_latent(q: torch.Tensor, cache: torch.Tensor, out: torch.Tensor, positions: torch.Tensor,
                     row_of_token: torch.Tensor, block_table: torch.Tensor, value_dim: int, scale: float,
                     window: Optional[int]) -> torch.Tensor:
    """Attention in which all heads read the same cached rows: a key is a whole row, its value the row's
    first `value_dim` numbers. One wave per (token, head); float32 or bfloat16."""
    n, heads, row_dim = q.shape
    n_pages, page_size, rd = cache.shape
    if rd != row_dim or value_dim > row_dim:
        raise KernelArgumentError(f"attention_latent: q has rows of {row_dim}, the cache of {rd}, values of {value_dim}")
    _check(library().imparo_attention_latent(
        _dev(q, "q"), _dev(cache, "latent cache", q.dtype), _dev(out, "attention out", q.dtype, (n, heads * value_dim)),
        _code(q, "q"), _dev(positions, "positions", torch.int32, (n,)), _dev(row_of_token, "row_of_token", torch.int32, (n,)),
        _dev(block_table, "block table", torch.int32), block_table.shape[1], page_size, n, heads, row_dim, value_dim,
        n_pages, float(scale), int(window or 0), _stream()), "attention_latent")
    return out


def attention_latent_tiles_takes(dtype: torch.dtype, row_dim: int, rank: int, page_size: int) -> bool:
    """Whether the matrix-core kernel over cached latents is built for these sizes."""
    if dtype != torch.bfloat16 or page_size < 32 or page_size & (page_size - 1):
        return False
    if rank < 8 or rank > 256 or rank % 8 or row_dim % 8 or row_dim < rank:
        return False
    value_tiles = 2 if rank <= 32 else 4 if rank <= 64 else 8 if rank <= 128 else 16
    return (row_dim + 31) // 32 <= value_tiles // 2 + 2


def attention_latent_tiles_split(n_tokens: int, heads: int, max_context: int):
    """(parts the keys of such a launch are cut into, keys a part)."""
    keys = ctypes.c_int(0)
    n = int(library().imparo_attention_latent_tiles_split(int(n_tokens), int(heads), int(max_context), ctypes.byref(keys)))
    return n, int(keys.value)


def attention_latent_tiles(q: torch.Tensor, cache: torch.Tensor, cache_t: torch.Tensor, out: torch.Tensor,
                           positions: torch.Tensor, row_of_token: torch.Tensor, block_table: torch.Tensor, scale: float,
                           window: Optional[int], n_splits: int = 1, split_keys: int = 0,
                           part_o: Optional[torch.Tensor] = None, part_ml: Optional[torch.Tensor] = None,
                           exact: bool = True) -> torch.Tensor:
    """attention_latent on the matrix cores (bfloat16): up to 16 heads of a token share a wave and every tile
    of keys. `cache_t` [pages, rank, page] holds the latents transposed inside a page; the values are the
    latents. `n_splits`, `split_keys` from attention_latent_tiles_split for a context bound that holds for every
    token; with n_splits > 1 `part_o` (tokens * heads * n_splits * rank) and `part_ml` (tokens * heads * n_splits
    * 2) float32 hold the parts. `exact`: the softmax weights keep float32's precision through the second product."""
    n, heads, row_dim = q.shape
    n_pages, page_size, rd = cache.shape
    rank = cache_t.shape[1]
    if rd != row_dim or not attention_latent_tiles_takes(q.dtype, row_dim, rank, page_size):
        raise KernelArgumentError(f"attention_latent_tiles: rows of {row_dim} (cache {rd}), latents of {rank}, pages of "
                                  f"{page_size}, {q.dtype} are not taken")
    if n_splits > 1:
        if part_o is None or part_ml is None or part_o.numel() < n * heads * n_splits * rank or part_ml.numel() < n * heads * n_splits * 2:
            raise KernelArgumentError("attention_latent_tiles: the buffers for the parts are missing or too small")
    _check(library().imparo_attention_latent_tiles(
        _dev(q, "q", torch.bfloat16), _dev(cache, "latent cache", torch.bfloat16),
        _dev(cache_t, "transposed latents", torch.bfloat16, (n_pages, rank, page_size)),
        _dev(out, "attention out", torch.bfloat16, (n, heads * rank)),
        _dev(part_o, "part_o", torch.float32) if n_splits > 1 else None,
        _dev(part_ml, "part_ml", torch.float32) if n_splits > 1 else None,
        _dev(positions, "positions", torch.int32, (n,)), _dev(row_of_token, "row_of_token", torch.int32, (n,)),
        _dev(block_table, "block table", torch.int32), block_table.shape[1], page_size, n_pages, n, heads, row_dim, rank,
        float(scale), int(window or 0), int(split_keys), int(n_splits), int(bool(exact)), _stream()), "attention_latent_tiles")
    return out


# ---------------------------------------------------------------- gated linear recurrence
def hgrn2_scan(rows: torch.Tensor, q_off: int, f_off: int, v_off: int, lower: torch.Tensor, state: torch.Tensor,
               seg_start: torch.Tensor, seg_len: torch.Tensor, slot: torch.Tensor, out: torch.Tensor, heads: int,
               dim: int, vdim: int, chunk_tokens: int = 0, max_chunks: int = 0,
               chunk_state: Optional[torch.Tensor] = None, chunk_decay: Optional[torch.Tensor] = None) -> torch.Tensor:
    """Per request and head, token by token: S <- diag(f) S + (1 - f) v^T, out = S^T q with q = silu(zq),
    f = lower + (1 - lower) sigmoid(zf); rows holds zq, zf, v at the given columns. With `chunk_tokens`
    (hgrn2_chunks) segments are walked in chunks side by side: `max_chunks` bounds the chunks of the longest,
    `chunk_state` (rows * max_chunks * heads * dim * vdim) and `chunk_decay` (rows * max_chunks * heads * dim)
    float32 are scratch."""
    n, ld = rows.shape
    R = seg_start.shape[0]
    if chunk_tokens:
        if (chunk_state is None or chunk_decay is None or chunk_state.numel() < R * max_chunks * heads * dim * vdim
                or chunk_decay.numel() < R * max_chunks * heads * dim):
            raise KernelArgumentError("hgrn2_scan: the scratch for the chunks is missing or too small")
        _dev(chunk_state, "chunk states", torch.float32)
        _dev(chunk_decay, "chunk decays", torch.float32)
    _check(library().imparo_hgrn2_scan(
        _dev(rows, "recurrence inputs", torch.float32), ld, q_off, f_off, v_off,
        _dev(lower, "lower bounds", torch.float32, (heads * dim,)),
        _dev(state, "recurrent state", torch.float32, (state.shape[0], heads, dim, vdim)),
        _dev(seg_start, "seg_start", torch.int32, (R,)), _dev(seg_len, "seg_len", torch.int32, (R,)),
        _dev(slot, "slot", torch.int32, (R,)), _dev(out, "recurrence out", torch.float32, (n, heads * vdim)),
        R, heads, dim, vdim, int(chunk_tokens), int(max_chunks),
        chunk_state.data_ptr() if chunk_tokens else None, chunk_decay.data_ptr() if chunk_tokens else None,
        _stream()), "hgrn2_scan")
    return out


def hgrn2_chunks(max_seg_len: int):
    """(tokens a chunk, chunks of the longest segment) for a step whose longest segment has `max_seg_len`
    tokens; (0, 0): too short to pay for three launches. At most 32 chunks a segment."""
    if max_seg_len < 256:
        return 0, 0
    tokens = max(128, (-(-max_seg_len // 32) + 7) // 8 * 8)
    return tokens, -(-max_seg_len // tokens)


# ---------------------------------------------------------------- a parallel block's elementwise pieces
def gated_sum(x: torch.Tensor, a: torch.Tensor, b: Optional[torch.Tensor], gates: torch.Tensor,
              copy: Optional[torch.Tensor] = None) -> torch.Tensor:
    """x += a * sigmoid(gates[:, :width]) (+ b * sigmoid(gates[:, width:])); `copy` also receives the new x.
    a and b are shaped like x, or [slices, *x.shape]: sums over parts of a product's inner size, added in order."""
    n, width = x.shape
    slices = lambda t: 1 if t is None or t.dim() == 2 else t.shape[0]
    shaped = lambda t: (n, width) if t.dim() == 2 else (t.shape[0], n, width)
    _check(library().imparo_gated_sum(
        _dev(x, "stream", torch.float32), _dev(a, "first sublayer's result", torch.float32, shaped(a)), slices(a),
        _dev(b, "second sublayer's result", torch.float32, None if b is None else shaped(b)), slices(b),
        _dev(gates, "gates", torch.float32, (n, 2 * width if b is not None else gates.shape[1])), gates.shape[1],
        _dev(copy, "stream copy", None, (n, width)), _code(copy, "stream copy") if copy is not None else 0,
        n, width, _stream()), "gated_sum")
    return x


def side_gate(z: torch.Tensor, table: torch.Tensor, offset: int, ids: torch.Tensor, out: torch.Tensor) -> torch.Tensor:
    """out[t, j] = gelu_tanh(z[t, j]) * table[ids[t], offset + j]; columns beyond z's width become zero."""
    n, dim = z.shape
    vocab, table_ld = table.shape
    _check(library().imparo_side_gate(
        _dev(z, "side gate", torch.float32), _dev(table, "side table"), _code(table, "side table"), table_ld, offset,
        _dev(ids, "token ids", torch.int32, (n,)), vocab, _dev(out, "gated side input", None, (n, out.shape[1])),
        _code(out, "gated side input"), n, dim, out.shape[1], _stream()), "side_gate")
    return out


def add_rows(x: torch.Tensor, y: torch.Tensor) -> torch.Tensor:
    """x += y, both float32 of one shape."""
    _check(library().imparo_add_rows(_dev(x, "x", torch.float32), _dev(y, "y", torch.float32, tuple(x.shape)),
                                     x.numel(), _stream()), "add_rows")
    return x


# ---------------------------------------------------------------- recurrences with one decay a head and token
DECAY_SCAN_MAX_DIM = 512          # state rows a head
DECAY_SCAN_CHUNK = 64             # tokens a chunk when a long segment's chunks run side by side


def decay_scan_chunks(max_seg_len: int, delta: bool = False, dim: int = 0, blocks: int = 0):
    """(chunk_tokens, max_chunks) for `decay_scan`: (0, 1) for one launch, which short segments take. Heads of up
    to the chunk form's largest dim: a segment's chunks in order, small products a chunk (the form the delta rule
    needs, and the faster one for a plain decay too where it fills the chip). Wider heads with a plain decay: chunks
    of DECAY_SCAN_CHUNK tokens side by side; wider heads of the delta rule: token by token."""
    chunk = int(library().imparo_delta_chunk_tokens())
    # `blocks`: segments x heads x runs of 8 value columns, the most blocks the chunks-in-order form can make. Where
    # that does not fill the chip, a plain decay's long segments run their chunks side by side instead.
    side_by_side = not delta and 0 < blocks < 256 and max_seg_len >= 4 * DECAY_SCAN_CHUNK
    if dim <= int(library().imparo_delta_chunk_max_dim()) and not side_by_side:
        if max_seg_len < 2 * chunk:
            return 0, 1
        return chunk, -(-int(max_seg_len) // chunk)
    if delta or max_seg_len < 4 * DECAY_SCAN_CHUNK:
        return 0, 1
    return DECAY_SCAN_CHUNK, -(-int(max_seg_len) // DECAY_SCAN_CHUNK)


def decay_scan_scratch(n_rows: int, max_chunks: int, heads: int, dim: int, vdim: int, chunk_tokens: int):
    """Floats of (chunk_state, chunk_decay) that `decay_scan` needs when it walks in chunks of `chunk_tokens`."""
    chunk = int(library().imparo_delta_chunk_tokens())
    if chunk_tokens == chunk:
        return n_rows * max_chunks * heads * 2 * chunk * chunk, n_rows * max_chunks * heads * 2 * chunk
    return n_rows * max_chunks * heads * dim * vdim, n_rows * max_chunks * heads


def decay_scan(q: torch.Tensor, q_off: int, q_div: int, k: torch.Tensor, k_off: int, k_div: int, v: torch.Tensor,
               v_off: int, state: torch.Tensor, seg_start: torch.Tensor, seg_len: torch.Tensor, slot: torch.Tensor,
               out: torch.Tensor, heads: int, dim: int, vdim: int, decay_const: Optional[torch.Tensor] = None,
               step: Optional[torch.Tensor] = None, step_off: int = 0, step_bias: Optional[torch.Tensor] = None,
               rate: Optional[torch.Tensor] = None, v_times_step: bool = False, beta: Optional[torch.Tensor] = None,
               beta_off: int = 0, skip: Optional[torch.Tensor] = None, chunk_tokens: int = 0, max_chunks: int = 1,
               chunk_state: Optional[torch.Tensor] = None, chunk_decay: Optional[torch.Tensor] = None) -> torch.Tensor:
    """Per request, head and token in order: S <- a S + k v^T, out = S^T q; with `beta` the gated delta rule
    S <- a S, u = sigmoid(beta) (v - S^T k), S <- S + k u^T, out = S^T q. q, k, v, step, beta are float32 row
    tensors [tokens, ld] read from a column offset on (they may be one tensor); head h reads q head h // q_div
    and k head h // k_div. a = decay_const[h] or exp(-rate[h] softplus(step[t, h] + step_bias[h])); with
    `v_times_step` v is multiplied by that softplus; with `skip`, out += skip[h] v. state [slots, heads, dim,
    vdim] float32 is carried on; out [tokens, heads * vdim] float32."""
    n = out.shape[0]
    n_rows = seg_start.shape[0]
    if dim > DECAY_SCAN_MAX_DIM:
        raise KernelArgumentError(f"decay_scan: up to {DECAY_SCAN_MAX_DIM} state rows a head, got {dim}")
    for t, what in ((q, "q"), (k, "k"), (v, "v"), (step, "step"), (beta, "beta")):
        if t is not None and (t.dim() != 2 or t.shape[0] != n):
            raise KernelArgumentError(f"decay_scan: {what} is not a row tensor of {n} tokens")
    if (decay_const is None) == (step is None):
        raise KernelArgumentError("decay_scan: the decay is a constant a head or comes from projected steps")
    if chunk_tokens:
        need_s, need_d = decay_scan_scratch(n_rows, max_chunks, heads, dim, vdim, chunk_tokens)
        if chunk_state is None or chunk_decay is None or chunk_state.numel() < need_s or chunk_decay.numel() < need_d:
            raise KernelArgumentError("decay_scan: the scratch for the chunks' states is too small")
    _check(library().imparo_decay_scan(
        _dev(q, "scan q", torch.float32), q.shape[1], int(q_off), int(q_div),
        _dev(k, "scan k", torch.float32), k.shape[1], int(k_off), int(k_div),
        _dev(v, "scan v", torch.float32), v.shape[1], int(v_off),
        _dev(decay_const, "decays", torch.float32, (heads,)),
        _dev(step, "steps", torch.float32), 0 if step is None else step.shape[1], int(step_off),
        _dev(step_bias, "step bias", torch.float32, (heads,)) if step is not None else 0,
        _dev(rate, "decay rates", torch.float32, (heads,)) if step is not None else 0, int(bool(v_times_step)),
        _dev(beta, "beta", torch.float32), 0 if beta is None else beta.shape[1], int(beta_off),
        _dev(skip, "skip weights", torch.float32, (heads,)),
        _dev(state, "scan state", torch.float32, (state.shape[0], heads, dim, vdim)),
        _dev(seg_start, "seg_start", torch.int32, (n_rows,)), _dev(seg_len, "seg_len", torch.int32, (n_rows,)),
        _dev(slot, "slot", torch.int32, (n_rows,)), _dev(out, "scan out", torch.float32, (n, heads * vdim)),
        n_rows, heads, dim, vdim, int(chunk_tokens), int(max_chunks),
        _dev(chunk_state, "chunk states", torch.float32) if chunk_tokens else 0,
        _dev(chunk_decay, "chunk decays", torch.float32) if chunk_tokens else 0, _stream()), "decay_scan")
    return out


def head_prepare(rows: torch.Tensor, off: int, heads: int, dim: int, unit: bool = False, unit_eps: float = 0.0,
                 inv_freq: Optional[torch.Tensor] = None, interleaved: bool = False,
                 positions: Optional[torch.Tensor] = None, n_first: int = 0, scale_first: float = 1.0,
                 scale_rest: float = 1.0) -> torch.Tensor:
    """In place on float32 rows [tokens, ld]: each of the `heads` heads of `dim` columns from `off` on is made a
    unit vector (x / sqrt(sum x^2 + unit_eps)) if `unit`, its first 2 len(inv_freq) dimensions are rotated by the
    token's position (pairs (i, i + half), or neighbours if `interleaved`), and it is multiplied by scale_first
    (heads below n_first) or scale_rest."""
    n, ld = rows.shape
    n_freq = 0 if inv_freq is None else inv_freq.shape[0]
    if off < 0 or off + heads * dim > ld or 2 * n_freq > dim:
        raise KernelArgumentError(f"head_prepare: {heads} heads of {dim} from column {off} in rows of {ld}, {n_freq} rotated pairs")
    _check(library().imparo_head_prepare(
        _dev(rows, "rows", torch.float32), ld, int(off), n, heads, dim, int(bool(unit)), float(unit_eps),
        _dev(inv_freq, "inverse frequencies", torch.float32), n_freq, int(bool(interleaved)),
        _dev(positions, "positions", torch.int32, (n,)) if n_freq else 0, int(n_first), float(scale_first),
        float(scale_rest), _stream()), "head_prepare")
    return rows


def gated_group_norm(x: torch.Tensor, gate: Optional[torch.Tensor], gate_off: int, weight: Optional[torch.Tensor],
                     groups: int, eps: float, out: torch.Tensor, gate_first: bool) -> torch.Tensor:
    """A row of x (float32 [tokens, width]) in `groups` equal parts, g = silu(gate[t, gate_off + c]):
    gate_first: (x g) / rms_part(x g) * weight; otherwise x / rms_part(x) * weight * g. weight [width] or None."""
    n, width = x.shape
    if gate is not None and (gate.dim() != 2 or gate.shape[0] != n or gate_off + width > gate.shape[1]):
        raise KernelArgumentError("gated_group_norm: the gate's rows do not hold the row's width from its offset on")
    _check(library().imparo_gated_group_norm(
        _dev(x, "heads' results", torch.float32), _dev(gate, "gate", torch.float32), 0 if gate is None else gate.shape[1],
        int(gate_off), _dev(weight, "norm weight", torch.float32, (width,)), _dev(out, "normed", None, (n, width)),
        _code(out, "normed"), n, width, int(groups), float(eps), int(bool(gate_first)), _stream()), "gated_group_norm")
    return out


def clamped_glu(gu: torch.Tensor, out: torch.Tensor, hidden: int, limit: float, alpha: float) -> torch.Tensor:
    """out[t, j] = g sigmoid(alpha g) (u + 1) with g = min(gu[t, j], limit), u = clamp(gu[t, hidden + j], -limit,
    limit); out may be wider than `hidden` (its further columns are zero)."""
    n = gu.shape[0]
    if gu.shape[1] != 2 * hidden or out.shape[0] != n or out.shape[1] < hidden:
        raise KernelArgumentError(f"clamped_glu: gu is {tuple(gu.shape)}, out {tuple(out.shape)}, hidden {hidden}")
    _check(library().imparo_clamped_glu(_dev(gu, "gate and up", torch.float32), _dev(out, "hidden"), _code(out, "hidden"),
                                        n, int(hidden), out.shape[1], float(limit), float(alpha), _stream()), "clamped_glu")
    return out


def normed_sum(a: torch.Tensor, wa: torch.Tensor, b: torch.Tensor, wb: torch.Tensor, eps: float, factor: float,
               out: torch.Tensor) -> torch.Tensor:
    """out = factor (rms_norm(a) wa + rms_norm(b) wb); a and b float32 [tokens, width] or [slices, tokens, width]
    (slices are added in order first)."""
    n, width = out.shape
    sa = a.shape[0] if a.dim() == 3 else 1
    sb = b.shape[0] if b.dim() == 3 else 1
    _dev(a, "first result", torch.float32, (sa, n, width) if a.dim() == 3 else (n, width))
    _dev(b, "second result", torch.float32, (sb, n, width) if b.dim() == 3 else (n, width))
    _check(library().imparo_normed_sum(a.data_ptr(), sa, _dev(wa, "first weight", torch.float32, (width,)), b.data_ptr(), sb,
                                       _dev(wb, "second weight", torch.float32, (width,)),
                                       _dev(out, "sum", torch.float32), n, width, float(eps), float(factor), _stream()),
           "normed_sum")
    return out


def gated_row_add(out: torch.Tensor, y: torch.Tensor, z: torch.Tensor, z_col: int) -> torch.Tensor:
    """out[t] += sigmoid(z[t, z_col]) * y[t]; y float32 [tokens, width] or [slices, tokens, width]."""
    n, width = out.shape
    sy = y.shape[0] if y.dim() == 3 else 1
    _dev(y, "rows to add", torch.float32, (sy, n, width) if y.dim() == 3 else (n, width))
    if z.dim() != 2 or z.shape[0] != n or not 0 <= z_col < z.shape[1]:
        raise KernelArgumentError("gated_row_add: one gate a token is read from a column of z")
    _check(library().imparo_gated_row_add(_dev(out, "sum", torch.float32), y.data_ptr(), sy, _dev(z, "gates", torch.float32),
                                          z.shape[1], int(z_col), n, width, _stream()), "gated_row_add")
    return out


def cast_rows(x: torch.Tensor, out: torch.Tensor, rows: Optional[torch.Tensor] = None) -> torch.Tensor:
    """out[i] = x[rows[i]] (rows None: x[i]) in out's dtype; x float32 [n, width]."""
    n_out, width = out.shape
    if x.shape[1] != width or (rows is None and x.shape[0] != n_out) or (rows is not None and rows.shape[0] != n_out):
        raise KernelArgumentError(f"cast_rows: x is {tuple(x.shape)}, out {tuple(out.shape)}")
    _check(library().imparo_cast_rows(_dev(x, "rows", torch.float32), _dev(rows, "row choice", torch.int32),
                                      _dev(out, "cast rows"), _code(out, "cast rows"), n_out, width, _stream()), "cast_rows")
    return out
