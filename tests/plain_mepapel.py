"""A plain, slow statement of the Mepapel design: float64 (or float32), whole
sequences, no cache, one function per mechanism. It shares no code with the
engine: tests hold the engine against it.

Notation: a sequence is a [tokens, width] matrix; positions count from 0; a
linear weight is [out, in] and applied as x @ W.T; `w` maps tensor names to
tensors and `L` is a layer's prefix ("l3").
"""
from __future__ import annotations

import json
import math
import os
import struct
from typing import Dict, List, Optional

import numpy as np
import torch


def read_tensors(path: str, dtype=torch.float64) -> Dict[str, torch.Tensor]:
    """A safetensors file by hand: 8 bytes of length, a JSON header, raw data."""
    with open(path, "rb") as f:
        (n,) = struct.unpack("<Q", f.read(8))
        header = json.loads(f.read(n))
        data = f.read()
    out = {}
    for name, meta in header.items():
        if name == "__metadata__":
            continue
        a, b = meta["data_offsets"]
        raw = np.frombuffer(data[a:b], dtype=np.uint8)
        if meta["dtype"] == "BF16":
            wide = raw.view(np.uint16).astype(np.uint32) << 16
            t = torch.from_numpy(wide.view(np.float32).copy())
        elif meta["dtype"] == "F32":
            t = torch.from_numpy(raw.view(np.float32).copy())
        elif meta["dtype"] == "I32":
            t = torch.from_numpy(raw.view(np.int32).copy())
        else:
            raise ValueError(meta["dtype"])
        t = t.reshape(meta["shape"])
        out[name] = t.to(dtype) if t.is_floating_point() else t
    return out


def silu(z):
    return z * torch.sigmoid(z)


def softplus(z):
    return torch.where(z > 30, z, torch.log1p(torch.exp(torch.clamp(z, max=30.0))))


def unit_rms(x, eps):
    """x divided by its root mean square over the last dimension, eps inside the root."""
    return x / torch.sqrt((x * x).mean(dim=-1, keepdim=True) + eps)


def causal_conv(u, taps_w, bias=None):
    """u [tokens, channels], taps_w [channels, taps]; the last tap is the current token's and
    there are zeros before the start: y_t = sum_j w[:, j] u_(t - taps + 1 + j)."""
    T, C = u.shape
    K = taps_w.shape[1]
    padded = torch.cat([u.new_zeros(K - 1, C), u], dim=0)
    y = u.new_zeros(T, C)
    for j in range(K):
        y = y + padded[j:j + T] * taps_w[:, j]
    return y if bias is None else y + bias


def frequencies(dims: int, base: float, dtype):
    i = torch.arange(dims // 2, dtype=torch.float64)
    return torch.pow(torch.tensor(float(base), dtype=torch.float64), -2.0 * i / dims).to(dtype)


def turn_neighbours(x, positions, dims: int, base: float):
    """x [tokens, heads, dim]: dimension 2i turns with 2i + 1, over the first `dims` dimensions."""
    if not dims:
        return x
    a = positions.to(x.dtype)[:, None, None] * frequencies(dims, base, x.dtype)[None, None, :]
    c, s = torch.cos(a), torch.sin(a)
    out = x.clone()
    u, v = x[..., 0:dims:2], x[..., 1:dims:2]
    out[..., 0:dims:2] = u * c - v * s
    out[..., 1:dims:2] = v * c + u * s
    return out


def turn_halves(x, positions, dims: int, base: float):
    """x [tokens, heads, dim]: dimension i turns with i + dims/2, over the first `dims` dimensions."""
    if not dims:
        return x
    half = dims // 2
    a = positions.to(x.dtype)[:, None, None] * frequencies(dims, base, x.dtype)[None, None, :]
    c, s = torch.cos(a), torch.sin(a)
    u, v = x[..., :half], x[..., half:dims]
    return torch.cat([u * c - v * s, v * c + u * s, x[..., dims:]], dim=-1)


# ---------------------------------------------------------------- mixers

def mamba2(h, w, L: str, mx: dict, eps: float):
    """State-space duality: one decay a head, a state of N x vdim a head."""
    T = h.shape[0]
    H, P, N, G = mx["heads"], mx["vdim"], mx["state"], mx.get("groups", 1)
    inner = H * P
    rows = h @ w[f"{L}.mix.in"].T
    z, xbc, dt = rows[:, :inner], rows[:, inner:2 * inner + 2 * G * N], rows[:, 2 * inner + 2 * G * N:]
    xbc = silu(causal_conv(xbc, w[f"{L}.mix.conv"], w[f"{L}.mix.conv.b"]))
    x = xbc[:, :inner].reshape(T, H, P)
    B = xbc[:, inner:inner + G * N].reshape(T, G, N)
    C = xbc[:, inner + G * N:].reshape(T, G, N)
    dt = softplus(dt + w[f"{L}.mix.dt_bias"])                       # [T, H]
    decay = torch.exp(-torch.exp(w[f"{L}.mix.A_log"]) * dt)          # [T, H]
    S = h.new_zeros(H, N, P)
    y = h.new_zeros(T, H, P)
    per = H // G
    for t in range(T):
        for hd in range(H):
            g = hd // per
            S[hd] = decay[t, hd] * S[hd] + dt[t, hd] * torch.outer(B[t, g], x[t, hd])
            y[t, hd] = S[hd].T @ C[t, g] + w[f"{L}.mix.D"][hd] * x[t, hd]
    y = y.reshape(T, inner) * silu(z)
    parts = mx.get("norm_groups", 1)
    y = unit_rms(y.reshape(T, parts, inner // parts), eps).reshape(T, inner) * w[f"{L}.mix.norm"]
    return y @ w[f"{L}.mix.o"].T


def delta_rule(h, w, L: str, mx: dict, eps: float):
    """Gated delta rule: S <- g S; u = beta (v - S^T k); S <- S + k u^T; o = S^T q."""
    T = h.shape[0]
    H, Hk, dk, dv = mx["heads"], mx["kv_heads"], mx["dim"], mx["vdim"]
    q = silu(causal_conv(h @ w[f"{L}.mix.q"].T, w[f"{L}.mix.q.conv"])).reshape(T, Hk, dk)
    k = silu(causal_conv(h @ w[f"{L}.mix.k"].T, w[f"{L}.mix.k.conv"])).reshape(T, Hk, dk)
    v = silu(causal_conv(h @ w[f"{L}.mix.v"].T, w[f"{L}.mix.v.conv"])).reshape(T, H, dv)
    q = q / torch.sqrt((q * q).sum(-1, keepdim=True) + 1e-6) * dk ** -0.5
    k = k / torch.sqrt((k * k).sum(-1, keepdim=True) + 1e-6)
    beta = torch.sigmoid(h @ w[f"{L}.mix.b"].T)                      # [T, H]
    g = torch.exp(-torch.exp(w[f"{L}.mix.A_log"]) * softplus(h @ w[f"{L}.mix.a"].T + w[f"{L}.mix.dt_bias"]))
    S = h.new_zeros(H, dk, dv)
    o = h.new_zeros(T, H, dv)
    per = H // Hk
    for t in range(T):
        for hd in range(H):
            kk, qq = k[t, hd // per], q[t, hd // per]
            S[hd] = g[t, hd] * S[hd]
            u = beta[t, hd] * (v[t, hd] - S[hd].T @ kk)
            S[hd] = S[hd] + torch.outer(kk, u)
            o[t, hd] = S[hd].T @ qq
    o = unit_rms(o, eps) * w[f"{L}.mix.norm"]
    o = o.reshape(T, H * dv) * silu(h @ w[f"{L}.mix.g"].T)
    return o @ w[f"{L}.mix.o"].T


def masked_attention(q, k, v, positions, scale: float, chunk: Optional[int] = None):
    """Softmax attention of q [T, H, d] over k [T, G, d], v [T, G, dv]: i sees j <= i, and with `chunk`
    only where both lie in the same run of `chunk` positions counted from 0. -> [T, H * dv]."""
    H, G = q.shape[1], k.shape[1]
    i, j = positions[:, None], positions[None, :]
    seen = j <= i
    if chunk is not None:
        seen = seen & (torch.div(i, chunk, rounding_mode="floor") == torch.div(j, chunk, rounding_mode="floor"))
    out = []
    for hd in range(H):
        g = hd // (H // G)
        s = (q[:, hd] @ k[:, g].T) * scale
        s = s.masked_fill(~seen, float("-inf"))
        out.append(torch.softmax(s, dim=-1) @ v[:, g])
    return torch.cat(out, dim=-1)


def chunk_attention(h, positions, w, P: str, mx: dict, eps: float):
    """Softmax attention with biases, a short conv on q, k, v, head norms, rotation of neighbours and a
    mask in chunks: i sees j <= i iff both lie in the same run of mask.size positions."""
    T = h.shape[0]
    H, G, d, dv = mx["heads"], mx["kv_heads"], mx["dim"], mx["vdim"]

    def proj(n):
        y = h @ w[f"{P}.{n}"].T + w[f"{P}.{n}.b"]
        return causal_conv(y, w[f"{P}.{n}.conv"]) if f"{P}.{n}.conv" in w else y

    q = proj("q").reshape(T, H, d)
    k = proj("k").reshape(T, G, d)
    v = proj("v").reshape(T, G, dv)
    q = unit_rms(q, eps) * w[f"{P}.q.norm"]
    k = unit_rms(k, eps) * w[f"{P}.k.norm"]
    rot = mx.get("rot") or {"dims": 0, "base": 1.0}
    q = turn_neighbours(q, positions, rot["dims"], rot["base"])
    k = turn_neighbours(k, positions, rot["dims"], rot["base"])
    size = (mx.get("mask") or {}).get("size")
    return masked_attention(q, k, v, positions, mx["scale"], size) @ w[f"{P}.o"].T + w[f"{P}.o.b"]


def retention(h, positions, w, P: str, mx: dict, eps: float):
    """Linear attention with one fixed decay a head: S <- decay S + k v^T, o = S^T q."""
    T = h.shape[0]
    H, d, dv = mx["heads"], mx["dim"], mx["vdim"]
    q = (h @ w[f"{P}.q"].T).reshape(T, H, d)
    k = (h @ w[f"{P}.k"].T).reshape(T, H, d)
    v = (h @ w[f"{P}.v"].T).reshape(T, H, dv)
    rot = mx.get("rot") or {"dims": 0, "base": 1.0}
    q = turn_halves(q, positions, rot["dims"], rot["base"])
    k = turn_halves(k, positions, rot["dims"], rot["base"]) * d ** -0.5
    S = h.new_zeros(H, d, dv)
    o = h.new_zeros(T, H, dv)
    decay = torch.tensor(mx["decay"], dtype=h.dtype)
    for t in range(T):
        S = decay[:, None, None] * S + k[t][:, :, None] * v[t][:, None, :]
        o[t] = torch.einsum("hkv,hk->hv", S, q[t])
    o = unit_rms(o, eps).reshape(T, H * dv) * silu(h @ w[f"{P}.g"].T)
    return o @ w[f"{P}.o"].T


def side_by_side(h, positions, w, L: str, mx: dict, eps: float):
    """Both mixers read h; each result is normed over the width with its own weight; half their sum."""
    a = chunk_attention(h, positions, w, f"{L}.mix.left", mx["left"], eps)
    b = retention(h, positions, w, f"{L}.mix.right", mx["right"], eps)
    return 0.5 * (unit_rms(a, eps) * w[f"{L}.mix.left.out"] + unit_rms(b, eps) * w[f"{L}.mix.right.out"])


# ---------------------------------------------------------------- feed-forwards

def clamped_unit(h, w, P: str, limit: float):
    g = torch.clamp(h @ w[f"{P}.gate"].T, max=limit)
    u = torch.clamp(h @ w[f"{P}.up"].T, min=-limit, max=limit)
    return (g * torch.sigmoid(1.702 * g) * (u + 1.0)) @ w[f"{P}.down"].T


def silu_unit(h, w, P: str):
    return (silu(h @ w[f"{P}.gate"].T) * (h @ w[f"{P}.up"].T)) @ w[f"{P}.down"].T


def route(h, w, P: str, router: dict):
    """Per token the chosen experts and their weights."""
    X, top = router["experts"], router["top"]
    s = torch.sigmoid(h @ w[f"{P}.router"].T)
    pick = s + w[f"{P}.correction"] if f"{P}.correction" in w else s.clone()
    groups = router.get("groups")
    if groups is not None:
        n, keep = groups["count"], groups["keep"]
        per = X // n
        grouped = pick.reshape(-1, n, per)
        gscore = torch.topk(grouped, min(2, per), dim=-1).values.sum(-1)        # [T, n]
        best = torch.topk(gscore, keep, dim=-1).indices
        allowed = torch.zeros_like(gscore, dtype=torch.bool).scatter_(1, best, True)
        pick = pick.masked_fill(~allowed[:, :, None].expand(-1, -1, per).reshape(-1, X), float("-inf"))
    chosen = torch.topk(pick, top, dim=-1).indices
    weights = torch.gather(s, 1, chosen)
    weights = weights / (weights.sum(-1, keepdim=True) + 1e-20) * router.get("scale", 1.0)
    return chosen, weights


def mixture(h, w, P: str, mlp: dict):
    chosen, weights = route(h, w, P, mlp["router"])
    out = torch.zeros_like(h)
    for t in range(h.shape[0]):
        for e, a in zip(chosen[t].tolist(), weights[t]):
            out[t] = out[t] + a * silu_unit(h[t:t + 1], w, f"{P}.e{e}")[0]
    if mlp.get("shared") is not None:
        out = out + torch.sigmoid(h @ w[f"{P}.shared.sg"].T) * silu_unit(h, w, f"{P}.shared")
    return out


# ---------------------------------------------------------------- the model

def forward(cfg: dict, w, tokens: List[int], dtype=torch.float64, layers_out: Optional[list] = None):
    """Logits [tokens, vocab] of one sequence from position 0."""
    eps, m = cfg["norm"]["eps"], cfg.get("residual_mult", 1.0)
    positions = torch.arange(len(tokens))
    x = w["embed"][torch.tensor(tokens)].to(dtype)
    for i, layer in enumerate(cfg["layers"]):
        L, kind, mx = f"l{i}", layer["type"], layer["mixer"]
        if kind == "mamba2":
            y = mamba2(x, w, L, mx, eps)
        elif kind == "delta":
            y = delta_rule(x, w, L, mx, eps)
        elif kind == "parallel":
            y = side_by_side(x, positions, w, L, mx, eps)
        else:
            raise ValueError(kind)
        x = x + m * unit_rms(y, eps) * w[f"{L}.norm1"]
        mlp = layer.get("mlp")
        if mlp is not None:
            if mlp["kind"] == "dense":
                y = clamped_unit(x, w, f"{L}.mlp", mlp["limit"])
            else:
                y = mixture(x, w, f"{L}.mlp", mlp)
            x = x + m * unit_rms(y, eps) * w[f"{L}.norm2"]
        if layers_out is not None:
            layers_out.append(x.clone())
    return (unit_rms(x, eps) * w["final.norm"]) @ w["head"].T


class PlainMepapel:
    def __init__(self, model_dir: str, dtype=torch.float64):
        with open(os.path.join(model_dir, "config.json")) as f:
            self.cfg = json.load(f)
        self.dtype = dtype
        self.w = read_tensors(os.path.join(model_dir, "model.safetensors"), dtype)

    def logits(self, tokens: List[int], order=None, layers_out: Optional[list] = None) -> torch.Tensor:
        return forward(self.cfg, self.w, list(tokens), self.dtype, layers_out).to(torch.float32)

    def greedy(self, prompt: List[int], n: int) -> List[int]:
        tokens, out = list(prompt), []
        for _ in range(n):
            nxt = int(self.logits(tokens)[-1].argmax())
            out.append(nxt)
            tokens.append(nxt)
        return out
