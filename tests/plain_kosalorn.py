"""A plain, slow statement of the Kosalorn design: float32 (or float64), whole
sequences, no cache, one function per mechanism. It shares no code with the
engine: tests hold the engine against it.

Notation: a sequence is a [tokens, width] matrix; positions count from 0; a
linear weight is [out, in] and applied as x @ W.T.
"""
from __future__ import annotations

import json
import math
import os
from typing import List, Optional

import torch

from plain_tumadra import read_safetensors, rms


def gelu_tanh(z: torch.Tensor) -> torch.Tensor:
    return 0.5 * z * (1.0 + torch.tanh(math.sqrt(2.0 / math.pi) * (z + 0.044715 * z ** 3)))


def silu(z: torch.Tensor) -> torch.Tensor:
    return z * torch.sigmoid(z)


def scalar_norm(x: torch.Tensor, g: torch.Tensor, eps: float) -> torch.Tensor:
    """RMS norm whose weight is one number for the whole row."""
    return rms(x, eps) * g


def frequencies(dims: int, base: float, dtype) -> torch.Tensor:
    i = torch.arange(dims // 2, dtype=torch.float64)
    return torch.pow(torch.tensor(base, dtype=torch.float64), -2.0 * i / dims).to(torch.float32).to(dtype)


def rotate_halves(x: torch.Tensor, positions: torch.Tensor, freq: torch.Tensor) -> torch.Tensor:
    """x [..., tokens, dims] with dims = 2 len(freq): dimension i turns with dimension i + dims/2."""
    half = freq.shape[0]
    angle = positions.to(x.dtype)[:, None] * freq.to(x.dtype)[None, :]
    c, s = torch.cos(angle), torch.sin(angle)
    u, v = x[..., :half], x[..., half:2 * half]
    return torch.cat([u * c - v * s, v * c + u * s, x[..., 2 * half:]], dim=-1)


def rotate_pairs(x: torch.Tensor, positions: torch.Tensor, freq: torch.Tensor) -> torch.Tensor:
    """x [..., tokens, dims]: dimension 2i turns with dimension 2i + 1."""
    half = freq.shape[0]
    angle = positions.to(x.dtype)[:, None] * freq.to(x.dtype)[None, :]
    c, s = torch.cos(angle), torch.sin(angle)
    out = x.clone()
    u, v = x[..., 0:2 * half:2], x[..., 1:2 * half:2]
    out[..., 0:2 * half:2] = u * c - v * s
    out[..., 1:2 * half:2] = v * c + u * s
    return out


def latent_attention(h, positions, w, L: str, mx: dict, eps: float, pairs: bool) -> torch.Tensor:
    """Both latent-attention mixers: keys and values are made from a latent of
    kv_rank numbers a token plus one rotated key part that all heads share.
    `pairs`: the rotation pairs neighbours (2i, 2i + 1) instead of halves."""
    T = h.shape[0]
    H, dn, dr, dv, r = mx["heads"], mx["dim"], mx["rot_dim"], mx["vdim"], mx["kv_rank"]
    if f"{L}.mix.dq" in w:
        cq = rms(h @ w[f"{L}.mix.dq"].T, eps) * w[f"{L}.mix.dq.norm"]
        q = cq @ w[f"{L}.mix.uq"].T
    else:
        q = h @ w[f"{L}.mix.q"].T
    q = q.reshape(T, H, dn + dr)
    ckr = h @ w[f"{L}.mix.dkv"].T
    c = rms(ckr[:, :r], eps) * w[f"{L}.mix.dkv.norm"]
    freq = frequencies(mx["rot"]["dims"], mx["rot"]["base"], h.dtype)
    turn = rotate_pairs if pairs else rotate_halves
    kr = turn(ckr[:, r:], positions, freq)                                # [T, dr], one for all heads
    qr = turn(q[:, :, dn:].transpose(0, 1), positions, freq)             # [H, T, dr]
    kn = (c @ w[f"{L}.mix.uk"].T).reshape(T, H, dn)
    v = (c @ w[f"{L}.mix.uv"].T).reshape(T, H, dv)
    dist = positions[:, None] - positions[None, :]
    seen = dist >= 0
    window = (mx.get("mask") or {}).get("size")
    if window is not None:
        seen = seen & (dist < window)
    out = []
    for hd in range(H):
        s = (q[:, hd, :dn] @ kn[:, hd, :].T + qr[hd] @ kr.T) * mx["scale"]
        s = s.masked_fill(~seen, float("-inf"))
        out.append(torch.softmax(s, dim=-1) @ v[:, hd, :])
    return torch.cat(out, dim=-1) @ w[f"{L}.mix.o"].T


def hgrn2(h, w, L: str, mx: dict, eps: float) -> torch.Tensor:
    """Gated linear recurrence: per head S <- diag(f) S + (1 - f) v^T, o = S^T q."""
    T = h.shape[0]
    H, dk, dv = mx["heads"], mx["dim"], mx["vdim"]
    q = silu(h @ w[f"{L}.mix.q"].T).reshape(T, H, dk)
    v = (h @ w[f"{L}.mix.v"].T).reshape(T, H, dv)
    low = w[f"{L}.mix.lower"]
    f = (low + (1.0 - low) * torch.sigmoid(h @ w[f"{L}.mix.f"].T + w[f"{L}.mix.f.b"])).reshape(T, H, dk)
    S = torch.zeros(H, dk, dv, dtype=h.dtype)
    out = torch.zeros(T, H, dv, dtype=h.dtype)
    for t in range(T):
        S = f[t][:, :, None] * S + (1.0 - f[t])[:, :, None] * v[t][:, None, :]
        out[t] = torch.einsum("hkv,hk->hv", S, q[t])
    out = rms(out, eps) * w[f"{L}.mix.norm"]
    return out.reshape(T, H * dv) @ w[f"{L}.mix.o"].T


def gated_unit(h, gate, up, down) -> torch.Tensor:
    return (silu(h @ gate.T) * (h @ up.T)) @ down.T


def mixture(h, w, L: str, mlp: dict) -> torch.Tensor:
    """Scores are sigmoids of the router's outputs; the `top` largest are chosen;
    a chosen expert reads score * h, and the results are added as they are."""
    scores = torch.sigmoid(h @ w[f"{L}.mlp.router"].T)
    top = mlp["router"]["top"]
    chosen = torch.topk(scores, top, dim=-1).indices
    out = torch.zeros_like(h)
    for t in range(h.shape[0]):
        for e in chosen[t].tolist():
            p = f"{L}.mlp.e{e}"
            out[t] += gated_unit(scores[t, e] * h[t:t + 1], w[p + ".gate"], w[p + ".up"], w[p + ".down"])[0]
    return out


def token_side(x, tokens, w, L: str, i: int, dim: int, eps: float) -> torch.Tensor:
    """The layer's own small embedding of the token, gated by the stream, projected, normed, added."""
    e = w["side.embed"][tokens][:, i * dim:(i + 1) * dim]
    y = (gelu_tanh(x @ w[f"{L}.side.gate"].T) * e) @ w[f"{L}.side.proj"].T
    return x + rms(y, eps) * w[f"{L}.side.norm"]


def run_order(cfg: dict) -> List[tuple]:
    """(layer, first of a later pass) in the order the layers run."""
    n = len(cfg["layers"])
    loop = cfg.get("loop") or dict(start=0, stop=0, times=1)
    order = [(i, False) for i in range(loop["start"])]
    for p in range(loop["times"]):
        order += [(i, p > 0 and i == loop["start"]) for i in range(loop["start"], loop["stop"])]
    return order + [(i, False) for i in range(loop["stop"], n)]


class PlainKosalorn:
    def __init__(self, model_dir: str, dtype=torch.float32):
        with open(os.path.join(model_dir, "config.json")) as f:
            self.cfg = json.load(f)
        self.dtype = dtype
        self.w = {k: (v if v.dtype == torch.int32 else v.to(dtype))
                  for k, v in read_safetensors(os.path.join(model_dir, "model.safetensors")).items()}

    def forward(self, tokens: List[int], layers_out: Optional[list] = None) -> torch.Tensor:
        """Logits [tokens, vocab]; `layers_out` collects the stream after every layer run."""
        cfg, w = self.cfg, self.w
        eps = cfg["norm"]["eps"]
        T = len(tokens)
        ids = torch.tensor(tokens)
        positions = torch.arange(T)
        x = scalar_norm(w["embed"][ids], w["embed.norm"], eps)
        first = x.clone()
        side = cfg.get("token_side")
        for i, again in run_order(cfg):
            layer, L = cfg["layers"][i], f"l{i}"
            mx = layer["mixer"]
            if again:
                x = x + first
            h = scalar_norm(x, w[f"{L}.norm1"], eps)
            if layer["type"] == "hgrn2":
                m = hgrn2(h, w, L, mx, eps)
            else:
                m = latent_attention(h, positions, w, L, mx, eps, pairs=layer["type"] == "latent_attention_2")
            delta = m * torch.sigmoid(h @ w[f"{L}.rg1"].T + w[f"{L}.rg1.b"])
            mlp = layer.get("mlp")
            if mlp is not None:
                if mlp["kind"] == "dense":
                    f = gated_unit(h, w[f"{L}.mlp.gate"], w[f"{L}.mlp.up"], w[f"{L}.mlp.down"])
                else:
                    f = mixture(h, w, L, mlp)
                delta = delta + f * torch.sigmoid(h @ w[f"{L}.rg2"].T + w[f"{L}.rg2.b"])
            x = x + delta
            if side is not None:
                x = token_side(x, ids, w, L, i, side["dim"], eps)
            if layers_out is not None:
                layers_out.append(x.clone())
        return scalar_norm(x, w["final.norm"], eps) @ w["head"].T

    def logits(self, tokens: List[int], order=None) -> torch.Tensor:
        return self.forward(list(tokens)).to(torch.float32)

    def greedy(self, prompt: List[int], n: int) -> List[int]:
        tokens, out = list(prompt), []
        for _ in range(n):
            out.append(int(self.forward(tokens)[-1].argmax()))
            tokens.append(out[-1])
        return out
