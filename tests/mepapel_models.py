"""Small Mepapel configurations with random weights, for tests. The weights are drawn so that every
mechanism matters: projections of unit gain, conv taps of unit size, norm weights away from one, biases,
decays and steps that spread, routers whose scores spread and a correction that changes choices; the queries
of the recurrences are drawn near their keys (see `near` below)."""
import json
import math
import os

import torch


def mamba2(heads, vdim, state, conv, groups=None, norm_groups=None):
    m = dict(heads=heads, vdim=vdim, state=state, conv=conv)
    if groups is not None:
        m["groups"] = groups
    if norm_groups is not None:
        m["norm_groups"] = norm_groups
    return dict(type="mamba2", mixer=m)


def delta(heads, kv_heads, dim, vdim, conv):
    return dict(type="delta", mixer=dict(heads=heads, kv_heads=kv_heads, dim=dim, vdim=vdim, conv=conv))


def left(heads, kv_heads, dim, vdim, scale=None, mask=None, rot=None, base=10000.0, conv=None):
    m = dict(heads=heads, kv_heads=kv_heads, dim=dim, vdim=vdim, scale=scale if scale is not None else 1.0 / math.sqrt(dim))
    if mask is not None:
        m["mask"] = dict(size=mask)
    if rot is not None:
        m["rot"] = dict(dims=rot, base=base)
    if conv is not None:
        m["conv"] = conv
    return m


def right(heads, dim, vdim, decay, rot=None, base=10000.0):
    m = dict(heads=heads, dim=dim, vdim=vdim, decay=list(decay))
    if rot is not None:
        m["rot"] = dict(dims=rot, base=base)
    return m


def parallel(l, r):
    return dict(type="parallel", mixer=dict(left=l, right=r))


def dense(ff, limit):
    return dict(kind="dense", ff=ff, limit=limit)


def moe(ff, experts, top, groups=None, scale=None, shared=None):
    router = dict(experts=experts, top=top)
    if groups is not None:
        router["groups"] = dict(count=groups[0], keep=groups[1])
    if scale is not None:
        router["scale"] = scale
    out = dict(kind="moe", expert=dict(ff=ff), router=router)
    if shared is not None:
        out["shared"] = dict(ff=shared)
    return out


def layer(mixer, mlp):
    return dict(mixer, mlp=mlp)


# A: every mixer; a rotation of part of a head; three groups of experts of which two stay; a layer without
# feed-forward; experts without groups, shared expert or scale; heads that share queries, keys, B and C
CONFIG_A = dict(
    architecture="Mepapel", vocab=200, width=64, norm=dict(eps=1e-6), residual_mult=0.5,
    layers=[
        layer(parallel(left(4, 2, 16, 16, scale=0.3, mask=24, rot=8, base=500.0, conv=3),
                       right(2, 16, 24, [0.9, 0.97], rot=16)), moe(24, 6, 2, groups=(3, 2), scale=1.5, shared=24)),
        layer(delta(4, 2, 16, 24, 4), dense(40, 1.0)),
        layer(mamba2(4, 16, 24, 2, groups=2, norm_groups=2), None),
        layer(delta(2, 2, 8, 8, 3), moe(16, 4, 1)),
    ])

# B: values that a model may happen to make equal or 1: no multiplier in the file, one head, one state row, one
# tap, no conv, no mask, no rotation, a decay of one, a mask of one position, groups of two experts of which one stays
CONFIG_B = dict(
    architecture="Mepapel", vocab=300, width=96, norm=dict(eps=1e-5),
    layers=[
        layer(mamba2(1, 32, 1, 1), dense(100, 3.0)),
        layer(parallel(left(1, 1, 24, 40, scale=0.2), right(1, 8, 8, [1.0])), dense(64, 0.5)),
        layer(delta(3, 1, 32, 16, 2), moe(40, 8, 2, groups=(4, 1), scale=2.5, shared=16)),
        layer(parallel(left(6, 3, 16, 16, mask=1, rot=16, base=100.0, conv=2),
                       right(3, 16, 32, [0.5, 0.99, 0.999], rot=8)), None),
    ])

# C: sizes that are no multiples of 8 (heads, keys, values, states, hidden widths), masks and taps that cut pages
CONFIG_C = dict(
    architecture="Mepapel", vocab=70, width=40, norm=dict(eps=1e-4), residual_mult=0.8,
    layers=[
        layer(delta(3, 3, 12, 10, 4), dense(28, 0.7)),
        layer(parallel(left(3, 1, 12, 20, mask=5, rot=4, base=50.0, conv=4), right(3, 20, 12, [0.8, 0.9, 0.95], rot=6, base=50.0)),
              moe(10, 3, 2, shared=12)),
        layer(mamba2(3, 12, 20, 3, groups=3, norm_groups=3), dense(20, 2.0)),
    ])

# D: sizes like a real model's layers in small: heads of 64 on the matrix cores, a mask of 100, states of 128 rows,
# a row of 640 values normed whole, sixteen experts in four groups of which two stay
CONFIG_D = dict(
    architecture="Mepapel", vocab=500, width=128, norm=dict(eps=2e-5), residual_mult=0.4,
    layers=[
        layer(parallel(left(4, 2, 64, 64, scale=0.1, mask=100, rot=64, base=5e5, conv=4),
                       right(2, 64, 128, [0.97, 0.999], rot=32, base=5e5)), moe(32, 16, 4, groups=(4, 2), scale=1.8, shared=64)),
        layer(mamba2(10, 64, 128, 4), dense(256, 7.0)),
        layer(delta(4, 2, 128, 64, 4), dense(192, 2.5)),
    ])

CONFIGS = {"A": (CONFIG_A, 41), "B": (CONFIG_B, 42), "C": (CONFIG_C, 43), "D": (CONFIG_D, 44)}
# How wide the routers are drawn: where many experts are chosen the scores lie further apart, so that bfloat16's
# rounding of the router's input turns few near-ties.
ROUTER_GAIN = {"D": 5.0}


def random_weights(config, seed, gain=1.0, router_gain=1.5):
    g = torch.Generator().manual_seed(seed)
    E, V = config["width"], config["vocab"]
    randn = lambda *shape: torch.randn(*shape, generator=g)
    rand = lambda *shape: torch.rand(*shape, generator=g)
    matrix = lambda out, inn: randn(out, inn) * (gain / math.sqrt(inn))
    weight = lambda n: 0.5 + rand(n)
    t = {"embed": randn(V, E), "final.norm": weight(E), "head": randn(V, E) / math.sqrt(E)}

    def near(a, b):
        # A recurrence's first token gives (k . q) u, which the norm behind the heads stretches to unit size: where
        # k . q happens to lie near zero, its sign, a matter of rounding, decides the token's result. The queries
        # are drawn near the keys, so that this dot product stays away from zero and float32 runs can be held to
        # the float32 bound at every row.
        t[a] = 0.8 * t[b] + 0.6 * t[a]

    def unit(p, F):
        t[p + ".gate"], t[p + ".up"], t[p + ".down"] = matrix(F, E), matrix(F, E), matrix(E, F)

    for i, l in enumerate(config["layers"]):
        p, m = f"l{i}", l["mixer"]
        t[f"{p}.norm1"] = weight(E)
        x = f"{p}.mix"
        if l["type"] == "mamba2":
            H, P, N, G, L = m["heads"], m["vdim"], m["state"], m.get("groups", 1), m["conv"]
            C = H * P + 2 * G * N
            t[f"{x}.in"] = matrix(H * P + C + H, E)
            t[f"{x}.conv"], t[f"{x}.conv.b"] = randn(C, L) * (0.8 / math.sqrt(L)), 0.3 * randn(C)
            t[f"{x}.dt_bias"], t[f"{x}.A_log"], t[f"{x}.D"] = randn(H), 0.7 * randn(H) - 1.0, weight(H)
            t[f"{x}.norm"], t[f"{x}.o"] = weight(H * P), matrix(E, H * P)
        elif l["type"] == "delta":
            H, Hk, dk, dv, L = m["heads"], m["kv_heads"], m["dim"], m["vdim"], m["conv"]
            for n, rows in (("q", Hk * dk), ("k", Hk * dk), ("v", H * dv)):
                t[f"{x}.{n}"], t[f"{x}.{n}.conv"] = matrix(rows, E), randn(rows, L) * (1.2 / math.sqrt(L))
            near(f"{x}.q", f"{x}.k")
            near(f"{x}.q.conv", f"{x}.k.conv")
            t[f"{x}.b"], t[f"{x}.a"] = matrix(H, E), matrix(H, E)
            t[f"{x}.A_log"], t[f"{x}.dt_bias"] = 0.7 * randn(H) - 1.5, randn(H)
            t[f"{x}.g"], t[f"{x}.norm"], t[f"{x}.o"] = matrix(H * dv, E), weight(dv), matrix(E, H * dv)
        else:
            a, b = m["left"], m["right"]
            H, G, d, dv = a["heads"], a["kv_heads"], a["dim"], a["vdim"]
            for n, rows in (("q", H * d), ("k", G * d), ("v", G * dv)):
                t[f"{x}.left.{n}"], t[f"{x}.left.{n}.b"] = matrix(rows, E), 0.3 * randn(rows)
                if a.get("conv"):
                    t[f"{x}.left.{n}.conv"] = randn(rows, a["conv"]) * (1.0 / math.sqrt(a["conv"]))
            t[f"{x}.left.q.norm"], t[f"{x}.left.k.norm"] = weight(d), weight(d)
            t[f"{x}.left.o"], t[f"{x}.left.o.b"] = matrix(E, H * dv), 0.3 * randn(E)
            H, d, dv = b["heads"], b["dim"], b["vdim"]
            t[f"{x}.right.q"], t[f"{x}.right.k"] = matrix(H * d, E), matrix(H * d, E)
            near(f"{x}.right.q", f"{x}.right.k")
            t[f"{x}.right.v"], t[f"{x}.right.g"], t[f"{x}.right.o"] = matrix(H * dv, E), matrix(H * dv, E), matrix(E, H * dv)
            t[f"{x}.left.out"], t[f"{x}.right.out"] = weight(E), weight(E)
        mlp = l["mlp"]
        if mlp is None:
            continue
        t[f"{p}.norm2"] = weight(E)
        if mlp["kind"] == "dense":
            unit(f"{p}.mlp", mlp["ff"])
        else:
            X = mlp["router"]["experts"]
            t[f"{p}.mlp.router"], t[f"{p}.mlp.correction"] = matrix(X, E) * router_gain, 0.3 * randn(X)
            for e in range(X):
                unit(f"{p}.mlp.e{e}", mlp["expert"]["ff"])
            if mlp.get("shared") is not None:
                unit(f"{p}.mlp.shared", mlp["shared"]["ff"])
                t[f"{p}.mlp.shared.sg"] = matrix(1, E)
    return t


def write_model(config, seed, out_dir, gain=1.0, overrides=None, router_gain=1.5):
    """Writes config.json and model.safetensors (bfloat16) and returns the folder."""
    from imparo_amd.weights.safetensors_io import save_file
    tensors = random_weights(config, seed, gain, router_gain)
    tensors.update(overrides or {})
    os.makedirs(out_dir, exist_ok=True)
    with open(os.path.join(out_dir, "config.json"), "w") as f:
        json.dump(config, f)
    save_file({k: v.to(torch.bfloat16).contiguous() for k, v in tensors.items()},
              os.path.join(out_dir, "model.safetensors"))
    return out_dir
