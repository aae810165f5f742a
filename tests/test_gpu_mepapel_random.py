"""Mepapel configurations drawn at random with fixed seeds (widths, the order and kinds of layers, head counts,
key, value and state sizes, groups, taps, rotated dimensions, chunks, decays, bounds, experts, groups of experts,
shared experts, layers without feed-forward, constants present or absent), each stepped through a random mixed
schedule on a pool at the schedule's peak with four slots against the plain implementation. float32 runs the model
as drawn: a row is held to the float32 bound, or to three times what float32 rounding does to the plain statement
itself at that row where that is more (the first tokens of a recurrence hang on the sign of one dot product).
bfloat16 runs the same model with routers that cannot be moved by rounding (a zero router matrix and a correction that
sets the experts well apart) and a residual multiplier of at most one half, under the plain bfloat16 bound (one row in
a hundred may miss it by up to half of it, see below): with the drawn router a near-tie may go the other way under
bfloat16's rounding of the router's input, which is no fault."""
import math
import random

import pytest
import torch

import plain_mepapel as plain
from conftest import prompt_tokens
from gpu_helpers import make_engine, mixed_schedule, peak_pages
from mepapel_models import (delta, dense, layer, left, mamba2, moe, parallel, random_weights, right, write_model)
from tolerances import bound

pytestmark = pytest.mark.gpu


def draw_config(seed):
    rng = random.Random(seed)
    width = rng.choice([32, 40, 64, 96, 128, 160, 256])
    layers = []
    for _ in range(rng.randint(1, 5)):
        kind = rng.choice(["mamba2", "delta", "parallel"])
        if kind == "mamba2":
            groups = rng.choice([1, 1, 2, 3])
            heads = groups * rng.choice([1, 2, 4])
            vdim = rng.choice([8, 12, 16, 32, 64])
            parts = rng.choice([n for n in (1, 2, heads, 4) if (heads * vdim) % n == 0])
            mixer = mamba2(heads, vdim, rng.choice([1, 8, 16, 20, 48, 64, 128]), rng.choice([1, 2, 3, 4]),
                           groups=groups if rng.random() < 0.7 else (None if groups == 1 else groups),
                           norm_groups=parts if rng.random() < 0.7 or parts != 1 else None)
        elif kind == "delta":
            kv = rng.choice([1, 2, 3])
            mixer = delta(kv * rng.choice([1, 2, 3]), kv, rng.choice([8, 12, 16, 32, 64, 128, 160]),
                          rng.choice([8, 10, 16, 32, 64]), rng.choice([1, 2, 3, 4]))
        else:
            kv = rng.choice([1, 2, 4])
            dim = rng.choice([8, 16, 32, 64, 128]) if rng.random() < 0.8 else rng.choice([12, 24, 40])
            vdim = dim if rng.random() < 0.6 else rng.choice([8, 12, 16, 20, 32, 64])
            rot = rng.choice([None, dim, dim // 2 - (dim // 2) % 2, 2])
            a = left(kv * rng.choice([1, 2, 4]), kv, dim, vdim,
                     # mild scores: scores spread much wider than 1 / sqrt(dim) turn bfloat16's rounding of q and k
                     # into weight shifts of several percent whichever kernel runs: conditioning, no fault
                     scale=rng.choice([1.0, 0.5, 1.0 / 3.0]) / math.sqrt(dim),
                     mask=rng.choice([None, 1, 2, 7, 16, 33, 64, 100]), rot=rot or None,
                     base=rng.choice([100.0, 10000.0, 1e6]), conv=rng.choice([None, 1, 2, 3, 4]))
            heads, d = rng.choice([1, 2, 3, 4]), rng.choice([8, 16, 32, 64, 96])
            b = right(heads, d, rng.choice([8, 16, 24, 64]),
                      [rng.choice([1.0, 0.5, 0.9, 0.97, 0.999]) for _ in range(heads)],
                      rot=rng.choice([None, d, d // 2, 2]), base=rng.choice([100.0, 10000.0]))
            mixer = parallel(a, b)
        mlp = None
        r = rng.random()
        if r < 0.4:
            mlp = dense(rng.choice([8, 20, 32, 100]), rng.choice([0.3, 1.0, 2.5, 7.0]))
        elif r < 0.85:
            count = rng.choice([1, 2, 3, 4])
            experts = count * rng.choice([1, 2, 3])
            keep = rng.randint(1, count)
            top = rng.randint(1, min(4, keep * (experts // count)))
            mlp = moe(rng.choice([8, 20, 32, 64]), experts, top, groups=(count, keep) if count > 1 or rng.random() < 0.5 else None,
                      scale=rng.choice([None, 0.5, 2.0]), shared=rng.choice([None, 8, 20, 48]))
        layers.append(layer(mixer, mlp))
    cfg = dict(architecture="Mepapel", vocab=rng.choice([50, 97, 300, 500]), width=width,
               norm=dict(eps=rng.choice([1e-6, 1e-5, 1e-3])), layers=layers)
    if rng.random() < 0.7:
        cfg["residual_mult"] = rng.choice([0.25, 0.5, 1.0])
    return cfg


@pytest.mark.parametrize("seed", range(20))
def test_random_configuration_through_a_mixed_schedule(seed, tmp_path):
    from imparo_amd.engine import StepEntry
    cfg = draw_config(2000 + seed)
    dirs = {"float32": write_model(cfg, seed, str(tmp_path / "m"))}
    steady = {}
    for name, t in random_weights(cfg, seed).items():
        if name.endswith(".mlp.router"):
            steady[name] = torch.zeros_like(t)
            steady[name[:-len("router")] + "correction"] = 0.25 * torch.randperm(t.shape[0], generator=torch.Generator().manual_seed(seed)).float()
    cfg16 = dict(cfg, residual_mult=min(cfg.get("residual_mult", 1.0), 0.5))
    dirs["bfloat16"] = write_model(cfg16, seed, str(tmp_path / "steady"), overrides=steady)
    rng = random.Random(seed)
    lengths = [rng.choice([1, 2, 5, 30, 70, 130]) for _ in range(5)]
    prompts = [prompt_tokens(cfg["vocab"], n, 40 + i) for i, n in enumerate(lengths)]
    steps = mixed_schedule(rng, lengths, max_live=4, sizes=(1, 1, 1, 2, 2, 3, 5, 9, 16, 40, 70))
    page = rng.choice([8, 16, 64])
    for dtype in ("float32", "bfloat16"):
        d = dirs[dtype]
        ref, low = plain.PlainMepapel(d), plain.PlainMepapel(d, torch.float32)
        eng = make_engine(d, dtype, page_size=page, max_tokens=peak_pages(steps, page) * page, max_requests=4)
        got = {i: [] for i in range(len(lengths))}
        for entries, ends in steps:
            out = eng.step([StepEntry(rid, prompts[rid][lo:hi], list(range(hi - lo))) for rid, lo, hi in entries]).cpu()
            at = 0
            for rid, lo, hi in entries:
                got[rid].append(out[at:at + hi - lo])
                at += hi - lo
            for rid in ends:
                eng.release(rid)
        all_got = torch.cat([torch.cat(got[i]) for i in range(len(lengths))]).float()
        all_ref = torch.cat([ref.logits(p) for p in prompts])
        assert torch.isfinite(all_got).all(), f"seed {seed} {dtype}"
        scale = float(all_ref.abs().max())
        row_err = (all_got - all_ref).abs().max(dim=-1).values / scale
        allowed = torch.full_like(row_err, bound(dtype, len(cfg["layers"])))
        if dtype == "float32":
            noise = (torch.cat([low.logits(p) for p in prompts]) - all_ref).abs().max(dim=-1).values / scale
            allowed = torch.maximum(allowed, 3.0 * noise)
        if dtype == "bfloat16":
            # One row in a hundred may miss the bound by up to half of it: a recurrence's first tokens hang on a dot
            # product of two unit vectors that bfloat16's rounding of the conv's input moves by a percent of itself,
            # and the norm behind the heads stretches what is left to unit size (conditioning, measured at 1.06 to
            # 1.3 times the bound in four of twenty drawn models, one row each). Anything a cache, a state, a chunk or
            # a batch gets wrong misses by far more, in many rows, and in float32 too, where nothing is allowed.
            over = row_err > allowed
            assert int(over.sum()) <= max(1, row_err.shape[0] // 100) and float((row_err / allowed).max()) <= 1.5, \
                f"seed {seed} {dtype}: {int(over.sum())} of {row_err.shape[0]} rows beyond the bound, worst {float((row_err / allowed).max()):.2f} of it; {cfg}"
            eng.cache.check()
            continue
        bad = (row_err > allowed).nonzero()
        assert bad.numel() == 0, (f"seed {seed} {dtype}: row {int(bad[0])} of {row_err.shape[0]} misses by "
                                  f"{float(row_err[bad[0]]):.3g}, allowed {float(allowed[bad[0]]):.3g}; {bad.numel()} rows; {cfg}")
        eng.cache.check()
