"""The Kosalorn configuration reader and plan, on the CPU: what the file's keys become, what is refused,
the run order of a loop, the plain implementation against itself where two statements of one mechanism exist."""
import copy
import math

import pytest
import torch

import plain_kosalorn as plain
from imparo_amd.config import ConfigError, plan_from_config
from imparo_amd.config.errors import BadValue, Inconsistent, MissingKey
from imparo_amd.engine.model import declared_tensors
from kosalorn_models import CONFIGS, layer_runs, random_weights, write_model


@pytest.mark.parametrize("name", sorted(CONFIGS))
def test_plan_declares_the_tensors_the_model_has(name):
    cfg, seed = CONFIGS[name]
    typed, plan = plan_from_config(cfg)
    assert typed.unread_keys == []
    declared = declared_tensors(plan)
    have = random_weights(cfg, seed)
    assert set(declared) == set(have)
    for k, (decl, _) in declared.items():
        assert tuple(decl.shape) == tuple(have[k].shape), k
    assert len(plan.order) == layer_runs(cfg)


def test_plan_of_a():
    typed, plan = plan_from_config(CONFIGS["A"][0])
    # layers 1 and 2 three times in a row; every pass after the first takes the embedding's output in again
    assert [c.layer for c in plan.order] == [0, 1, 2, 1, 2, 1, 2, 3]
    assert [c.add_input for c in plan.order] == [False, False, False, True, False, True, False, False]
    assert all(c.cache_of is None for c in plan.order)
    assert [l.arrangement for l in plan.layers] == ["parallel"] * 4
    assert "ffn" not in plan.layers[2].parts and "ffn_gate" not in plan.layers[2].parts
    m1, m2 = plan.layers[1].mixer, plan.layers[2].mixer
    assert (m1.kind, m1["q_rank"], m1["window"], m1["scale"], m1["position"].kind) == ("latent_attention", 24, 24, 0.3, "rope_neox")
    assert (m2.kind, m2["q_rank"], m2["window"], m2["position"].kind) == ("latent_attention", None, None, "rope_pairs")
    assert plan.layers[0].mixer.kind == "hgrn2" and plan.layers[0].ffn.kind == "swiglu"
    f = plan.layers[1].ffn
    assert (f.kind, f["scoring"], f["weigh"], f["activation"], f["top"]) == ("routed_experts", "sigmoid", "input", "swiglu", 2)
    assert plan.layers[3].side["offset"] == 24 and plan.layers[3].side["table_width"] == 32
    assert plan.embedding["norm"]["scalar"] and plan.final_norm["scalar"]
    _, plan_b = plan_from_config(CONFIGS["B"][0])
    assert "side" not in plan_b.layers[0].parts and not any(c.add_input for c in plan_b.order)
    _, plan_c = plan_from_config(CONFIGS["C"][0])
    assert [c.layer for c in plan_c.order] == [0, 1, 2] and not any(c.add_input for c in plan_c.order)
    assert plan_c.layers[0].mixer["position"]["rotary_dim"] == 4


def _broken(change):
    cfg = copy.deepcopy(CONFIGS["A"][0])
    change(cfg)
    return cfg


@pytest.mark.parametrize("change,error", [
    (lambda c: c.pop("norm"), MissingKey),
    (lambda c: c["layers"][1]["mixer"].pop("kv_rank"), MissingKey),
    (lambda c: c["layers"][1]["mixer"].pop("q_rank"), MissingKey),          # this kind's queries go through a latent
    (lambda c: c["layers"][0]["mixer"].pop("vdim"), MissingKey),
    (lambda c: c["layers"][0].__setitem__("type", "conv"), BadValue),
    (lambda c: c["layers"][0]["mlp"].__setitem__("kind", "poly"), BadValue),
    (lambda c: c["layers"][1]["mlp"].pop("router"), MissingKey),
    (lambda c: c["layers"][1]["mixer"]["rot"].__setitem__("dims", 10), Inconsistent),
    (lambda c: c["layers"][1]["mixer"]["rot"].__setitem__("dims", 7), Inconsistent),
    (lambda c: c["layers"][1]["mlp"]["router"].__setitem__("top", 7), Inconsistent),
    (lambda c: c["layers"][1]["mixer"]["mask"].__setitem__("size", 0), BadValue),
    (lambda c: c["loop"].__setitem__("stop", 5), Inconsistent),
    (lambda c: c["loop"].__setitem__("times", 0), BadValue),
    (lambda c: c["token_side"].__setitem__("dim", 0), BadValue),
])
def test_refused(change, error):
    with pytest.raises(error):
        plan_from_config(_broken(change))
    assert issubclass(error, ConfigError)


def test_the_two_rotations_are_one_up_to_the_order_of_dimensions():
    """Pairs of neighbours are pairs of halves after a shuffle of the dimensions."""
    g = torch.Generator().manual_seed(0)
    x = torch.randn(3, 7, 12, generator=g, dtype=torch.float64)
    pos = torch.tensor([0, 1, 5, 9, 100, 1000, 70000])
    f = plain.frequencies(8, 300.0, torch.float64)
    shuffle = torch.tensor([0, 2, 4, 6, 1, 3, 5, 7, 8, 9, 10, 11])          # halves layout -> where it sits among neighbours
    halves = plain.rotate_halves(x[..., shuffle], pos, f)
    pairs = plain.rotate_pairs(x, pos, f)
    assert torch.allclose(pairs[..., shuffle], halves, atol=1e-12)
    assert torch.equal(pairs[..., 8:], x[..., 8:])


def test_recurrence_equals_its_unrolled_sum():
    """S_t = sum_s (prod_{s < u <= t} f_u) (1 - f_s) v_s: the recurrence against the closed form."""
    g = torch.Generator().manual_seed(1)
    T, E, H, dk, dv = 9, 16, 2, 4, 3
    w = {"l0.mix.q": torch.randn(H * dk, E, generator=g, dtype=torch.float64),
         "l0.mix.f": torch.randn(H * dk, E, generator=g, dtype=torch.float64),
         "l0.mix.f.b": torch.randn(H * dk, generator=g, dtype=torch.float64),
         "l0.mix.lower": torch.rand(H * dk, generator=g, dtype=torch.float64) * 0.9,
         "l0.mix.v": torch.randn(H * dv, E, generator=g, dtype=torch.float64),
         "l0.mix.norm": torch.ones(dv, dtype=torch.float64), "l0.mix.o": torch.eye(H * dv, dtype=torch.float64)}
    h = torch.randn(T, E, generator=g, dtype=torch.float64)
    got = plain.hgrn2(h, w, "l0", dict(heads=H, dim=dk, vdim=dv), 1e-6)
    q = plain.silu(h @ w["l0.mix.q"].T).reshape(T, H, dk)
    v = (h @ w["l0.mix.v"].T).reshape(T, H, dv)
    low = w["l0.mix.lower"]
    f = (low + (1 - low) * torch.sigmoid(h @ w["l0.mix.f"].T + w["l0.mix.f.b"])).reshape(T, H, dk)
    out = torch.zeros(T, H, dv, dtype=torch.float64)
    for t in range(T):
        for s in range(t + 1):
            decay = torch.ones(H, dk, dtype=torch.float64)
            for u in range(s + 1, t + 1):
                decay = decay * f[u]
            out[t] += torch.einsum("hk,hv->hv", q[t] * decay * (1 - f[s]), v[s])
    want = plain.rms(out, 1e-6).reshape(T, H * dv)
    assert torch.allclose(got, want, atol=1e-10)


def test_latent_attention_equals_attention_over_made_keys_in_its_absorbed_form():
    """(W_uk c) . q = c . (W_uk^T q): scores and values taken from the latent alone give the same result."""
    g = torch.Generator().manual_seed(2)
    T, E, H, dn, dr, dv, r = 11, 24, 3, 6, 4, 5, 8
    mx = dict(heads=H, dim=dn, rot_dim=dr, vdim=dv, kv_rank=r, rot=dict(base=100.0, dims=dr), scale=0.37, mask=dict(size=4))
    rnd = lambda *s: torch.randn(*s, generator=g, dtype=torch.float64)
    w = {"l0.mix.q": rnd(H * (dn + dr), E), "l0.mix.dkv": rnd(r + dr, E), "l0.mix.dkv.norm": rnd(r), "l0.mix.uk": rnd(H * dn, r),
         "l0.mix.uv": rnd(H * dv, r), "l0.mix.o": torch.eye(H * dv, dtype=torch.float64)}
    h = rnd(T, E)
    pos = torch.arange(T)
    got = plain.latent_attention(h, pos, w, "l0", mx, 1e-6, pairs=True)
    q = (h @ w["l0.mix.q"].T).reshape(T, H, dn + dr)
    ckr = h @ w["l0.mix.dkv"].T
    c = plain.rms(ckr[:, :r], 1e-6) * w["l0.mix.dkv.norm"]
    f = plain.frequencies(dr, 100.0, torch.float64)
    kr = plain.rotate_pairs(ckr[:, r:], pos, f)
    outs = []
    for hd in range(H):
        qa = q[:, hd, :dn] @ w["l0.mix.uk"][hd * dn:(hd + 1) * dn]            # [T, r]
        s = (qa @ c.T + plain.rotate_pairs(q[:, hd, dn:], pos, f) @ kr.T) * 0.37
        dist = pos[:, None] - pos[None, :]
        s = s.masked_fill((dist < 0) | (dist >= 4), float("-inf"))
        outs.append((torch.softmax(s, -1) @ c) @ w["l0.mix.uv"][hd * dv:(hd + 1) * dv].T)
    assert torch.allclose(got, torch.cat(outs, -1), atol=1e-10)


def test_plain_model_runs_and_every_part_matters(tmp_path):
    """The plain model on configuration A: silencing the side input, the gates' biases, the loop's added embedding
    or the recurrence's lower bound moves the logits (so a comparison with it can notice their absence)."""
    cfg, seed = CONFIGS["A"]
    d = write_model(cfg, seed, str(tmp_path / "a"))
    tokens = [3, 17, 150, 8, 8, 41, 99, 0, 7]
    base = plain.PlainKosalorn(d, torch.float64).forward(tokens)
    assert base.shape == (9, 200) and torch.isfinite(base).all()
    for key in ("l1.side.norm", "l1.rg1.b", "l0.mix.lower", "embed.norm", "l3.mix.dq.norm"):
        m = plain.PlainKosalorn(d, torch.float64)
        m.w[key] = m.w[key] * 0.5
        assert float((m.forward(tokens) - base).abs().max()) > 1e-3 * float(base.abs().max()), key
    once = plain.PlainKosalorn(d, torch.float64)
    once.cfg = dict(once.cfg, loop=dict(start=1, stop=3, times=1))
    assert float((once.forward(tokens) - base).abs().max()) > 1e-2 * float(base.abs().max())
    assert math.isclose(float(base.abs().max()), float(base.abs().max()))


def test_random_weights_mode_writes_a_loadable_model(tmp_path):
    from imparo_amd import write_random_model
    from imparo_amd.weights import load_weights
    cfg = CONFIGS["C"][0]
    d = write_random_model(cfg, 5, str(tmp_path / "m"))
    _, plan = plan_from_config(cfg)
    declared = {k: decl for k, (decl, _) in declared_tensors(plan).items()}
    tensors = load_weights(d, declared)
    tensors.pop("__file__").close()
    assert set(tensors) == set(declared)
    assert tuple(tensors["l0.norm1"].shape) == () and tuple(tensors["embed.norm"].shape) == ()
    low = tensors["l1.mix.lower"].float()
    assert float(low.min()) >= 0.0 and float(low.max()) < 1.0
    assert torch.isfinite(plain.PlainKosalorn(d).forward([1, 2, 3])).all()
