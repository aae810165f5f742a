"""Typed Mepapel configuration and its plan.

A Mepapel model is a decoder whose layers are listed one by one in config.json
(`layers`: each with a `type`, the `mixer`'s sizes and an `mlp` or null). A
sublayer reads the stream itself and a norm sits on its result only:
x <- x + m * N1(mixer(x)), then x <- x + m * N2(ff(x)), with RMS norms N and
m = `residual_mult`.

Mixers: `mamba2` (a state-space layer with one decay a head), `delta` (the
gated delta rule) and `parallel` (two mixers side by side on one input:
softmax attention with biases, a short conv on q, k and v, head norms, a
rotation of neighbouring pairs and a mask in chunks; and retention, linear
attention with a fixed decay a head and a rotation in halves; each result
normed over the width, half their sum). Feed-forwards: `dense` (a gated unit
with bounds) and `moe` (sigmoid scores, a correction on the choice, groups of
experts of which only the best can be chosen, chosen scores normed to a sum of
one and scaled, and a shared expert with a gate a token). Every size and
every constant that may differ between models comes from the file; what the
file leaves out (a mask, a rotation, groups, a shared expert, an mlp) is not
there.
"""
from __future__ import annotations

from dataclasses import dataclass, field
from typing import Any, Dict, List, Optional

from .errors import BadValue, Inconsistent, MissingKey
from .plan import LayerCall, LayerPlan, ModelPlan, PartSpec
from .tumadra import _int, _num

ARCHITECTURE = "Mepapel"
MIXER_KINDS = ("mamba2", "delta", "parallel")
MLP_KINDS = ("dense", "moe")
MAX_POSITION = 1 << 30        # positions are int32 and enter only through angles and masks
GLU_ALPHA = 1.702             # the dense unit's g * sigmoid(alpha g)

_MAMBA2_KEYS = ("heads", "vdim", "state", "conv")
_DELTA_KEYS = ("heads", "kv_heads", "dim", "vdim", "conv")
_LEFT_KEYS = ("heads", "kv_heads", "dim", "vdim", "scale")
_RIGHT_KEYS = ("heads", "dim", "vdim", "decay")


def _object(d: Dict[str, Any], key: str, where: str, required: bool = True) -> Optional[Dict[str, Any]]:
    v = d.get(key)
    if v is None:
        if required:
            raise MissingKey(f"config.json: {where} lacks the object {key!r}")
        return None
    if not isinstance(v, dict):
        raise BadValue(f"config.json: {where}.{key} must be an object")
    return v


def _rotation(m: Dict[str, Any], where: str, dim: int) -> Optional[Dict[str, Any]]:
    rot = _object(m, "rot", where, required=False)
    if rot is None:
        return None
    dims = _int(rot, "dims", f"{where}.rot", 0)
    if dims % 2 or dims > dim:
        raise Inconsistent(f"{where}.rot.dims = {dims} must be even and at most dim = {dim}")
    if _num(rot, "base", f"{where}.rot") <= 0:
        raise BadValue(f"{where}.rot.base must be positive")
    return dict(dims=dims, base=float(rot["base"])) if dims else None


@dataclass
class MepapelMlp:
    kind: str                  # "dense" | "moe"
    ff: int                    # the hidden width (an expert's, for "moe")
    limit: float = 0.0         # dense: the bound on gate and up
    experts: int = 0
    top: int = 0
    group_count: int = 1
    group_keep: int = 1
    scale: float = 1.0
    shared_ff: int = 0         # 0: no shared expert


@dataclass
class MepapelLayer:
    type: str
    mixer: Dict[str, Any]
    mlp: Optional[MepapelMlp]


@dataclass
class MepapelConfig:
    vocab: int
    width: int
    layers: List[MepapelLayer]
    norm_eps: float
    residual_mult: float = 1.0
    raw: Dict[str, Any] = field(default_factory=dict)
    unread_keys: List[str] = field(default_factory=list)

    @classmethod
    def from_dict(cls, d: Dict[str, Any]) -> "MepapelConfig":
        for key in ("vocab", "width", "layers", "norm"):
            if key not in d:
                raise MissingKey(f"config.json: required key {key!r} is missing")
        norm = d["norm"]
        if not isinstance(norm, dict):
            raise BadValue("config.json: norm must be an object with eps")
        if not isinstance(d["layers"], list) or not d["layers"]:
            raise BadValue("config.json: layers must be a non-empty list")
        cfg = cls(vocab=_int(d, "vocab", "the model"), width=_int(d, "width", "the model"),
                  layers=[cls._layer(i, entry) for i, entry in enumerate(d["layers"])],
                  norm_eps=_num(norm, "eps", "norm"),
                  residual_mult=_num(d, "residual_mult", "the model") if "residual_mult" in d else 1.0, raw=d)
        known = {"architecture", "architectures", "vocab", "width", "layers", "norm", "residual_mult"}
        cfg.unread_keys = sorted(k for k in d if k not in known)
        if cfg.norm_eps <= 0:
            raise BadValue("norm.eps must be positive")
        return cfg

    @staticmethod
    def _layer(i: int, entry: Any) -> MepapelLayer:
        where = f"layers[{i}]"
        if not isinstance(entry, dict) or "type" not in entry or "mixer" not in entry:
            raise BadValue(f"config.json: {where} must be an object with type, mixer and mlp")
        kind = entry["type"]
        if kind not in MIXER_KINDS:
            raise BadValue(f"config.json: {where}.type is {kind!r}; known mixers are {', '.join(MIXER_KINDS)}")
        mixer = entry["mixer"]
        if not isinstance(mixer, dict):
            raise BadValue(f"config.json: {where}.mixer must be an object")
        w = f"{where}.mixer"
        if kind == "mamba2":
            for key in _MAMBA2_KEYS:
                _int(mixer, key, w)
            groups = _int(mixer, "groups", w) if "groups" in mixer else 1
            parts = _int(mixer, "norm_groups", w) if "norm_groups" in mixer else 1
            if mixer["heads"] % groups:
                raise Inconsistent(f"{w}: {mixer['heads']} heads in {groups} groups")
            if (mixer["heads"] * mixer["vdim"]) % parts:
                raise Inconsistent(f"{w}: {mixer['heads'] * mixer['vdim']} values in {parts} norm groups")
            parsed = dict(heads=mixer["heads"], vdim=mixer["vdim"], state=mixer["state"], taps=mixer["conv"],
                          groups=groups, norm_groups=parts)
        elif kind == "delta":
            for key in _DELTA_KEYS:
                _int(mixer, key, w)
            if mixer["heads"] % mixer["kv_heads"]:
                raise Inconsistent(f"{w}: {mixer['heads']} heads on {mixer['kv_heads']} query/key heads")
            parsed = dict(heads=mixer["heads"], kv_heads=mixer["kv_heads"], dim=mixer["dim"], vdim=mixer["vdim"],
                          taps=mixer["conv"])
        else:
            left, right = _object(mixer, "left", w), _object(mixer, "right", w)
            wl, wr = f"{w}.left", f"{w}.right"
            for key in _LEFT_KEYS:
                (_num if key == "scale" else _int)(left, key, wl)
            if left["heads"] % left["kv_heads"]:
                raise Inconsistent(f"{wl}: {left['heads']} heads on {left['kv_heads']} key/value heads")
            mask = _object(left, "mask", wl, required=False)
            for key in _RIGHT_KEYS[:3]:
                _int(right, key, wr)
            decay = right.get("decay")
            if not isinstance(decay, list) or len(decay) != right["heads"] or any(
                    isinstance(x, bool) or not isinstance(x, (int, float)) for x in decay):
                raise BadValue(f"config.json: {wr}.decay must be a list of one number a head")
            parsed = dict(
                left=dict(heads=left["heads"], kv_heads=left["kv_heads"], dim=left["dim"], vdim=left["vdim"],
                          scale=float(left["scale"]), taps=_int(left, "conv", wl) if left.get("conv") is not None else 0,
                          chunk=None if mask is None else _int(mask, "size", f"{wl}.mask"),
                          rot=_rotation(left, wl, left["dim"])),
                right=dict(heads=right["heads"], dim=right["dim"], vdim=right["vdim"], decay=[float(x) for x in decay],
                           rot=_rotation(right, wr, right["dim"])))
        return MepapelLayer(kind, parsed, MepapelConfig._mlp(entry.get("mlp"), f"{where}.mlp"))

    @staticmethod
    def _mlp(mlp: Any, where: str) -> Optional[MepapelMlp]:
        if mlp is None:
            return None
        if not isinstance(mlp, dict) or "kind" not in mlp:
            raise BadValue(f"config.json: {where} must be an object with kind, or null")
        if mlp["kind"] not in MLP_KINDS:
            raise BadValue(f"config.json: {where}.kind is {mlp['kind']!r}; known: {', '.join(MLP_KINDS)}")
        if mlp["kind"] == "dense":
            limit = _num(mlp, "limit", where)
            if not limit > 0:
                raise BadValue(f"config.json: {where}.limit must be positive")
            return MepapelMlp("dense", _int(mlp, "ff", where), limit=limit)
        expert, router = _object(mlp, "expert", where), _object(mlp, "router", where)
        wr = f"{where}.router"
        out = MepapelMlp("moe", _int(expert, "ff", f"{where}.expert"), experts=_int(router, "experts", wr),
                         top=_int(router, "top", wr), scale=_num(router, "scale", wr) if "scale" in router else 1.0)
        groups = _object(router, "groups", wr, required=False)
        if groups is not None:
            out.group_count, out.group_keep = _int(groups, "count", f"{wr}.groups"), _int(groups, "keep", f"{wr}.groups")
            if out.experts % out.group_count or out.group_keep > out.group_count:
                raise Inconsistent(f"{wr}: {out.experts} experts in {out.group_count} groups of which {out.group_keep} stay")
            if out.group_keep * (out.experts // out.group_count) < out.top:
                raise Inconsistent(f"{wr}: {out.group_keep} groups of {out.experts // out.group_count} experts "
                                   f"cannot give {out.top} choices")
        if not 1 <= out.top <= out.experts:
            raise Inconsistent(f"{wr}: top = {out.top} of {out.experts} experts")
        shared = _object(mlp, "shared", where, required=False)
        if shared is not None:
            out.shared_ff = _int(shared, "ff", f"{where}.shared")
        return out

    def to_dict(self) -> Dict[str, Any]:
        return dict(self.raw)


def _rope(rot: Optional[Dict[str, Any]], kind: str) -> Optional[PartSpec]:
    if rot is None:
        return None
    return PartSpec(kind, "", dict(rotary_dim=rot["dims"], base=rot["base"], precise=True))


def build_plan(cfg: MepapelConfig) -> ModelPlan:
    E, eps, m = cfg.width, cfg.norm_eps, cfg.residual_mult
    through = PartSpec("none", "", dict(width=E))                     # the sublayers read the stream itself
    behind = lambda name: PartSpec("rms_norm", "", dict(width=E, eps=eps, tensor=name, multiplier=m))
    layers: List[LayerPlan] = []
    for i, layer in enumerate(cfg.layers):
        base, x = f"l{i}", layer.mixer
        if layer.type == "mamba2":
            mixer = PartSpec("mamba2", f"{base}.mix", dict(width=E, eps=eps, **x))
        elif layer.type == "delta":
            mixer = PartSpec("gated_delta", f"{base}.mix", dict(width=E, eps=eps, **x))
        else:
            a, b = x["left"], x["right"]
            left = PartSpec("attention", f"{base}.mix.left", dict(
                width=E, heads=a["heads"], kv_heads=a["kv_heads"], head_dim=a["dim"], value_dim=a["vdim"],
                scale=a["scale"], chunk=a["chunk"], conv_taps=a["taps"], bias=True, bias_suffix=".b",
                weight_suffix="", qk_norm=PartSpec("rms_norm", "", dict(eps=eps)), exact_weights=True,
                names=dict(q="q", k="k", v="v", o="o", q_norm="q.norm", k_norm="k.norm"),
                position=_rope(a["rot"], "rope_pairs")))
            right = PartSpec("retention", f"{base}.mix.right", dict(
                width=E, heads=b["heads"], dim=b["dim"], vdim=b["vdim"], decay=b["decay"], eps=eps,
                position=_rope(b["rot"], "rope_neox")))
            mixer = PartSpec("mixer_pair", f"{base}.mix", dict(width=E, eps=eps, left=left, right=right, factor=0.5))
        parts = dict(mixer_norm=("norm", through), mixer=("mixer", mixer), mixer_post=("norm", behind(f"{base}.norm1")))
        p = layer.mlp
        if p is not None:
            unit = dict(gate="gate", up="up", down="down")
            if p.kind == "dense":
                ffn = PartSpec("clamped_glu", f"{base}.mlp", dict(width=E, hidden=p.ff, limit=p.limit, alpha=GLU_ALPHA,
                                                                   weight_suffix="", names=unit))
            else:
                shared = None
                if p.shared_ff:
                    shared = PartSpec("swiglu", f"{base}.mlp.shared", dict(width=E, hidden=p.shared_ff, weight_suffix="",
                                                                            names=unit, scratch_tag="shared_"))
                ffn = PartSpec("routed_experts", f"{base}.mlp", dict(
                    width=E, hidden=p.ff, experts=p.experts, identity=0, top=p.top, activation="swiglu",
                    scoring="sigmoid", weigh="output", group_count=p.group_count, group_keep=p.group_keep,
                    normalize=True, route_scale=p.scale, shared=shared))
            parts.update(ffn_norm=("norm", through), ffn=("feed_forward", ffn), ffn_post=("norm", behind(f"{base}.norm2")))
        layers.append(LayerPlan(parts, "sandwich"))
    plan = ModelPlan(
        architecture=ARCHITECTURE,
        vocab_size=cfg.vocab,
        hidden_size=E,
        max_position=MAX_POSITION,
        embedding=PartSpec("embedding", "embed", dict(vocab=cfg.vocab, width=E, tensor="embed")),
        layers=layers,
        order=[LayerCall(i) for i in range(len(layers))],
        final_norm=PartSpec("rms_norm", "", dict(width=E, eps=eps, tensor="final.norm")),
        head=PartSpec("linear_head", "head", dict(vocab=cfg.vocab, width=E, tensor="head")),
    )
    plan.validate()
    return plan
