"""Typed Kosalorn configuration and its plan.

A Kosalorn model is a decoder whose layers are listed one by one in
config.json (`layers`: each with a `type`, the `mixer`'s sizes and an `mlp` or
null). A layer is parallel: one norm (an RMS norm whose weight is a single
number) feeds the mixer and the feed-forward alike, each result is gated by
sigmoid(W h + b) of the same normed input, and both are added to the stream.
Behind that a layer may take a small embedding of the token itself
(`token_side`), gate it by the stream, project it, norm it and add it. The
embedding's rows are normed before the first layer. Layers `loop.start ..
loop.stop - 1` run `loop.times` times in a row with the same weights and a
cache or state of their own per pass, and every pass after the first starts
by adding the embedding's output to the stream again.

Mixers: `latent_attention` (queries through a normed latent, keys and values
from a cached latent plus one rotated key part for all heads, rotation in
halves, a sliding window), `latent_attention_2` (queries projected directly,
rotation of neighbouring pairs, causal) and `hgrn2` (a gated linear
recurrence with a matrix of state a head). Feed-forwards: `dense` (SwiGLU) and
`moe` (sigmoid scores, the chosen experts read their input times their
score). Every size and every constant that may differ between models comes
from the file.
"""
from __future__ import annotations

from dataclasses import dataclass, field
from typing import Any, Dict, List, Optional

from .errors import BadValue, Inconsistent, MissingKey
from .plan import LayerCall, LayerPlan, ModelPlan, PartSpec
from .tumadra import _int, _num

ARCHITECTURE = "Kosalorn"
LATENT_KINDS = ("latent_attention", "latent_attention_2")
MIXER_KINDS = LATENT_KINDS + ("hgrn2",)
MLP_KINDS = ("dense", "moe")
MAX_POSITION = 1 << 30        # positions are int32 and enter only through angles

_LATENT_KEYS = ("heads", "dim", "rot_dim", "vdim", "kv_rank", "scale", "rot")
_HGRN2_KEYS = ("heads", "dim", "vdim")


@dataclass
class KosalornMlp:
    kind: str                  # "dense" | "moe"
    ff: int                    # the hidden width (an expert's, for "moe")
    experts: int = 0
    top: int = 0


@dataclass
class KosalornLayer:
    type: str
    mixer: Dict[str, Any]
    mlp: Optional[KosalornMlp]

    @property
    def window(self) -> Optional[int]:
        mask = self.mixer.get("mask")
        return None if mask is None else mask["size"]


@dataclass
class KosalornConfig:
    vocab: int
    width: int
    layers: List[KosalornLayer]
    norm_eps: float
    side_dim: int = 0          # width of the per-layer token embedding; 0: none
    loop_start: int = 0
    loop_stop: int = 0
    loop_times: int = 1
    raw: Dict[str, Any] = field(default_factory=dict)
    unread_keys: List[str] = field(default_factory=list)

    @classmethod
    def from_dict(cls, d: Dict[str, Any]) -> "KosalornConfig":
        for key in ("vocab", "width", "layers", "norm"):
            if key not in d:
                raise MissingKey(f"config.json: required key {key!r} is missing")
        norm = d["norm"]
        if not isinstance(norm, dict):
            raise BadValue("config.json: norm must be an object with eps")
        if not isinstance(d["layers"], list) or not d["layers"]:
            raise BadValue("config.json: layers must be a non-empty list")
        loop = d.get("loop")
        start, stop, times = 0, 0, 1
        if loop is not None:
            if not isinstance(loop, dict):
                raise BadValue("config.json: loop must be an object with start, stop and times")
            start, stop = _int(loop, "start", "loop", 0), _int(loop, "stop", "loop", 0)
            times = _int(loop, "times", "loop", 1)
        side = d.get("token_side")
        if side is not None and not isinstance(side, dict):
            raise BadValue("config.json: token_side must be an object with dim, or null")
        cfg = cls(vocab=_int(d, "vocab", "the model"), width=_int(d, "width", "the model"),
                  layers=[cls._layer(i, entry) for i, entry in enumerate(d["layers"])],
                  norm_eps=_num(norm, "eps", "norm"),
                  side_dim=0 if side is None else _int(side, "dim", "token_side"),
                  loop_start=start, loop_stop=stop, loop_times=times, raw=d)
        known = {"architecture", "architectures", "vocab", "width", "layers", "norm", "loop", "token_side"}
        cfg.unread_keys = sorted(k for k in d if k not in known)
        cfg.validate()
        return cfg

    @staticmethod
    def _layer(i: int, entry: Any) -> KosalornLayer:
        where = f"layers[{i}]"
        if not isinstance(entry, dict) or "type" not in entry or "mixer" not in entry:
            raise BadValue(f"config.json: {where} must be an object with type, mixer and mlp")
        kind = entry["type"]
        if kind not in MIXER_KINDS:
            raise BadValue(f"config.json: {where}.type is {kind!r}; known mixers are {', '.join(MIXER_KINDS)}")
        mixer = entry["mixer"]
        if not isinstance(mixer, dict):
            raise BadValue(f"config.json: {where}.mixer must be an object")
        for key in (_LATENT_KEYS if kind in LATENT_KINDS else _HGRN2_KEYS):
            if key not in mixer:
                raise MissingKey(f"config.json: {where}.mixer lacks {key!r}")
        mlp = entry.get("mlp")
        parsed = None
        if mlp is not None:
            if not isinstance(mlp, dict) or "kind" not in mlp:
                raise BadValue(f"config.json: {where}.mlp must be an object with kind, or null")
            if mlp["kind"] not in MLP_KINDS:
                raise BadValue(f"config.json: {where}.mlp.kind is {mlp['kind']!r}; known: {', '.join(MLP_KINDS)}")
            if mlp["kind"] == "dense":
                parsed = KosalornMlp("dense", _int(mlp, "ff", f"{where}.mlp"))
            else:
                expert, router = mlp.get("expert"), mlp.get("router")
                if not isinstance(expert, dict) or not isinstance(router, dict):
                    raise MissingKey(f"config.json: {where}.mlp needs the objects 'expert' and 'router'")
                parsed = KosalornMlp("moe", _int(expert, "ff", f"{where}.mlp.expert"),
                                     experts=_int(router, "experts", f"{where}.mlp.router"),
                                     top=_int(router, "top", f"{where}.mlp.router"))
        return KosalornLayer(kind, dict(mixer), parsed)

    def validate(self) -> None:
        if self.norm_eps <= 0:
            raise BadValue("norm.eps must be positive")
        if not 0 <= self.loop_start <= self.loop_stop <= len(self.layers):
            raise Inconsistent(f"loop {self.loop_start}..{self.loop_stop} does not lie inside {len(self.layers)} layers")
        for i, layer in enumerate(self.layers):
            m, where = layer.mixer, f"layers[{i}].mixer"
            if layer.type in LATENT_KINDS:
                for key in ("heads", "dim", "rot_dim", "vdim", "kv_rank"):
                    _int(m, key, where)
                _num(m, "scale", where)
                if "q_rank" in m and m["q_rank"] is not None:
                    _int(m, "q_rank", where)
                elif layer.type == "latent_attention":
                    raise MissingKey(f"config.json: {where} lacks 'q_rank'")
                rot = m["rot"]
                if not isinstance(rot, dict):
                    raise BadValue(f"{where}.rot must be an object with base and dims")
                dims = _int(rot, "dims", f"{where}.rot", 0)
                if dims % 2 or dims > m["rot_dim"]:
                    raise Inconsistent(f"{where}.rot.dims = {dims} must be even and at most rot_dim = {m['rot_dim']}")
                if _num(rot, "base", f"{where}.rot") <= 0:
                    raise BadValue(f"{where}.rot.base must be positive")
                mask = m.get("mask")
                if mask is not None:
                    if not isinstance(mask, dict):
                        raise BadValue(f"{where}.mask must be an object with size, or null")
                    _int(mask, "size", f"{where}.mask")
            else:
                for key in _HGRN2_KEYS:
                    _int(m, key, where)
            if layer.mlp is not None and layer.mlp.kind == "moe" and not 1 <= layer.mlp.top <= layer.mlp.experts:
                raise Inconsistent(f"layers[{i}].mlp.router: top = {layer.mlp.top} of {layer.mlp.experts} experts")

    def order(self) -> List[LayerCall]:
        """The layers in the order they run: those of the loop `times` times in a row; the first
        layer of every pass after the first takes the embedding's output into the stream again."""
        n = len(self.layers)
        calls = [LayerCall(i) for i in range(self.loop_start)]
        for p in range(self.loop_times):
            calls += [LayerCall(i, add_input=(p > 0 and i == self.loop_start))
                      for i in range(self.loop_start, self.loop_stop)]
        return calls + [LayerCall(i) for i in range(self.loop_stop, n)]

    def to_dict(self) -> Dict[str, Any]:
        return dict(self.raw)


def build_plan(cfg: KosalornConfig) -> ModelPlan:
    E = cfg.width
    norm = lambda name: PartSpec("rms_norm", "", dict(width=E, eps=cfg.norm_eps, tensor=name, scalar=True))
    layers: List[LayerPlan] = []
    for i, layer in enumerate(cfg.layers):
        base, m = f"l{i}", layer.mixer
        if layer.type in LATENT_KINDS:
            rot = m["rot"]
            pairs = layer.type == "latent_attention_2"
            position = None
            if rot["dims"] > 0:
                position = PartSpec("rope_pairs" if pairs else "rope_neox", "",
                                    dict(rotary_dim=rot["dims"], base=float(rot["base"]), precise=True))
            mixer = PartSpec("latent_attention", f"{base}.mix", dict(
                width=E, heads=m["heads"], dim=m["dim"], rot_dim=m["rot_dim"], vdim=m["vdim"],
                kv_rank=m["kv_rank"], q_rank=m.get("q_rank"), scale=float(m["scale"]), window=layer.window,
                eps=cfg.norm_eps, position=position))
        else:
            mixer = PartSpec("hgrn2", f"{base}.mix", dict(width=E, heads=m["heads"], dim=m["dim"], vdim=m["vdim"],
                                                           eps=cfg.norm_eps))
        gate = lambda n: PartSpec("sigmoid_gate", base, dict(width=E, weight=f"{base}.{n}", bias=f"{base}.{n}.b"))
        parts = dict(mixer_norm=("norm", norm(f"{base}.norm1")), mixer=("mixer", mixer), mixer_gate=("gate", gate("rg1")))
        if layer.mlp is not None:
            p = layer.mlp
            if p.kind == "dense":
                ffn = PartSpec("swiglu", f"{base}.mlp", dict(width=E, hidden=p.ff, weight_suffix="",
                                                              names=dict(gate="gate", up="up", down="down")))
            else:
                ffn = PartSpec("routed_experts", f"{base}.mlp", dict(
                    width=E, hidden=p.ff, experts=p.experts, identity=0, top=p.top, activation="swiglu",
                    scoring="sigmoid", weigh="input",
                    names=dict(correction=None, expert_gate="e{e}.gate", expert_up="e{e}.up", expert_down="e{e}.down")))
            parts["ffn"] = ("feed_forward", ffn)
            parts["ffn_gate"] = ("gate", gate("rg2"))
        if cfg.side_dim:
            parts["side"] = ("side", PartSpec("token_side", f"{base}.side", dict(
                width=E, dim=cfg.side_dim, vocab=cfg.vocab, table="side.embed", table_width=cfg.side_dim * len(cfg.layers),
                offset=i * cfg.side_dim, eps=cfg.norm_eps)))
        layers.append(LayerPlan(parts, "parallel"))
    plan = ModelPlan(
        architecture=ARCHITECTURE,
        vocab_size=cfg.vocab,
        hidden_size=E,
        max_position=MAX_POSITION,
        embedding=PartSpec("embedding", "embed", dict(vocab=cfg.vocab, width=E, tensor="embed",
                                                      norm=norm("embed.norm"))),
        layers=layers,
        order=cfg.order(),
        final_norm=norm("final.norm"),
        head=PartSpec("linear_head", "head", dict(vocab=cfg.vocab, width=E, tensor="head")),
    )
    plan.validate()
    return plan
