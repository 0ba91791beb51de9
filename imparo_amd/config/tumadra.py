"""Typed Tumadra configuration and its plan.

A Tumadra model is a pre-norm decoder whose layers are listed one by one in
config.json (`layers`: each with a `type`, the `mixer`'s sizes and an `mlp` or
null), whose norms cut a row into groups, whose mixers read their input
through a token shift, and whose layers `loop.start .. loop.stop - 1` run
`loop.times` times in a row with the same weights and a cache or state of
their own per pass. Mixers: `attention` (differential attention with a query
temperature and an output gate) and `mamba1` (a selective scan). The
feed-forward is dense with a PolyNorm activation. The embedding adds a
sinusoidal position vector. Every size and every constant that may differ
between models comes from the file.
"""
from __future__ import annotations

from dataclasses import dataclass, field
from typing import Any, Dict, List, Optional

from .errors import BadValue, Inconsistent, MissingKey
from .plan import LayerCall, LayerPlan, ModelPlan, PartSpec

ARCHITECTURE = "Tumadra"
MIXER_KINDS = ("attention", "mamba1")
SINUSOID_BASE = 10000.0
MAX_POSITION = 1 << 30        # positions are int32 and enter only through angles and a logarithm

_ATTENTION_KEYS = ("heads", "kv_heads", "dim", "vdim", "scale", "diff")
_SCAN_KEYS = ("inner", "state", "dt_rank", "conv")


def _int(d: Dict[str, Any], key: str, where: str, lo: int = 1) -> int:
    if key not in d:
        raise MissingKey(f"config.json: {where} lacks {key!r}")
    v = d[key]
    if isinstance(v, bool) or not isinstance(v, int):
        raise BadValue(f"config.json: {where}.{key} must be an integer, got {v!r}")
    if v < lo:
        raise BadValue(f"config.json: {where}.{key} must be at least {lo}, got {v}")
    return v


def _num(d: Dict[str, Any], key: str, where: str) -> float:
    if key not in d:
        raise MissingKey(f"config.json: {where} lacks {key!r}")
    v = d[key]
    if isinstance(v, bool) or not isinstance(v, (int, float)):
        raise BadValue(f"config.json: {where}.{key} must be a number, got {v!r}")
    return float(v)


@dataclass
class TumadraLayer:
    type: str
    mixer: Dict[str, Any]
    ff: Optional[int]          # the feed-forward's hidden width, None for a layer without one


@dataclass
class TumadraConfig:
    vocab: int
    width: int
    layers: List[TumadraLayer]
    norm_eps: float
    norm_groups: int
    loop_start: int = 0
    loop_stop: int = 0
    loop_times: int = 1
    raw: Dict[str, Any] = field(default_factory=dict)
    unread_keys: List[str] = field(default_factory=list)

    @classmethod
    def from_dict(cls, d: Dict[str, Any]) -> "TumadraConfig":
        for key in ("vocab", "width", "layers", "norm"):
            if key not in d:
                raise MissingKey(f"config.json: required key {key!r} is missing")
        norm = d["norm"]
        if not isinstance(norm, dict):
            raise BadValue("config.json: norm must be an object with eps and groups")
        if not isinstance(d["layers"], list) or not d["layers"]:
            raise BadValue("config.json: layers must be a non-empty list")
        layers = [cls._layer(i, entry) for i, entry in enumerate(d["layers"])]
        loop = d.get("loop")
        start, stop, times = 0, 0, 1
        if loop is not None:
            if not isinstance(loop, dict):
                raise BadValue("config.json: loop must be an object with start, stop and times")
            start, stop = _int(loop, "start", "loop", 0), _int(loop, "stop", "loop", 0)
            times = _int(loop, "times", "loop", 1)
        cfg = cls(vocab=_int(d, "vocab", "the model"), width=_int(d, "width", "the model"), layers=layers,
                  norm_eps=_num(norm, "eps", "norm"), norm_groups=_int(norm, "groups", "norm") if "groups" in norm else 1,
                  loop_start=start, loop_stop=stop, loop_times=times, raw=d)
        known = {"architecture", "architectures", "vocab", "width", "layers", "norm", "loop"}
        cfg.unread_keys = sorted(k for k in d if k not in known)
        cfg.validate()
        return cfg

    @staticmethod
    def _layer(i: int, entry: Any) -> TumadraLayer:
        where = f"layers[{i}]"
        if not isinstance(entry, dict) or "type" not in entry or "mixer" not in entry:
            raise BadValue(f"config.json: {where} must be an object with type, mixer and mlp")
        kind = entry["type"]
        if kind not in MIXER_KINDS:
            raise BadValue(f"config.json: {where}.type is {kind!r}; known mixers are {', '.join(MIXER_KINDS)}")
        mixer = entry["mixer"]
        if not isinstance(mixer, dict):
            raise BadValue(f"config.json: {where}.mixer must be an object")
        for key in (_ATTENTION_KEYS if kind == "attention" else _SCAN_KEYS):
            if key not in mixer:
                raise MissingKey(f"config.json: {where}.mixer lacks {key!r}")
        mlp = entry.get("mlp")
        ff = None
        if mlp is not None:
            if not isinstance(mlp, dict):
                raise BadValue(f"config.json: {where}.mlp must be an object or null")
            if mlp.get("kind", "dense") != "dense":
                raise BadValue(f"config.json: {where}.mlp.kind is {mlp.get('kind')!r}; only 'dense' is implemented")
            ff = _int(mlp, "ff", f"{where}.mlp")
        return TumadraLayer(kind, dict(mixer), ff)

    def validate(self) -> None:
        if self.norm_eps <= 0:
            raise BadValue("norm.eps must be positive")
        if self.width % self.norm_groups:
            raise Inconsistent(f"width {self.width} cannot be cut into {self.norm_groups} equal norm groups")
        if not 0 <= self.loop_start <= self.loop_stop <= len(self.layers):
            raise Inconsistent(f"loop {self.loop_start}..{self.loop_stop} does not lie inside {len(self.layers)} layers")
        for i, layer in enumerate(self.layers):
            m = layer.mixer
            where = f"layers[{i}].mixer"
            if layer.type == "attention":
                heads, kv = _int(m, "heads", where), _int(m, "kv_heads", where)
                _int(m, "dim", where), _int(m, "vdim", where), _num(m, "scale", where)
                if heads % kv:
                    raise Inconsistent(f"{where}: {heads} heads cannot share {kv} kv heads evenly")
                if not 0.0 <= _num(m, "diff", where) < 1.0 + 1e-9:
                    raise BadValue(f"{where}.diff must lie in [0, 1]")
                temp = m.get("q_temp")
                if temp is not None:
                    if not isinstance(temp, dict):
                        raise BadValue(f"{where}.q_temp must be an object with coef and every, or null")
                    _num(temp, "coef", f"{where}.q_temp"), _int(temp, "every", f"{where}.q_temp")
            else:
                for key in _SCAN_KEYS:
                    _int(m, key, where)

    def order(self) -> List[int]:
        """Layers in the order they run: those of the loop `times` times in a row."""
        n = len(self.layers)
        inside = list(range(self.loop_start, self.loop_stop))
        return list(range(self.loop_start)) + inside * self.loop_times + list(range(self.loop_stop, n))

    def to_dict(self) -> Dict[str, Any]:
        return dict(self.raw)


def build_plan(cfg: TumadraConfig) -> ModelPlan:
    E = cfg.width
    norm = lambda name: PartSpec("rms_norm", "", dict(width=E, eps=cfg.norm_eps, groups=cfg.norm_groups, tensor=name))
    layers: List[LayerPlan] = []
    for i, layer in enumerate(cfg.layers):
        base, m = f"l{i}", layer.mixer
        if layer.type == "attention":
            temp = m.get("q_temp")
            mixer = PartSpec("differential_attention", f"{base}.mix", dict(
                width=E, heads=m["heads"], kv_heads=m["kv_heads"], dim=m["dim"], vdim=m["vdim"],
                scale=float(m["scale"]), diff=float(m["diff"]), eps=cfg.norm_eps, qkv_bias=True, gate=True,
                q_temp=None if temp is None else dict(coef=float(temp["coef"]), every=int(temp["every"]))))
        else:
            mixer = PartSpec("selective_scan", f"{base}.mix", dict(
                width=E, inner=m["inner"], state=m["state"], dt_rank=m["dt_rank"], taps=m["conv"]))
        parts = dict(mixer_norm=("norm", norm(f"{base}.norm1")),
                     shift=("shift", PartSpec("token_shift", base, dict(width=E, tensor=f"{base}.shift"))),
                     mixer=("mixer", mixer))
        if layer.ff is not None:
            parts["ffn_norm"] = ("norm", norm(f"{base}.norm2"))
            parts["ffn"] = ("feed_forward", PartSpec("poly_norm", f"{base}.mlp", dict(
                width=E, hidden=layer.ff, eps=cfg.norm_eps)))
        layers.append(LayerPlan(parts, "pre_norm"))
    plan = ModelPlan(
        architecture=ARCHITECTURE,
        vocab_size=cfg.vocab,
        hidden_size=E,
        max_position=MAX_POSITION,
        embedding=PartSpec("sinusoid_embedding", "embed", dict(vocab=cfg.vocab, width=E, tensor="embed",
                                                               base=SINUSOID_BASE)),
        layers=layers,
        order=[LayerCall(i) for i in cfg.order()],
        final_norm=norm("final.norm"),
        head=PartSpec("linear_head", "head", dict(vocab=cfg.vocab, width=E, tensor="head")),
    )
    plan.validate()
    return plan
