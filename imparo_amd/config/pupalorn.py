"""Typed Pupalorn configuration and its plan.

A Pupalorn model is a decoder whose layers are listed one by one in
config.json (`layers`: each with a `type`, the `mixer`'s sizes and an `mlp` or
null). Every sublayer sits between two norms, x += m * ls * post(f(pre(x))),
with norm weights kept as their distance from one, a layer scale `ls` per sublayer and one
residual multiplier `m`. The mixer is grouped-query attention with per-head
query and key norms, a rotation of part of each head whose frequencies may be
rescaled by wavelength, and a sliding window; a layer may have no keys and
values of its own and read those of an earlier layer (`kv_from`). The
feed-forward is a mixture of experts with a softmax router, a correction that
moves the choice only, and experts that pass their input through. The
embedding is scaled by a constant. Every size and every constant that may
differ between models comes from the file.
"""
from __future__ import annotations

from dataclasses import dataclass, field
from typing import Any, Dict, List, Optional

from .errors import BadValue, Inconsistent, MissingKey
from .plan import LayerCall, LayerPlan, ModelPlan, PartSpec
from .tumadra import _int, _num

ARCHITECTURE = "Pupalorn"
MIXER_KINDS = ("attention",)
MLP_KINDS = ("moe",)
MAX_POSITION = 1 << 30        # positions are int32 and enter only through angles

_ATTENTION_KEYS = ("heads", "kv_heads", "dim", "vdim", "scale")
_SCALING_KEYS = ("factor", "low", "high", "original")


@dataclass
class PupalornMlp:
    ff: int                    # an expert's hidden width
    experts: int               # real experts
    identity: int              # router outputs past them that pass the input through
    top: int


@dataclass
class PupalornLayer:
    type: str
    mixer: Dict[str, Any]
    mlp: Optional[PupalornMlp]

    @property
    def kv_from(self) -> Optional[int]:
        return self.mixer.get("kv_from")

    @property
    def window(self) -> Optional[int]:
        mask = self.mixer.get("mask")
        return None if mask is None else mask["size"]


@dataclass
class PupalornConfig:
    vocab: int
    width: int
    layers: List[PupalornLayer]
    norm_eps: float
    residual_mult: float = 1.0
    embedding_scale: float = 1.0
    raw: Dict[str, Any] = field(default_factory=dict)
    unread_keys: List[str] = field(default_factory=list)

    @classmethod
    def from_dict(cls, d: Dict[str, Any]) -> "PupalornConfig":
        for key in ("vocab", "width", "layers", "norm"):
            if key not in d:
                raise MissingKey(f"config.json: required key {key!r} is missing")
        norm = d["norm"]
        if not isinstance(norm, dict):
            raise BadValue("config.json: norm must be an object with eps")
        if not isinstance(d["layers"], list) or not d["layers"]:
            raise BadValue("config.json: layers must be a non-empty list")
        emb = d.get("embedding") or {}
        if not isinstance(emb, dict):
            raise BadValue("config.json: embedding must be an object with scale")
        cfg = cls(vocab=_int(d, "vocab", "the model"), width=_int(d, "width", "the model"),
                  layers=[cls._layer(i, entry) for i, entry in enumerate(d["layers"])],
                  norm_eps=_num(norm, "eps", "norm"),
                  residual_mult=_num(d, "residual_mult", "the model") if "residual_mult" in d else 1.0,
                  embedding_scale=_num(emb, "scale", "embedding") if "scale" in emb else 1.0, raw=d)
        known = {"architecture", "architectures", "vocab", "width", "layers", "norm", "residual_mult", "embedding"}
        cfg.unread_keys = sorted(k for k in d if k not in known)
        cfg.validate()
        return cfg

    @staticmethod
    def _layer(i: int, entry: Any) -> PupalornLayer:
        where = f"layers[{i}]"
        if not isinstance(entry, dict) or "type" not in entry or "mixer" not in entry:
            raise BadValue(f"config.json: {where} must be an object with type, mixer and mlp")
        kind = entry["type"]
        if kind not in MIXER_KINDS:
            raise BadValue(f"config.json: {where}.type is {kind!r}; known mixers are {', '.join(MIXER_KINDS)}")
        mixer = entry["mixer"]
        if not isinstance(mixer, dict):
            raise BadValue(f"config.json: {where}.mixer must be an object")
        for key in _ATTENTION_KEYS:
            if key not in mixer:
                raise MissingKey(f"config.json: {where}.mixer lacks {key!r}")
        mlp = entry.get("mlp")
        parsed = None
        if mlp is not None:
            if not isinstance(mlp, dict):
                raise BadValue(f"config.json: {where}.mlp must be an object or null")
            if mlp.get("kind", "moe") not in MLP_KINDS:
                raise BadValue(f"config.json: {where}.mlp.kind is {mlp.get('kind')!r}; known: {', '.join(MLP_KINDS)}")
            expert, router = mlp.get("expert"), mlp.get("router")
            if not isinstance(expert, dict) or not isinstance(router, dict):
                raise MissingKey(f"config.json: {where}.mlp needs the objects 'expert' and 'router'")
            parsed = PupalornMlp(ff=_int(expert, "ff", f"{where}.mlp.expert"),
                                 experts=_int(router, "experts", f"{where}.mlp.router", 0),
                                 identity=_int(router, "identity", f"{where}.mlp.router", 0) if "identity" in router else 0,
                                 top=_int(router, "top", f"{where}.mlp.router"))
        return PupalornLayer(kind, dict(mixer), parsed)

    def validate(self) -> None:
        if self.norm_eps <= 0:
            raise BadValue("norm.eps must be positive")
        for i, layer in enumerate(self.layers):
            m, where = layer.mixer, f"layers[{i}].mixer"
            heads, kv = _int(m, "heads", where), _int(m, "kv_heads", where)
            dim = _int(m, "dim", where)
            _int(m, "vdim", where), _num(m, "scale", where)
            if heads % kv:
                raise Inconsistent(f"{where}: {heads} heads cannot share {kv} kv heads evenly")
            mask = m.get("mask")
            if mask is not None:
                if not isinstance(mask, dict):
                    raise BadValue(f"{where}.mask must be an object with size, or null")
                _int(mask, "size", f"{where}.mask")
            rot = m.get("rot")
            if rot is not None:
                if not isinstance(rot, dict):
                    raise BadValue(f"{where}.rot must be an object with base and dims, or null")
                dims = _int(rot, "dims", f"{where}.rot", 0)
                if dims % 2 or dims > dim:
                    raise Inconsistent(f"{where}.rot.dims = {dims} must be even and at most dim = {dim}")
                if _num(rot, "base", f"{where}.rot") <= 0:
                    raise BadValue(f"{where}.rot.base must be positive")
                scaling = rot.get("scaling")
                if scaling is not None:
                    if not isinstance(scaling, dict):
                        raise BadValue(f"{where}.rot.scaling must be an object or null")
                    for key in _SCALING_KEYS:
                        if _num(scaling, key, f"{where}.rot.scaling") <= 0:
                            raise BadValue(f"{where}.rot.scaling.{key} must be positive")
            src = m.get("kv_from")
            if src is not None:
                if isinstance(src, bool) or not isinstance(src, int) or not 0 <= src < i:
                    raise Inconsistent(f"{where}.kv_from = {src!r} names no earlier layer")
                other = self.layers[src].mixer
                if other.get("kv_from") is not None:
                    raise Inconsistent(f"{where}.kv_from names layer {src}, which has no keys and values of its own")
                # the cache's shape must be the reader's own; its rotation is applied to its own queries as its
                # own entry says (a model whose layers rotate differently has said so itself)
                for key in ("heads", "kv_heads", "dim", "vdim"):
                    if other.get(key) != m.get(key):
                        raise Inconsistent(f"{where}: {key} differs from layer {src}'s, whose keys and values it reads")
            if layer.mlp is not None:
                p = layer.mlp
                if not 1 <= p.top <= p.experts + p.identity:
                    raise Inconsistent(f"layers[{i}].mlp.router: top = {p.top} of {p.experts + p.identity} experts")

    def keep_window(self, i: int) -> Optional[int]:
        """What layer i's cache must keep: the widest window of the layers that read it (None: everything)."""
        windows = [self.layers[i].window] + [l.window for l in self.layers if l.kv_from == i]
        return None if any(w is None for w in windows) else max(windows)

    def to_dict(self) -> Dict[str, Any]:
        return dict(self.raw)


def build_plan(cfg: PupalornConfig) -> ModelPlan:
    E = cfg.width

    def norm(name: str, scale_tensor: Optional[str] = None) -> PartSpec:
        params = dict(width=E, eps=cfg.norm_eps, tensor=name, offset=1.0)
        if scale_tensor is not None:
            params.update(scale_tensor=scale_tensor, multiplier=cfg.residual_mult)
        return PartSpec("rms_norm", "", params)

    layers: List[LayerPlan] = []
    for i, layer in enumerate(cfg.layers):
        base, m = f"l{i}", layer.mixer
        rot = m.get("rot")
        position = None
        if rot is not None and rot["dims"] > 0:
            position = PartSpec("rope_neox", "", dict(rotary_dim=rot["dims"], base=float(rot["base"]), precise=True,
                                                      wavelength_scaling=rot.get("scaling")))
        owner = i if layer.kv_from is None else layer.kv_from
        mixer = PartSpec("attention", f"{base}.mix", dict(
            width=E, heads=m["heads"], kv_heads=m["kv_heads"], head_dim=m["dim"], value_dim=m["vdim"],
            scale=float(m["scale"]), window=layer.window, keep_window=cfg.keep_window(owner),
            shared_kv=layer.kv_from is not None, exact_weights=True,
            qk_norm=PartSpec("rms_norm", "", dict(eps=cfg.norm_eps)), position=position, weight_suffix="",
            names=dict(q="q", k="k", v="v", o="o", q_norm="q.norm", k_norm="k.norm")))
        parts = dict(mixer_norm=("norm", norm(f"{base}.norm1")), mixer=("mixer", mixer),
                     mixer_post=("norm", norm(f"{base}.norm1b", f"{base}.ls1")))
        if layer.mlp is not None:
            p = layer.mlp
            parts["ffn_norm"] = ("norm", norm(f"{base}.norm2"))
            parts["ffn"] = ("feed_forward", PartSpec("routed_experts", f"{base}.mlp", dict(
                width=E, hidden=p.ff, experts=p.experts, identity=p.identity, top=p.top, activation="relu2")))
            parts["ffn_post"] = ("norm", norm(f"{base}.norm2b", f"{base}.ls2"))
        layers.append(LayerPlan(parts, "sandwich"))
    order = [LayerCall(i, layer.kv_from) for i, layer in enumerate(cfg.layers)]
    plan = ModelPlan(
        architecture=ARCHITECTURE,
        vocab_size=cfg.vocab,
        hidden_size=E,
        max_position=MAX_POSITION,
        embedding=PartSpec("embedding", "embed", dict(vocab=cfg.vocab, width=E, tensor="embed",
                                                      scale=cfg.embedding_scale)),
        layers=layers,
        order=order,
        final_norm=norm("final.norm"),
        head=PartSpec("linear_head", "head", dict(vocab=cfg.vocab, width=E, tensor="head")),
    )
    plan.validate()
    return plan
