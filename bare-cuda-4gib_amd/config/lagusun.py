"""Configuration of the Lagusun decoder: a stack of pre-norm layers, each with one of two attention mixers and a mixture of
experts, whose sublayer outputs are multiplied by a learned number a channel before they join the stream; norms are RMS
norms in groups; the embedding is multiplied by a constant; and a run of neighbouring layers may be gone through several
times with the same weights, each pass with a cache of its own, the stream being replaced before every pass (the first
too) by a linear map of itself and the embedding's output plus a vector of the pass.

``attention``    q and k only: a value head is its key head straight out of the product, untouched; q and k normed across
                 all their heads together with a weight, then rotated (a head's first ``rot.dims`` elements in two halves); a
                 row sees the keys of its own block of ``mask.size`` positions; softmax with a one in the denominator.
``attention_2``  q, k, v with biases; rotation with frequencies scaled by wavelength (``rot.scaling``); q and k divided by their
                 root mean square a head after the rotation, the values too; scores capped by ``softcap`` tanh(s / softcap); a
                 window of the last ``mask.size`` keys; the weight of a key is sigmoid(score + ``pb``[head]), no softmax.

config.json keys: ``vocab``, ``width``, ``norm.eps``, ``norm.groups``, ``embedding.scale``, ``loop`` (``start``, ``stop``,
``times``; optional) and ``layers``, a list of ``{"type": "attention" | "attention_2", "mixer": {...}, "mlp": {...} | null}``.
A mixer names ``heads``, ``kv_heads``, ``dim``, ``vdim``, ``scale``, ``mask.size`` (absent: every key), ``rot`` (``base``,
``dims``, and for ``attention_2`` ``scaling``: ``factor``, ``low``, ``high``, ``original``; absent: no rotation) and, for
``attention_2``, ``softcap`` (absent: none).  A feed-forward is ``{"kind": "moe", "expert": {"ff"}, "router": {"experts",
"top", "scale"}, "shared": {"ff"} | null}``.
Tensor names: ``embed``, ``head``, ``final.norm``, ``loop.in``, ``loop.step``, and for layer i ``l<i>.norm1``, ``l<i>.norm2``,
``l<i>.ls1``, ``l<i>.ls2``, ``l<i>.mix.{q,k,o}`` with ``q.norm``, ``k.norm`` (``attention``) or ``v``, ``q.b``, ``k.b``, ``v.b``,
``pb`` (``attention_2``), ``l<i>.mlp.{router,correction,e<j>.{up,down},shared.{up,down}}``.
"""
from __future__ import annotations

import dataclasses
from typing import Any, Dict, List, Optional, Tuple

from ..errors import ConfigError
from .base import ModelConfig, field_from_json
from .milenex import _number, _object
from .registry import Architecture, register_architecture

_MIXER_TYPES = ("attention", "attention_2")
_MIXER_KEYS = ("heads", "kv_heads", "dim", "vdim", "scale")


def _mask(where: str, m: Dict[str, Any]) -> int:
    mask = _object(where, m, "mask", required=False)
    return _number(where + ".mask", mask, "size") if mask is not None else 0


def _rotation(where: str, m: Dict[str, Any], scaled: bool):
    """The mixer's ``rot`` as the parameters of a rotary part with the rotate-half pairing (None: nothing is turned)."""
    rot = _object(where, m, "rot", required=False)
    if rot is None:
        return None
    dims = _number(where + ".rot", rot, "dims")
    if dims == 0:
        return None
    out = dict(theta=_number(where + ".rot", rot, "base", integer=False), dim=dims)
    scaling = _object(where + ".rot", rot, "scaling", required=False) if scaled else None
    if scaling is not None:
        out["scaling"] = {k: _number(where + ".rot.scaling", scaling, k, integer=False) for k in ("factor", "low", "high", "original")}
    return out


def _experts(where: str, mlp: Dict[str, Any]) -> Dict[str, Any]:
    """The parameters of a routed feed-forward from a ``moe`` entry."""
    expert, router = _object(where, mlp, "expert"), _object(where, mlp, "router")
    shared = _object(where, mlp, "shared", required=False)
    return dict(experts=_number(where + ".router", router, "experts"), top=_number(where + ".router", router, "top"),
                route_scale=_number(where + ".router", router, "scale", integer=False) if "scale" in router else 1.0,
                intermediate_size=_number(where + ".expert", expert, "ff"),
                shared_size=_number(where + ".shared", shared, "ff") if shared is not None else 0,
                router="sigmoid", normalize=True, unit="gelu", shared_gate=False)


@dataclasses.dataclass
class LagusunConfig(ModelConfig):
    vocab_size: int = field_from_json("vocab")
    hidden_size: int = field_from_json("width")
    layers: List[Dict[str, Any]] = field_from_json("layers")
    norm: Dict[str, Any] = field_from_json("norm")
    embedding: Optional[Dict[str, Any]] = field_from_json("embedding", None)
    loop: Optional[Dict[str, Any]] = field_from_json("loop", None)
    max_seq_len: int = field_from_json("max_positions", 1 << 20)     # (nothing in the design bounds a position)

    def derive(self, raw: Dict[str, Any]) -> None:
        if not isinstance(self.norm, dict):
            raise ConfigError("config.json: 'norm' must be an object")
        self.norm_eps = _number("norm", self.norm, "eps", integer=False)
        self.norm_groups = _number("norm", self.norm, "groups") if "groups" in self.norm else 1
        if self.embedding is not None and not isinstance(self.embedding, dict):
            raise ConfigError("config.json: 'embedding' must be an object")
        self.embedding_scale = (_number("embedding", self.embedding, "scale", integer=False)
                                if self.embedding is not None and "scale" in self.embedding else 1.0)

    def validate(self) -> None:
        if self.vocab_size <= 0 or self.hidden_size <= 0 or self.max_seq_len <= 0:
            raise ConfigError(f"config.json: vocab {self.vocab_size} and width {self.hidden_size} must be positive")
        if self.norm_eps < 0 or self.norm_groups <= 0 or self.hidden_size % self.norm_groups:
            raise ConfigError(f"config.json: norm.eps {self.norm_eps} must not be negative, and norm.groups {self.norm_groups} "
                              f"must cut width {self.hidden_size} into equal parts")
        if not isinstance(self.layers, list) or not self.layers:
            raise ConfigError("config.json: 'layers' must be a list with at least one layer")
        for n, layer in enumerate(self.layers):
            where = f"layers[{n}]"
            if not isinstance(layer, dict) or layer.get("type") not in _MIXER_TYPES:
                raise ConfigError(f"config.json: {where}.type must be one of {list(_MIXER_TYPES)}, got "
                                  f"{layer.get('type') if isinstance(layer, dict) else layer!r}")
            m = _object(where, layer, "mixer")
            missing = [k for k in _MIXER_KEYS if k not in m]
            if missing:
                raise ConfigError(f"config.json: {where}.mixer lacks {', '.join(missing)}")
            for k in ("heads", "kv_heads", "dim", "vdim"):
                _number(where + ".mixer", m, k)
            _number(where + ".mixer", m, "scale", integer=False)
            _mask(where + ".mixer", m)
            _rotation(where + ".mixer", m, scaled=layer["type"] == "attention_2")
            if layer["type"] == "attention" and m["dim"] != m["vdim"]:
                raise ConfigError(f"config.json: {where}.mixer: the values are the keys, so vdim {m['vdim']} must be dim {m['dim']}")
            if m.get("softcap") is not None and _number(where + ".mixer", m, "softcap", integer=False) < 0:
                raise ConfigError(f"config.json: {where}.mixer.softcap must not be negative")
            mlp = layer.get("mlp")
            if mlp is not None:
                if not isinstance(mlp, dict) or mlp.get("kind") != "moe":
                    raise ConfigError(f"config.json: {where}.mlp must be null or of kind 'moe', got {mlp!r}")
                _experts(where + ".mlp", mlp)
        self.runs()

    def loop_range(self) -> Tuple[int, int, int]:
        """(start, stop, times) of the run of layers that is gone through several times; (0, 0, 1) without one."""
        if self.loop is None:
            return 0, 0, 1
        if not isinstance(self.loop, dict):
            raise ConfigError("config.json: 'loop' must be an object")
        start, stop, times = (_number("loop", self.loop, k) for k in ("start", "stop", "times"))
        if not (0 <= start <= stop <= len(self.layers)) or times < 1:
            raise ConfigError(f"config.json: loop {start}..{stop} x {times} does not fit {len(self.layers)} layers")
        return (start, stop, times) if start < stop else (0, 0, 1)

    def runs(self) -> List[Tuple[int, int, Optional[int]]]:
        """The order in which the layers run: (layer, pass, the number of the pass if the run begins one) for every run."""
        n = len(self.layers)
        start, stop, times = self.loop_range()
        out: List[Tuple[int, int, Optional[int]]] = [(i, 0, None) for i in range(start)]
        for turn in range(times if start < stop else 0):
            out += [(i, turn, turn if i == start else None) for i in range(start, stop)]
        return out + [(i, 0, None) for i in range(stop, n)]

    def to_dict(self) -> Dict[str, Any]:
        out = super().to_dict()
        for k in ("loop", "embedding"):
            if out.get(k) is None:
                out.pop(k, None)
        out["architecture"] = "Lagusun"
        return out


def describe_lagusun(cfg: LagusunConfig):
    """The layer stack as data: every layer a ``prenorm`` block with scaled sublayers; a layer that the loop runs several
    times is one layer with a schedule entry, and a cache stream, per pass; the entry that begins a pass says so."""
    from ..engine.spec import LayerSpec, ModelSpec, PartSpec, ScheduleEntry

    width, eps, groups = cfg.hidden_size, cfg.norm_eps, cfg.norm_groups

    def norm(prefix: str, name: str) -> "PartSpec":
        return PartSpec("rmsnorm", dict(size=width, eps=eps, groups=groups), prefix=prefix, rename={"weight": name})

    def scale(prefix: str, name: str):
        return "scale", PartSpec("layer_scale", dict(size=width), prefix=prefix, rename={"weight": name})

    layers = []
    for n, layer in enumerate(cfg.layers):
        p, m, where = f"l{n}.", layer["mixer"], f"layers[{n}].mixer"
        second = layer["type"] == "attention_2"
        rot = _rotation(where, m, scaled=second)
        sizes = dict(hidden_size=width, heads=int(m["heads"]), kv_heads=int(m["kv_heads"]), dim=int(m["dim"]), vdim=int(m["vdim"]),
                     scale=float(m["scale"]), eps=eps, position=PartSpec("rotary", rot) if rot is not None else None)
        if second:
            how = dict(bias=True, unit_norm=True, value_unit_norm=True, window=_mask(where, m), cap=float(m.get("softcap") or 0.0),
                       weights="sigmoid", sink=False)
        else:
            how = dict(values="keys", row_norm=True, block=_mask(where, m), sink="unit")
        extras = {"mixer_scale": scale(p, "ls1")}
        ffn = ffn_norm = None
        mlp = layer.get("mlp")
        if mlp is not None:
            ffn = PartSpec("routed_experts", dict(_experts(f"layers[{n}].mlp", mlp), hidden_size=width), prefix=p + "mlp.")
            ffn_norm = norm(p, "norm2")
            extras["ffn_scale"] = scale(p, "ls2")
        layers.append(LayerSpec(block="prenorm", mixer=PartSpec("sink_attention", dict(sizes, **how), prefix=p + "mix."), ffn=ffn,
                                mixer_norm=norm(p, "norm1"), ffn_norm=ffn_norm, extras=extras))
    start, stop, times = cfg.loop_range()
    return ModelSpec(
        vocab_size=cfg.vocab_size, hidden_size=width, max_seq_len=cfg.max_seq_len,
        embedding=PartSpec("embedding", dict(vocab_size=cfg.vocab_size, hidden_size=width, scale=cfg.embedding_scale),
                           rename={"weight": "embed"}),
        layers=layers,
        schedule=[ScheduleEntry(layer=i, cache=(i, turn), writes=True, reenter=begins) for i, turn, begins in cfg.runs()],
        final_norm=norm("final.", "norm"),
        head=PartSpec("lm_head", dict(vocab_size=cfg.vocab_size, hidden_size=width), rename={"weight": "head"}),
        reentry=PartSpec("stream_reentry", dict(hidden_size=width, passes=times), prefix="loop.") if start < stop else None,
    )


LAGUSUN = register_architecture(Architecture(name="Lagusun", model_type="lagusun", config_class=LagusunConfig,
                                             describe=describe_lagusun))
