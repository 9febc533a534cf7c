"""Configuration of the Milenex decoder: a stack of pre-norm layers that each name their mixer -- ``attention`` (short
convolutions behind the projections, rotation of neighbouring pairs, unit-normed queries and keys, a window, a sink) or
``attention_2`` (no rotation: a penalty on distance, a window, a sink, heads that mix their weights, a gate per head) --
and a feed-forward, dense with the exact gelu or a mixture of clamped gated experts with a shared one, or none.  Every
mixer reads its input through a token shift; the norms' weights are stored around zero; a run of neighbouring layers may
be gone through several times with the same weights, each pass with a cache of its own, the embedding's output being
added to the stream before every pass but the first.

config.json keys: ``vocab``, ``width``, ``norm.eps``, ``loop`` (``start``, ``stop``, ``times``; optional) and ``layers``, a
list of ``{"type": "attention" | "attention_2", "mixer": {...}, "mlp": {...} | null}``.  A mixer names ``heads``,
``kv_heads``, ``dim``, ``vdim``, ``scale``, ``mask.size`` (absent: no window) and, for ``attention``, ``conv`` (taps; absent:
no convolution) and ``rot`` (``base``, ``dims``; absent: no rotation).  A feed-forward is ``{"kind": "dense", "ff": N}`` or
``{"kind": "moe", "expert": {"ff", "limit"}, "router": {"experts", "top", "groups": {"count", "keep"}},
"shared": {"ff", "limit"} | null}``.
Tensor names: ``embed``, ``head``, ``final.norm``, and for layer i ``l<i>.norm1``, ``l<i>.norm2``, ``l<i>.shift``,
``l<i>.mix.{q,k,v,o,sink}`` (``attention``: ``q.conv``, ``k.conv``, ``v.conv``; ``attention_2``: ``r1``, ``r2``, ``talk``, ``g``),
``l<i>.mlp.{up,down}`` or ``l<i>.mlp.{router,correction,e<j>.{gate,up,down},shared.{gate,up,down,sg}}``.
"""
from __future__ import annotations

import dataclasses
from typing import Any, Dict, List, Optional, Tuple

from ..errors import ConfigError
from .base import ModelConfig, field_from_json
from .registry import Architecture, register_architecture

_MIXER_TYPES = ("attention", "attention_2")
_MIXER_KEYS = ("heads", "kv_heads", "dim", "vdim", "scale")


def _number(where: str, d: Dict[str, Any], key: str, integer: bool = True):
    v = d.get(key)
    if isinstance(v, bool) or not isinstance(v, (int, float)) or (integer and int(v) != v):
        raise ConfigError(f"config.json: {where}.{key} must be {'an integer' if integer else 'a number'}, got {v!r}")
    return int(v) if integer else float(v)


def _object(where: str, d: Dict[str, Any], key: str, required: bool = True) -> Optional[Dict[str, Any]]:
    v = d.get(key)
    if v is None and not required:
        return None
    if not isinstance(v, dict):
        raise ConfigError(f"config.json: {where}.{key} must be an object, got {v!r}")
    return v


def _rotation(where: str, m: Dict[str, Any]):
    """The mixer's ``rot`` as the parameters of a rotary part that turns neighbouring pairs (None: nothing is turned)."""
    rot = _object(where, m, "rot", required=False)
    if rot is None:
        return None
    dims = _number(where + ".rot", rot, "dims")
    if dims == 0:
        return None
    return dict(theta=_number(where + ".rot", rot, "base", integer=False), dim=dims, pairing="neighbours")


def _window(where: str, m: Dict[str, Any]) -> int:
    mask = _object(where, m, "mask", required=False)
    return _number(where + ".mask", mask, "size") if mask is not None else 0


def _experts(where: str, mlp: Dict[str, Any]) -> Dict[str, Any]:
    """The parameters of a routed feed-forward from a ``moe`` entry."""
    expert, router = _object(where, mlp, "expert"), _object(where, mlp, "router")
    groups = _object(where + ".router", router, "groups", required=False)
    shared = _object(where, mlp, "shared", required=False)
    return dict(experts=_number(where + ".router", router, "experts"), top=_number(where + ".router", router, "top"),
                intermediate_size=_number(where + ".expert", expert, "ff"),
                limit=_number(where + ".expert", expert, "limit", integer=False),
                groups=_number(where + ".router.groups", groups, "count") if groups is not None else 1,
                keep=_number(where + ".router.groups", groups, "keep") if groups is not None else 1,
                shared_size=_number(where + ".shared", shared, "ff") if shared is not None else 0,
                shared_limit=_number(where + ".shared", shared, "limit", integer=False) if shared is not None else 0.0)


@dataclasses.dataclass
class MilenexConfig(ModelConfig):
    vocab_size: int = field_from_json("vocab")
    hidden_size: int = field_from_json("width")
    layers: List[Dict[str, Any]] = field_from_json("layers")
    norm: Dict[str, Any] = field_from_json("norm")
    loop: Optional[Dict[str, Any]] = field_from_json("loop", None)
    max_seq_len: int = field_from_json("max_positions", 1 << 20)     # (nothing in the design bounds a position)

    def derive(self, raw: Dict[str, Any]) -> None:
        if not isinstance(self.norm, dict):
            raise ConfigError("config.json: 'norm' must be an object")
        self.norm_eps = _number("norm", self.norm, "eps", integer=False)

    def validate(self) -> None:
        if self.vocab_size <= 0 or self.hidden_size <= 0 or self.max_seq_len <= 0:
            raise ConfigError(f"config.json: vocab {self.vocab_size} and width {self.hidden_size} must be positive")
        if self.norm_eps < 0:
            raise ConfigError(f"config.json: norm.eps {self.norm_eps} must not be negative")
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
            _window(where + ".mixer", m)
            if layer["type"] == "attention":
                _rotation(where + ".mixer", m)
                if m.get("conv") is not None and _number(where + ".mixer", m, "conv") < 0:
                    raise ConfigError(f"config.json: {where}.mixer.conv must not be negative")
            mlp = layer.get("mlp")
            if mlp is not None:
                if not isinstance(mlp, dict) or mlp.get("kind") not in ("dense", "moe"):
                    raise ConfigError(f"config.json: {where}.mlp must be null or of kind 'dense' or 'moe', got {mlp!r}")
                if mlp["kind"] == "dense":
                    _number(where + ".mlp", mlp, "ff")
                else:
                    _experts(where + ".mlp", mlp)
        self.runs()

    def runs(self) -> List[Tuple[int, int, bool]]:
        """The order in which the layers run: (layer, pass, whether the embedding's output is added to the stream right
        before it) for every run.  Layers ``start`` .. ``stop - 1`` are gone through ``times`` times in a row."""
        n = len(self.layers)
        if self.loop is None:
            return [(i, 0, False) for i in range(n)]
        if not isinstance(self.loop, dict):
            raise ConfigError("config.json: 'loop' must be an object")
        start, stop, times = (_number("loop", self.loop, k) for k in ("start", "stop", "times"))
        if not (0 <= start <= stop <= n) or times < 1:
            raise ConfigError(f"config.json: loop {start}..{stop} x {times} does not fit {n} layers")
        if start == stop:
            return [(i, 0, False) for i in range(n)]
        out = [(i, 0, False) for i in range(start)]
        for turn in range(times):
            out += [(i, turn, turn > 0 and i == start) for i in range(start, stop)]
        return out + [(i, 0, False) for i in range(stop, n)]

    def to_dict(self) -> Dict[str, Any]:
        out = super().to_dict()
        if out.get("loop") is None:
            out.pop("loop", None)
        out["architecture"] = "Milenex"
        return out


def describe_milenex(cfg: MilenexConfig):
    """The layer stack as data: every layer a ``prenorm`` block whose mixer reads through a token shift; a layer that the
    loop runs several times is one layer with a schedule entry, and a cache stream, per pass."""
    from ..engine.spec import LayerSpec, ModelSpec, PartSpec, ScheduleEntry

    width, eps = cfg.hidden_size, cfg.norm_eps

    def norm(prefix: str, name: str) -> "PartSpec":
        return PartSpec("rmsnorm", dict(size=width, eps=eps, offset=1.0), prefix=prefix, rename={"weight": name})

    layers = []
    for n, layer in enumerate(cfg.layers):
        p, m, where = f"l{n}.", layer["mixer"], f"layers[{n}].mixer"
        sizes = dict(hidden_size=width, heads=int(m["heads"]), kv_heads=int(m["kv_heads"]), dim=int(m["dim"]), vdim=int(m["vdim"]),
                     scale=float(m["scale"]), eps=eps, window=_window(where, m), sink=True)
        if layer["type"] == "attention":
            rot = _rotation(where, m)
            mixer = PartSpec("sink_attention", dict(sizes, conv_taps=int(m.get("conv") or 0), unit_norm=True,
                                                    position=PartSpec("rotary", rot) if rot is not None else None), prefix=p + "mix.")
        else:
            mixer = PartSpec("sink_attention", dict(sizes, distance=True, talking=True, head_gate=True), prefix=p + "mix.")
        ffn = ffn_norm = None
        mlp = layer.get("mlp")
        if mlp is not None:
            if mlp["kind"] == "dense":
                ffn = PartSpec("dense_gelu", dict(hidden_size=width, intermediate_size=int(mlp["ff"])), prefix=p + "mlp.")
            else:
                ffn = PartSpec("routed_experts", dict(_experts(f"layers[{n}].mlp", mlp), hidden_size=width), prefix=p + "mlp.")
            ffn_norm = norm(p, "norm2")
        extras = {"mixer_shift": ("conv", PartSpec("token_shift", dict(channels=width), prefix=p, rename={"weight": "shift"}))}
        layers.append(LayerSpec(block="prenorm", mixer=mixer, ffn=ffn, mixer_norm=norm(p, "norm1"), ffn_norm=ffn_norm, extras=extras))
    return ModelSpec(
        vocab_size=cfg.vocab_size, hidden_size=width, max_seq_len=cfg.max_seq_len,
        embedding=PartSpec("embedding", dict(vocab_size=cfg.vocab_size, hidden_size=width), rename={"weight": "embed"}),
        layers=layers,
        schedule=[ScheduleEntry(layer=i, cache=(i, turn), writes=True, add_embedding=add) for i, turn, add in cfg.runs()],
        final_norm=norm("final.", "norm"),
        head=PartSpec("lm_head", dict(vocab_size=cfg.vocab_size, hidden_size=width), rename={"weight": "head"}),
    )


MILENEX = register_architecture(Architecture(name="Milenex", model_type="milenex", config_class=MilenexConfig,
                                             describe=describe_milenex))
