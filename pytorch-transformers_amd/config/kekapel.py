"""Typed configuration of the Kekapel design: a decoder whose layers are listed one by one in ``config.json``, each an
attention mixer whose scores are capped and mixed over the heads before the softmax, with a window, and a feed-forward
(dense with a PolyNorm activation, routed experts with a clamped gate, or none); a norm stands in front of and behind
every sublayer; tokens get a scaled embedding plus a learned position vector; a run of layers may run several times in
a row with the same weights, with the embedding's output and a learned vector added in front of the passes.

Keys of ``config.json``: ``architecture`` ("Kekapel"), ``vocab``, ``width``, ``max_positions``, ``embedding``
(``{"scale"}``), ``norm`` (``{"eps"}``), ``residual_mult``, ``layers`` (a list of ``{"type", "mixer": {...}, "mlp":
{...} or null}``), ``loop`` (``{"start", "stop", "times"}`` or absent).

Mixer ``attention``: ``heads``, ``kv_heads``, ``dim``, ``vdim``, ``scale``, ``softcap`` (absent or 0: none), ``mask``
(``{"size"}``: a token sees itself and the ``size - 1`` positions before it; absent: every position before it).
``mlp``: ``{"kind": "dense", "ff"}`` or ``{"kind": "moe", "expert": {"ff", "limit"}, "router": {"experts", "top"}}``.

Every size and constant is read from there (or, by the weight loader, checked against the tensors' shapes).
"""
from __future__ import annotations

import dataclasses
from typing import Any, ClassVar, Dict, List, Optional

from .base import ConfigError, ModelConfig
from .bimepel import _number, _positive_int

MIXER_KEYS = {"attention": ("heads", "kv_heads", "dim", "vdim", "scale")}
MLP_KINDS = ("dense", "moe")


@dataclasses.dataclass
class KekapelConfig(ModelConfig):
    model_type: ClassVar[str] = "kekapel"

    architecture: str = "Kekapel"
    vocab: int = 512
    width: int = 256
    max_positions: int = 2048
    embedding: Dict[str, Any] = dataclasses.field(default_factory=lambda: {"scale": 1.0})
    layers: List[Dict[str, Any]] = dataclasses.field(default_factory=list)
    loop: Optional[Dict[str, Any]] = None
    norm: Dict[str, Any] = dataclasses.field(default_factory=lambda: {"eps": 1e-5})
    residual_mult: float = 1.0
    tie_word_embeddings: bool = False
    initializer_range: float = 0.05

    @property
    def vocab_size(self) -> int:
        return self.vocab

    @property
    def eps(self) -> float:
        return float(self.norm["eps"])

    @property
    def embedding_scale(self) -> float:
        return float(self.embedding["scale"])

    @property
    def max_position_embeddings(self) -> int:
        return self.max_positions

    def loop_range(self):
        """``(start, stop, times)`` of the run of layers that runs several times; an empty run if there is none."""
        if not self.loop:
            return 0, 0, 1
        return int(self.loop["start"]), int(self.loop["stop"]), int(self.loop["times"])

    def run_order(self):
        """``(layer, pass or None)`` in the order the layers run: those of the loop ``times`` times in a row; the pass's
        number stands at the pass's first layer."""
        n = len(self.layers)
        a, b, t = self.loop_range()
        out = [(i, None) for i in range(a)]
        for p in range(t):
            out += [(i, p if i == a else None) for i in range(a, b)]
        return out + [(i, None) for i in range(b, n)]

    def validate(self) -> None:
        me = dataclasses.asdict(self)
        for key in ("vocab", "width", "max_positions"):
            _positive_int("config", me, key)
        _number("config", me, "residual_mult")
        if not isinstance(self.norm, dict) or "eps" not in self.norm:
            raise ConfigError("config: 'norm' must be an object with the key 'eps'")
        if not isinstance(self.embedding, dict):
            raise ConfigError("config: 'embedding' must be an object with the key 'scale'")
        _number("config.embedding", self.embedding, "scale")
        if not isinstance(self.layers, list) or not self.layers:
            raise ConfigError("config: 'layers' must list at least one layer")
        if self.loop:
            for key in ("start", "stop", "times"):
                v = self.loop.get(key) if isinstance(self.loop, dict) else None
                if isinstance(v, bool) or not isinstance(v, int) or v < 0:
                    raise ConfigError(f"config.loop: {key!r} must be an integer from 0, got {v!r}")
            if not (self.loop["start"] <= self.loop["stop"] <= len(self.layers)) or self.loop["times"] < 1:
                raise ConfigError(f"config.loop: layers {self.loop['start']} .. {self.loop['stop']} - 1 of "
                                  f"{len(self.layers)}, {self.loop['times']} times, is no run of layers")
        for i, layer in enumerate(self.layers):
            where = f"layers[{i}]"
            kind = layer.get("type") if isinstance(layer, dict) else None
            if kind not in MIXER_KEYS:
                raise ConfigError(f"{where}: type {kind!r} is not built; built: {', '.join(sorted(MIXER_KEYS))}")
            mixer = layer.get("mixer")
            if not isinstance(mixer, dict):
                raise ConfigError(f"{where}: 'mixer' must hold the mixer's sizes")
            missing = [k for k in MIXER_KEYS[kind] if k not in mixer]
            if missing:
                raise ConfigError(f"{where} ({kind}): the mixer lacks {', '.join(missing)}")
            for k in ("heads", "kv_heads", "dim", "vdim"):
                _positive_int(f"{where}.mixer", mixer, k)
            _number(f"{where}.mixer", mixer, "scale")
            if mixer["heads"] % mixer["kv_heads"]:
                raise ConfigError(f"{where}: {mixer['heads']} heads are no multiple of {mixer['kv_heads']} kv heads")
            if mixer.get("softcap") is not None and _number(f"{where}.mixer", mixer, "softcap") < 0:
                raise ConfigError(f"{where}.mixer: 'softcap' must not be negative")
            if mixer.get("mask") is not None:
                _positive_int(f"{where}.mixer.mask", mixer["mask"], "size")
            mlp = layer.get("mlp")
            if mlp is not None:
                if not isinstance(mlp, dict) or mlp.get("kind") not in MLP_KINDS:
                    raise ConfigError(f"{where}.mlp: kind {mlp.get('kind') if isinstance(mlp, dict) else mlp!r} is not "
                                      f"built; built: {', '.join(MLP_KINDS)}, or null for no feed-forward")
                if mlp["kind"] == "dense":
                    _positive_int(f"{where}.mlp", mlp, "ff")
                else:
                    _positive_int(f"{where}.mlp.expert", mlp.get("expert"), "ff")
                    _number(f"{where}.mlp.expert", mlp.get("expert"), "limit")
                    router = mlp.get("router")
                    for k in ("experts", "top"):
                        _positive_int(f"{where}.mlp.router", router, k)
                    if router["top"] > router["experts"]:
                        raise ConfigError(f"{where}.mlp.router: top {router['top']} of {router['experts']} experts")
