"""Typed configuration of the Nopuzen design: a decoder whose layers are listed one by one in ``config.json``, each with
the kind of its token mixer (``latent_attention``: attention over cached latents, queries through a latent of their
own, an output gate; or ``attention``: grouped heads with biases, normed and rotated queries and keys, capped scores
with a number per head, sigmoid weights in place of a softmax and a gate per head), that mixer's sizes and constants,
and its feed-forward (dense with an xIELU activation, routed experts with groups and a shared expert, or none).  A
LayerNorm with weight and bias stands on every sublayer's output.

Keys of ``config.json``: ``architecture`` ("Nopuzen"), ``vocab``, ``width``, ``norm`` (``{"eps"}``), ``layers`` (a
list of ``{"type", "mixer": {...}, "mlp": {...} or null}``).

Mixer ``latent_attention``: ``heads``, ``dim``, ``rot_dim``, ``vdim``, ``kv_rank``, ``q_rank``, ``scale``, ``rot``
(``{"base", "dims", "scaling": {"factor", "original", "fast", "slow"} or absent}``).  Mixer ``attention``: ``heads``,
``kv_heads``, ``dim``, ``vdim``, ``scale``, ``softcap`` (absent or 0: none), ``rot`` (``{"base", "dims"}``, with or
without ``scaling``; absent: no rotation).  ``mlp``: ``{"kind": "dense", "ff"}`` or ``{"kind": "moe", "expert": {"ff"},
"router": {"experts", "top", "scale", "groups": {"count", "keep"} or absent}, "shared": {"ff"} or absent}``.

Every size and constant is read from there (or, by the weight loader, checked against the tensors' shapes).
"""
from __future__ import annotations

import dataclasses
from typing import Any, ClassVar, Dict, List

from .base import ConfigError, ModelConfig
from .bimepel import _number, _positive_int

MIXER_KEYS = {
    "latent_attention": ("heads", "dim", "rot_dim", "vdim", "kv_rank", "q_rank", "scale", "rot"),
    "attention": ("heads", "kv_heads", "dim", "vdim", "scale"),
}
MLP_KINDS = ("dense", "moe")


def _check_rot(where: str, rot, most: int, what: str) -> None:
    if not isinstance(rot, dict) or "base" not in rot or "dims" not in rot:
        raise ConfigError(f"{where}.rot must give 'base' and 'dims'")
    _positive_int(f"{where}.rot", rot, "dims")
    if _number(f"{where}.rot", rot, "base") <= 0:
        raise ConfigError(f"{where}.rot: 'base' must be positive")
    if rot["dims"] % 2 or rot["dims"] > most:
        raise ConfigError(f"{where}.rot.dims ({rot['dims']}) must be even and at most {what} ({most})")
    sc = rot.get("scaling")
    if sc is not None:
        for k in ("factor", "original", "fast", "slow"):
            if _number(f"{where}.rot.scaling", sc, k) <= 0:
                raise ConfigError(f"{where}.rot.scaling: {k!r} must be positive")


@dataclasses.dataclass
class NopuzenConfig(ModelConfig):
    model_type: ClassVar[str] = "nopuzen"

    architecture: str = "Nopuzen"
    vocab: int = 512
    width: int = 256
    layers: List[Dict[str, Any]] = dataclasses.field(default_factory=list)
    norm: Dict[str, Any] = dataclasses.field(default_factory=lambda: {"eps": 1e-6})
    tie_word_embeddings: bool = True
    initializer_range: float = 0.05

    @property
    def vocab_size(self) -> int:
        return self.vocab

    @property
    def eps(self) -> float:
        return float(self.norm["eps"])

    def validate(self) -> None:
        me = dataclasses.asdict(self)
        for key in ("vocab", "width"):
            _positive_int("config", me, key)
        if not isinstance(self.norm, dict) or "eps" not in self.norm:
            raise ConfigError("config: 'norm' must be an object with the key 'eps'")
        if not isinstance(self.layers, list) or not self.layers:
            raise ConfigError("config: 'layers' must list at least one layer")
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
            _number(f"{where}.mixer", mixer, "scale")
            if kind == "latent_attention":
                for k in ("heads", "dim", "rot_dim", "vdim", "kv_rank", "q_rank"):
                    _positive_int(f"{where}.mixer", mixer, k)
                _check_rot(f"{where}.mixer", mixer["rot"], mixer["rot_dim"], "rot_dim")
            else:
                for k in ("heads", "kv_heads", "dim", "vdim"):
                    _positive_int(f"{where}.mixer", mixer, k)
                if mixer["heads"] % mixer["kv_heads"]:
                    raise ConfigError(f"{where}: {mixer['heads']} heads are no multiple of {mixer['kv_heads']} kv heads")
                if mixer.get("softcap") is not None and _number(f"{where}.mixer", mixer, "softcap") < 0:
                    raise ConfigError(f"{where}.mixer: 'softcap' must not be negative")
                if mixer.get("rot") is not None:
                    _check_rot(f"{where}.mixer", mixer["rot"], mixer["dim"], "dim")
            mlp = layer.get("mlp")
            if mlp is None:
                continue
            if not isinstance(mlp, dict) or mlp.get("kind") not in MLP_KINDS:
                raise ConfigError(f"{where}.mlp: kind {mlp.get('kind') if isinstance(mlp, dict) else mlp!r} is not "
                                  f"built; built: {', '.join(MLP_KINDS)}, or null for no feed-forward")
            if mlp["kind"] == "dense":
                _positive_int(f"{where}.mlp", mlp, "ff")
                continue
            _positive_int(f"{where}.mlp.expert", mlp.get("expert"), "ff")
            router = mlp.get("router")
            for k in ("experts", "top"):
                _positive_int(f"{where}.mlp.router", router, k)
            _number(f"{where}.mlp.router", router, "scale")
            can = router["experts"]
            groups = router.get("groups")
            if groups is not None:
                for k in ("count", "keep"):
                    _positive_int(f"{where}.mlp.router.groups", groups, k)
                if router["experts"] % groups["count"] or groups["keep"] > groups["count"]:
                    raise ConfigError(f"{where}.mlp.router: {router['experts']} experts do not form {groups['count']} equal "
                                      f"groups of which {groups['keep']} are kept")
                can = router["experts"] // groups["count"] * groups["keep"]
            if router["top"] > can:
                raise ConfigError(f"{where}.mlp.router: top {router['top']} of {can} experts that can be taken")
            if mlp.get("shared") is not None:
                _positive_int(f"{where}.mlp.shared", mlp["shared"], "ff")
