"""The Nopuzen design as a list of parts: the builder registered for ``model_type: nopuzen`` (a ``config.json`` that
says ``"architecture": "Nopuzen"``).

A layer is a ``PostNormBlock``: the mixer and the feed-forward read the stream itself (kept in 32-bit), and a LayerNorm
with weight and bias stands on each one's output before it is added.  The mixer is attention over a cache of latents
(queries through a latent of their own, half-split rotation with a frequency ramp, softmax, an output gate element by
element), or attention with grouped heads (biases, normed heads, interleaved rotation, a learned number per head on the
scores, a cap, sigmoid weights with a learned bias per head in place of the softmax, a gate per head).  The
feed-forward is dense with an xIELU activation, or routed experts without gates (squared relu) chosen among the best
groups of experts by softmax scores that are not renormalised, plus a shared expert times a sigmoid gate; or absent.
The head is the embedding table on the final LayerNorm's output.

Tensor names: ``embed``, ``final.norm`` (+ ``.b``), and per layer i ``l<i>.norm1``, ``l<i>.norm2`` (each + ``.b``),
``l<i>.mix.<name>``, ``l<i>.mlp.<name>``.

Storage per sequence: latent layers with equal cache rows share a page pool without values; attention layers with equal
kv heads and page head size share a page pool.
"""
from __future__ import annotations

from typing import Dict, List, Tuple

from ..config.nopuzen import NopuzenConfig
from ..config.registry import register
from ..parts import (Embedding, GatedAttentionMixer, LatentAttentionMixer, LayerNorm, NoPositions, OutputHead,
                     PostNormBlock, RotaryPositions, RoutedFeedForward, XieluFeedForward)
from ..parts.positions import yarn_ramp_frequencies
from .spec import CACHE_FULL, CacheGroupSpec, LayerCall, ModelSpec

EXPERT_ACT = "relu2"  # an expert is down(relu(up h)^2)


def _norm(name: str, cfg: NopuzenConfig) -> LayerNorm:
    return LayerNorm(name, cfg.width, cfg.eps, weight_name=name, bias_name=name + ".b")


def _positions(rot, head_dim: int, pairing: str):
    if not rot:
        return NoPositions()
    dims, base = int(rot["dims"]), float(rot["base"])
    sc = rot.get("scaling")
    if not sc:
        return RotaryPositions(head_dim, base, rotary_dim=dims, pairing=pairing)
    table, mult = yarn_ramp_frequencies(dims, base, float(sc["factor"]), float(sc["original"]), float(sc["fast"]),
                                        float(sc["slow"]))
    return RotaryPositions(head_dim, base, attention_scaling=mult, inv_freq=table, rotary_dim=dims, pairing=pairing)


def _mixer(cfg: NopuzenConfig, prefix: str, layer: dict):
    m = layer["mixer"]
    if layer["type"] == "latent_attention":
        return LatentAttentionMixer(prefix, cfg.width, m["heads"], m["dim"], m["rot_dim"], m["vdim"], m["kv_rank"],
                                    float(m["scale"]), cfg.eps, _positions(m["rot"], m["rot_dim"], "half"),
                                    q_rank=m["q_rank"], gate=True)
    return GatedAttentionMixer(prefix, cfg.width, m["heads"], m["kv_heads"], m["dim"], m["vdim"], float(m["scale"]),
                               cfg.eps, _positions(m.get("rot"), m["dim"], "interleaved"), v_norm=False, gate=True,
                               softcap=float(m.get("softcap") or 0.0), bias=True, head_scale=True, weights="sigmoid",
                               gate_per_head=True)


def _feed_forward(cfg: NopuzenConfig, prefix: str, mlp: dict):
    if mlp["kind"] == "dense":
        return XieluFeedForward(prefix, cfg.width, mlp["ff"])
    r = mlp["router"]
    groups = r.get("groups")
    shared = mlp.get("shared")
    return RoutedFeedForward(prefix, cfg.width, mlp["expert"]["ff"], r["experts"], r["top"], float(r["scale"]),
                             score="softmax", normalise=False, act=EXPERT_ACT, gated=False,
                             groups=(groups["count"], groups["keep"]) if groups else None,
                             shared_ff=int(shared["ff"]) if shared else 0, shared_gate=bool(shared))


def build_nopuzen(cfg: NopuzenConfig) -> ModelSpec:
    H = cfg.width
    blocks, order = [], []
    groups: Dict[Tuple, List] = {}  # what a layer keeps -> [name, layers so far]
    for i, layer in enumerate(cfg.layers):
        p = f"l{i}"
        mixer = _mixer(cfg, f"{p}.mix", layer)
        ffn = norm2 = None
        if layer.get("mlp") is not None:
            ffn, norm2 = _feed_forward(cfg, f"{p}.mlp", layer["mlp"]), _norm(f"{p}.norm2", cfg)
        # (the last layer's last norm and addition ride in the final norm's launch)
        blocks.append(PostNormBlock(mixer, ffn, _norm(f"{p}.norm1", cfg), norm2, hand_on_unformed=i == len(cfg.layers) - 1))
        if isinstance(mixer, LatentAttentionMixer):
            key = ("latent", 1, mixer.cache_row)
        else:
            key = ("kv", mixer.kv_heads, mixer.frame)
        g = groups.setdefault(key, [f"{key[0]}{len(groups)}", 0])
        order.append(LayerCall(i, g[0], g[1]))
        g[1] += 1
    cache_groups = [CacheGroupSpec(name, CACHE_FULL, count, heads, size, values=(kind == "kv"))
                    for (kind, heads, size), (name, count) in groups.items()]
    return ModelSpec(
        config=cfg,
        embedding=Embedding("embed", cfg.vocab, H, weight_name="embed"),
        blocks=blocks,
        order=order,
        final_norm=_norm("final.norm", cfg),
        head=OutputHead("head", cfg.vocab, H, "embed"),
        cache_groups=cache_groups,
    )


register("nopuzen", NopuzenConfig, build_nopuzen, exist_ok=True, aliases=("Nopuzen",))
