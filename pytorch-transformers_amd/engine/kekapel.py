"""The Kekapel design as a list of parts: the builder registered for ``model_type: kekapel`` (a ``config.json`` that
says ``"architecture": "Kekapel"``).

Tokens enter as ``embed[token] * scale + pos[position]``, a 32-bit stream.  A layer is a ``SandwichBlock``: LayerNorms
with weight and bias in front of and behind the mixer and the feed-forward, each sublayer's normed output entering the
stream times ``residual_mult``.  The mixer is attention with normed query and key heads and no rotation, whose scores
are capped by a tanh and mixed over the heads by a learned matrix before the softmax, over a window of positions; the
feed-forward is dense with a PolyNorm activation, routed experts with a clamped gate and a softmax over the taken
experts' logits, or absent.  A run of layers may run several times in a row with the same weights: the run order names
the block again, with cache pages of its own for every pass, and in front of each pass the embedding's output (but for
the first pass) and a learned vector for the pass are added (``LoopEntry``).  The head is a matrix of its own on the
final LayerNorm's output.

Tensor names: ``embed``, ``pos``, ``loop.step``, ``final.norm`` (+ ``.b``), ``head``, and per layer i ``l<i>.norm1``,
``l<i>.norm1b``, ``l<i>.norm2``, ``l<i>.norm2b`` (each + ``.b`` for the bias), ``l<i>.mix.<name>``, ``l<i>.mlp.<name>``.

Storage per sequence: attention passes with equal kv heads, page head size and window share a page pool; of a layer
with a window a sequence holds the pages that its window still touches.
"""
from __future__ import annotations

from typing import Dict, List, Tuple

from ..config.kekapel import KekapelConfig
from ..config.registry import register
from ..parts import (Embedding, GatedAttentionMixer, LayerNorm, LoopEntry, NoPositions, OutputHead, PolyNormFeedForward,
                     RoutedFeedForward, SandwichBlock)
from .spec import CACHE_FULL, CACHE_WINDOW, CacheGroupSpec, LayerCall, ModelSpec

GATE_ALPHA = 1.702  # an expert's gate is g * sigmoid(1.702 g)


def _norm(name: str, cfg: KekapelConfig) -> LayerNorm:
    return LayerNorm(name, cfg.width, cfg.eps, weight_name=name, bias_name=name + ".b")


def _mixer(cfg: KekapelConfig, prefix: str, layer: dict):
    m = layer["mixer"]
    return GatedAttentionMixer(prefix, cfg.width, m["heads"], m["kv_heads"], m["dim"], m["vdim"], float(m["scale"]),
                               cfg.eps, NoPositions(), window=int((m.get("mask") or {}).get("size", 0)), v_norm=False,
                               gate=False, softcap=float(m.get("softcap") or 0.0), talk=True)


def _feed_forward(cfg: KekapelConfig, prefix: str, mlp: dict):
    if mlp["kind"] == "dense":
        return PolyNormFeedForward(prefix, cfg.width, mlp["ff"], cfg.eps)
    r = mlp["router"]
    # the softmax over the taken logits alone is the softmax over all of them, divided by the taken ones' sum
    return RoutedFeedForward(prefix, cfg.width, mlp["expert"]["ff"], r["experts"], r["top"], 1.0, score="softmax",
                             normalise=True, router_bias=True, gate=("clamped", GATE_ALPHA, float(mlp["expert"]["limit"])))


def build_kekapel(cfg: KekapelConfig) -> ModelSpec:
    H = cfg.width
    start, stop, times = cfg.loop_range()
    entry = LoopEntry("loop.step", times, H) if stop > start else None
    blocks = []
    for i, layer in enumerate(cfg.layers):
        p = f"l{i}"
        ffn = norm2 = norm2b = None
        if layer.get("mlp") is not None:
            ffn = _feed_forward(cfg, f"{p}.mlp", layer["mlp"])
            norm2, norm2b = _norm(f"{p}.norm2", cfg), _norm(f"{p}.norm2b", cfg)
        blocks.append(SandwichBlock(_mixer(cfg, f"{p}.mix", layer), ffn, _norm(f"{p}.norm1", cfg), _norm(f"{p}.norm1b", cfg),
                                    norm2, norm2b, cfg.residual_mult, loop_entry=entry if (entry and i == start) else None))
    order: List[LayerCall] = []
    groups: Dict[Tuple, List] = {}  # (kv heads, page head size, window) -> [name, passes so far]
    for i, loop_pass in cfg.run_order():
        mixer = blocks[i].mixer
        key = (mixer.kv_heads, mixer.frame, mixer.window)
        g = groups.setdefault(key, [f"kv{len(groups)}", 0])
        order.append(LayerCall(i, g[0], g[1], loop_pass=loop_pass))
        g[1] += 1
    cache_groups = [CacheGroupSpec(name, CACHE_WINDOW if window else CACHE_FULL, count, kv, frame, window=window or None)
                    for (kv, frame, window), (name, count) in groups.items()]
    return ModelSpec(
        config=cfg,
        embedding=Embedding("embed", cfg.vocab, H, weight_name="embed", scale=cfg.embedding_scale, position_name="pos",
                            max_positions=cfg.max_positions),
        blocks=blocks,
        order=order,
        final_norm=_norm("final.norm", cfg),
        head=OutputHead("head", cfg.vocab, H, None, weight_name="head"),
        cache_groups=cache_groups,
        keep_embedding_output=entry is not None and times > 1,
    )


register("kekapel", KekapelConfig, build_kekapel, exist_ok=True, aliases=("Kekapel",))
