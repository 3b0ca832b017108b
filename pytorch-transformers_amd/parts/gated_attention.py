"""Attention with normed heads and an output gate.

With h the mixer's input, H query heads on G key/value heads, queries and keys of ``key_dim`` elements and values of
``value_dim``:

    q = W_q h, k = W_k h, v = W_v h                       (no biases)
    q, k <- head / sqrt(mean(head^2) + eps) * w_q | w_k    one weight [key_dim] for all heads, before the rotation
    q, k <- rotated by position                            (``positions``: any rotation the kernels take)
    v    <- head / sqrt(mean(head^2) + eps)                no weight; cached so
    score(i, j) = q_i . k_j * scale
    score <- softcap * tanh(score / softcap)               (``softcap`` > 0)
    score_h <- sum_g T[h, g] score_g                       (``talk``: a learned [H, H] matrix mixes the heads' scores)
    softmax over the keys j <= i that i sees:
        all of them, those of i's own block of ``chunk`` positions (blocks counted from the sequence's start),
        and / or the last ``window``
    out = W_o (heads side by side * sigmoid(W_g h))

Options beside these: ``bias`` (q, k, v and the output projection have biases, ``name.q.b`` and so on); ``head_scale`` (a
learned number per head, ``name.temp``, multiplies the head's scores before the cap); ``weights="sigmoid"`` (no softmax:
a seen key's weight is ``sigmoid(score + pb[h])`` with a learned number per head ``name.pb``, not normalised over the
keys); ``gate_per_head`` (the gate is one number a head, ``W_g`` has a row per head).

The four products of h run as one (``Linear.stacked``).  The cache pages hold heads of ``frame`` >= max(key_dim,
value_dim) elements, a size the attention kernels are built for; what lies past a head's own elements is zero, which
changes neither scores nor sums.  Norms, angles, scores and the softmax are 32-bit.
"""
from __future__ import annotations

from typing import Dict, List, Optional, Sequence

import torch

from .. import ops
from ..engine.spec import INIT_EYE_NOISE, INIT_ONE_NOISE, INIT_ZERO_NOISE, VECTOR, TensorSpec
from .base import Part, StepContext, register_part
from .linear import Linear
from .positions import as_rotation


def attention_frame(key_dim: int, value_dim: int) -> int:
    """The head size of the cache pages for keys of ``key_dim`` and values of ``value_dim`` elements: the next size
    the matrix-core attention is built for (multiples of 16 up to 128, and 256)."""
    d = max(int(key_dim), int(value_dim))
    return (d + 15) // 16 * 16 if d <= 128 else 256


class GatedAttentionMixer(Part):
    def __init__(self, name: str, hidden_size: int, num_heads: int, kv_heads: int, key_dim: int, value_dim: int,
                 scale: float, eps: float, positions: Part, chunk: int = 0, window: int = 0, qk_norm: bool = True,
                 v_norm: bool = True, gate: bool = True, softcap: float = 0.0, talk: bool = False, bias: bool = False,
                 head_scale: bool = False, weights: str = "softmax", gate_per_head: bool = False):
        if num_heads % kv_heads:
            raise ValueError(f"{name}: heads ({num_heads}) must be a multiple of kv heads ({kv_heads})")
        self.name, self.hidden_size = name, int(hidden_size)
        self.num_heads, self.kv_heads, self.key_dim, self.value_dim = int(num_heads), int(kv_heads), int(key_dim), int(value_dim)
        self.scale, self.eps, self.positions = float(scale), float(eps), positions
        self.chunk, self.window = int(chunk), int(window)
        self.qk_norm, self.v_norm, self.gate = bool(qk_norm), bool(v_norm), bool(gate)
        self.softcap, self.talk = float(softcap), bool(talk)
        if weights not in ops.WEIGHTS_CODES:
            raise ValueError(f"{name}: attention weights of kind {weights!r} are not built; built: {sorted(ops.WEIGHTS_CODES)}")
        self.bias, self.head_scale, self.weights, self.gate_per_head = bool(bias), bool(head_scale), weights, bool(gate_per_head)
        self.talk_w: Optional[torch.Tensor] = None
        self.temp = self.head_bias = None
        self.frame = attention_frame(key_dim, value_dim)
        bare = lambda short, i, o, b=False: Linear(f"{name}.{short}", i, o, b, weight_name=f"{name}.{short}",
                                                   bias_name=f"{name}.{short}.b")
        self.q = bare("q", hidden_size, self.num_heads * self.key_dim, self.bias)
        self.k = bare("k", hidden_size, self.kv_heads * self.key_dim, self.bias)
        self.v = bare("v", hidden_size, self.kv_heads * self.value_dim, self.bias)
        self.g = bare("g", hidden_size, self.num_heads * (1 if self.gate_per_head else self.value_dim)) if self.gate else None
        self.out = bare("o", self.num_heads * self.value_dim, hidden_size, self.bias)
        self.q_w = self.k_w = None
        self.inp: Optional[Linear] = None

    def children(self) -> Sequence[Part]:
        return tuple(p for p in (self.q, self.k, self.v, self.g, self.out, self.positions) if p is not None)

    def tensor_specs(self) -> List[TensorSpec]:
        specs = []
        if self.qk_norm:
            specs += [TensorSpec(f"{self.name}.q.norm", (self.key_dim,), VECTOR, INIT_ONE_NOISE),
                      TensorSpec(f"{self.name}.k.norm", (self.key_dim,), VECTOR, INIT_ONE_NOISE)]
        if self.talk:
            specs.append(TensorSpec(f"{self.name}.talk", (self.num_heads, self.num_heads), VECTOR, INIT_EYE_NOISE))
        if self.head_scale:
            specs.append(TensorSpec(f"{self.name}.temp", (self.num_heads,), VECTOR, INIT_ONE_NOISE))
        if self.weights == "sigmoid":
            specs.append(TensorSpec(f"{self.name}.pb", (self.num_heads,), VECTOR, INIT_ZERO_NOISE))
        return specs

    def load(self, tensors: Dict[str, torch.Tensor]) -> None:
        if self.qk_norm:
            self.q_w, self.k_w = tensors[f"{self.name}.q.norm"], tensors[f"{self.name}.k.norm"]
        if self.talk:
            self.talk_w = tensors[f"{self.name}.talk"]
        if self.head_scale:
            self.temp = tensors[f"{self.name}.temp"]
        if self.weights == "sigmoid":
            self.head_bias = tensors[f"{self.name}.pb"]

    def after_load(self) -> None:
        self.inp = Linear.stacked(f"{self.name}.qkvg", [p for p in (self.q, self.k, self.v, self.g) if p is not None],
                                  pad_to=8, with_bias=self.bias)

    def check_sizes(self) -> None:
        rot = as_rotation(self.positions.rotation())
        problem = ops.attention_sizes_problem(self.num_heads, self.kv_heads, self.frame, False)
        if problem is None and max(self.key_dim, self.value_dim) > 256:
            problem = f"heads of {max(self.key_dim, self.value_dim)} elements are more than the 256 the kernels take"
        if problem is None and rot is not None:
            problem = ops.rotation_problem(self.key_dim, rot.rotary_dim, rot.pairing)
        if problem is None and (self.chunk < 0 or self.window < 0 or self.softcap < 0):
            problem = "chunk, window and softcap are 0 (none) or positive"
        if problem is None and self._talk_kernels():
            problem = ops.attn_talk_sizes_problem(self.num_heads, self.kv_heads, self.frame)
        if problem is not None:
            raise ValueError(f"{self.name}: {problem}")

    def _talk_kernels(self) -> bool:
        """Whether the scores pass through more than the plain kernels do (cap, mix, a number per head, weights that
        are no softmax): the kernels that own all heads of a token then run."""
        return bool(self.talk or self.softcap or self.head_scale or self.weights != "softmax")

    def input_projection(self):
        """The first product of ``forward``: a block may run it in one launch with another part's and hand the result
        in as ``projected``."""
        return self.inp, {}

    def forward(self, x: torch.Tensor, ctx: StepContext, call, residual: Optional[torch.Tensor] = None, projected=None):
        k_pool, v_pool = ctx.cache.kv_layer(call.cache_group, call.cache_layer)
        table = ctx.block_tables[call.cache_group]
        H, G, dk, dv = self.num_heads, self.kv_heads, self.key_dim, self.value_dim
        proj = projected if projected is not None else self.inp(x)
        at = [0, H * dk, (H + G) * dk, (H + G) * dk + G * dv]
        q = ops.head_norm_rope_cache(proj[:, at[0]:at[1]], proj[:, at[1]:at[2]], proj[:, at[2]:at[3]], self.q_w, self.k_w,
                                     self.eps, self.v_norm, as_rotation(self.positions.rotation()), ctx, table, k_pool,
                                     v_pool, H, G, dk, dv, write_cache=call.write_cache)
        if self._talk_kernels():
            o = ops.attention_talk(q, k_pool, v_pool, table, ctx, self.scale, talk=self.talk_w, softcap=self.softcap,
                                   window=self.window, chunk=self.chunk, head_scale=self.temp, head_bias=self.head_bias,
                                   weights=self.weights)
        else:
            o = ops.attention(q, k_pool, v_pool, table, ctx, None, self.scale, self.window, chunk=self.chunk)
        if self.gate:
            g_cols = H if self.gate_per_head else H * dv
            o = ops.gated_heads(o, self.frame, proj[:, at[3]:at[3] + g_cols], H, dv, x.dtype, per_head=self.gate_per_head)
        elif self.frame != dv:
            o = o.view(-1, H, self.frame)[:, :, :dv].reshape(-1, H * dv).contiguous()
        return self.out(o, add1=residual)


register_part("mixer", "gated_attention", GatedAttentionMixer)
