"""Attention over a cache of latents: per token the cache holds one small vector c (``rank`` elements, the
RMS-normed first rows of a down-projection) and one rotated key part (``rot_dim`` elements, the rest of it) that
all heads share.  Per head the plain key is ``U_k c`` and the value ``U_v c``; the score of a query and a key is
``(q_plain . k_plain + q_rot . k_rot) * scale``, softmax over the causal keys, output projection on the heads' values.

The two expansions are moved to the query side (``csrc/attn_latent.hip``): every head's query becomes
``[U_k^T q_plain | q_rot]``, the attention runs over the cache rows as they lie, and ``U_v`` is applied to each
head's weighted sum of latents.  A step costs the same whether its keys were cached a step or a thousand steps ago,
and nothing but c and the rotated part is ever stored.

Options: the queries may themselves come through a latent (``q_rank``: ``q = W_uq (rmsnorm(W_dq h) * w)``, the file's
``dq``, ``dq.norm`` and ``uq`` in place of ``q``), and the heads' values side by side may be multiplied by ``sigmoid(W_g
h)`` element by element before the output projection (``gate``).
"""
from __future__ import annotations

from typing import Dict, List, Optional, Sequence

import torch

from .. import ops
from ..engine.spec import INIT_NORMAL, INIT_ONE_NOISE, MATRIX, VECTOR, TensorSpec
from .base import Part, StepContext, register_part
from .linear import Linear
from .positions import as_rotation


class LatentAttentionMixer(Part):
    def __init__(self, name: str, hidden_size: int, heads: int, dim: int, rot_dim: int, value_dim: int, rank: int,
                 scale: float, eps: float, positions: Part, q_rank: int = 0, gate: bool = False):
        """``dim`` / ``rot_dim``: plain and rotated elements of a head's query and key; ``positions`` says how the
        rotated part turns (a ``Rotation`` over ``rot_dim`` elements); ``q_rank`` > 0: the size of the queries' latent;
        ``gate``: an output gate ``name.g``."""
        self.name, self.hidden_size = name, int(hidden_size)
        self.heads, self.dim, self.rot_dim, self.value_dim, self.rank = int(heads), int(dim), int(rot_dim), int(value_dim), int(rank)
        self.scale, self.eps = float(scale), float(eps)
        self.positions = positions
        bare = lambda short, i, o: Linear(f"{name}.{short}", i, o, False, weight_name=f"{name}.{short}")
        self.q_rank, self.gate = int(q_rank), bool(gate)
        q_cols = self.heads * (self.dim + self.rot_dim)
        if self.q_rank:
            self.q_latent, self.q = bare("dq", hidden_size, self.q_rank), bare("uq", self.q_rank, q_cols)
        else:
            self.q_latent, self.q = None, bare("q", hidden_size, q_cols)
        self.down = bare("dkv", hidden_size, self.rank + self.rot_dim)
        self.g = bare("g", hidden_size, self.heads * self.value_dim) if self.gate else None
        self.out = bare("o", self.heads * self.value_dim, hidden_size)
        self.q_down: Optional[Linear] = None
        self.norm_w = self.q_norm_w = self.up_k = self.up_v = None

    @property
    def cache_row(self) -> int:
        """Elements the cache holds per token."""
        return self.rank + self.rot_dim

    def children(self) -> Sequence[Part]:
        return tuple(p for p in (self.q_latent, self.q, self.down, self.g, self.out, self.positions) if p is not None)

    def tensor_specs(self) -> List[TensorSpec]:
        n = self.name
        q_norm = [TensorSpec(f"{n}.dq.norm", (self.q_rank,), VECTOR, INIT_ONE_NOISE)] if self.q_rank else []
        return q_norm + [TensorSpec(f"{n}.dkv.norm", (self.rank,), VECTOR, INIT_ONE_NOISE),
                TensorSpec(f"{n}.uk", (self.heads * self.dim, self.rank), MATRIX, INIT_NORMAL),
                TensorSpec(f"{n}.uv", (self.heads * self.value_dim, self.rank), MATRIX, INIT_NORMAL)]

    def load(self, tensors: Dict[str, torch.Tensor]) -> None:
        n = self.name
        self.norm_w, self.up_k, self.up_v = tensors[f"{n}.dkv.norm"], tensors[f"{n}.uk"], tensors[f"{n}.uv"]
        self.q_norm_w = tensors[f"{n}.dq.norm"] if self.q_rank else None

    def after_load(self) -> None:
        # everything that reads the layer's input, as one product: [q or its latent | down-projection | gate]
        first = [p for p in (self.q_latent or self.q, self.down, self.g) if p is not None]
        self.q_down = Linear.stacked(f"{self.name}.q_dkv", first, pad_to=8)
        # per head, with a head's rows its inputs: the key expansion as the file has it, the value expansion turned
        self.k_side = self.up_k.view(self.heads, self.dim, self.rank)
        self.v_side = self.up_v.view(self.heads, self.value_dim, self.rank).transpose(1, 2).contiguous()

    def check_sizes(self) -> None:
        problem = ops.latent_sizes_problem(self.heads, self.dim, self.rot_dim, self.rank)
        rot = as_rotation(self.positions.rotation())
        if problem is None and rot is not None:
            if self.rot_dim == 0:
                problem = "a rotation needs a rotated part"
            else:
                problem = ops.rotation_problem(self.rot_dim, rot.rotary_dim, rot.pairing)
        if problem is not None:
            raise ValueError(f"{self.name}: {problem}")

    def forward(self, x: torch.Tensor, ctx: StepContext, call, residual: Optional[torch.Tensor] = None):
        k_pool, _ = ctx.cache.kv_layer(call.cache_group, call.cache_layer)
        table = ctx.block_tables[call.cache_group]
        rot = as_rotation(self.positions.rotation())
        proj = self.q_down(x)
        M, D, H = x.shape[0], self.cache_row, self.heads
        q_cols = H * (self.dim + self.rot_dim)
        if self.q_rank:  # the queries through their own latent: norm in 32-bit, then the second product
            lat_q = ops.rmsnorm(proj[:, :self.q_rank], self.q_norm_w, self.eps, x.dtype)[0]
            queries, at = self.q(lat_q), self.q_rank
        else:
            queries, at = proj[:, :q_cols], q_cols
        q_full = ops.latent_prep(proj[:, at:at + D], self.norm_w, self.eps, None if rot is None else rot.inv_freq,
                                 1.0 if rot is None else rot.scale, None if rot is None else rot.rotary_dim,
                                 "half" if rot is None else rot.pairing, ctx.token_pos, ctx.token_seq, table, k_pool,
                                 self.heads, self.dim, self.rot_dim, self.rank, write_cache=call.write_cache, q=queries)
        gate = proj[:, at + D:at + D + H * self.value_dim] if self.gate else None
        library = x.dtype == torch.bfloat16 and M > ops.HEAD_PROJECT_LIBRARY_ROWS
        # each head's plain query through the transpose of its key expansion: the first `rank` of its frame
        if library:
            plain = queries.unflatten(1, (H, self.dim + self.rot_dim))[:, :, :self.dim]
            q_full[:, :, :self.rank].copy_(ops.head_project_library(plain, self.k_side, torch.float32).transpose(0, 1))
        else:
            ops.head_project(queries, self.dim + self.rot_dim, self.k_side, H, self.dim, self.rank,
                             out=q_full.view(M, H * D), out_head=D)
        lat = ops.attn_latent(q_full, k_pool, table, ctx.token_seq, ctx.token_pos, self.rank, self.scale, ctx=ctx)
        if library:
            o = ops.head_project_library(lat.to(x.dtype), self.v_side).transpose(0, 1).reshape(M, H * self.value_dim)
        else:
            o = ops.head_project(lat.view(M, H * self.rank), self.rank, self.v_side, H, self.rank, self.value_dim,
                                 out_dtype=x.dtype)
        if gate is not None:
            o = ops.gated_heads(o, self.value_dim, gate, H, self.value_dim, x.dtype)
        return self.out(o, add1=residual)


register_part("mixer", "latent_attention", LatentAttentionMixer)
