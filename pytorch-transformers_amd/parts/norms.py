"""Norms.  ``LayerNorm``: mean and biased variance over the features, affine always
(``torch.nn.LayerNorm`` as built at src/transformers/models/falcon/modeling_falcon.py:603-612, :843)."""
from __future__ import annotations

from typing import Dict, List, Optional

import torch

from .. import ops
from ..engine.spec import INIT_ONE_NOISE, INIT_ZERO_NOISE, VECTOR, TensorSpec
from .base import Part, ResidualSum, register_part


class LayerNorm(Part):
    def __init__(self, name: str, hidden_size: int, eps: float, weight_name: Optional[str] = None,
                 bias_name: Optional[str] = None):
        """``weight_name``, ``bias_name``: the two vectors' names in the file as they stand (default ``name.weight``,
        ``name.bias``)."""
        self.name = name
        self.hidden_size = hidden_size
        self.eps = float(eps)
        self.weight_name, self.bias_name = weight_name or name + ".weight", bias_name or name + ".bias"
        self.weight: Optional[torch.Tensor] = None
        self.bias: Optional[torch.Tensor] = None

    def tensor_specs(self) -> List[TensorSpec]:
        return [TensorSpec(self.weight_name, (self.hidden_size,), VECTOR, INIT_ONE_NOISE),
                TensorSpec(self.bias_name, (self.hidden_size,), VECTOR, INIT_ZERO_NOISE)]

    def load(self, tensors: Dict[str, torch.Tensor]) -> None:
        self.weight = tensors[self.weight_name]
        self.bias = tensors[self.bias_name]

    def affine(self):
        """(weight, bias), for a launch that applies this norm beside other work (``ops.layernorm_stream``)."""
        return self.weight, self.bias

    def apply(self, y: torch.Tensor, dtype: torch.dtype, *, residual: Optional[torch.Tensor] = None, mult: float = 1.0,
              want_wide: bool = True, out_wide=None, mix=None):
        """This norm on a sublayer's output ``y`` (compute type), times ``mult``, added to the 32-bit stream
        ``residual``: ``(the new stream in dtype, the new stream in 32-bit)``, one launch (the interface of
        ``RMSNorm.apply`` as far as a block whose norms stand on the sublayers' outputs uses it)."""
        if out_wide is not None or mix is not None:
            raise ValueError(f"{self.name}: a LayerNorm on a sublayer's output writes a stream of its own and mixes none")
        if dtype == torch.float32:  # the stream is its own copy in the compute type
            wide = ops.layernorm_stream(dtype, x=residual, y=y, post=self.affine(), mult=mult, eps=self.eps)[1]
            return wide, wide
        return ops.layernorm_stream(dtype, x=residual, y=y, post=self.affine(), mult=mult, eps=self.eps, want_wide=want_wide,
                                    want_narrow=True)

    def forward_wide(self, x, rows: Optional[torch.Tensor] = None) -> torch.Tensor:
        """The norm of a stream held in 32-bit (a ``WideResidual``), in its compute type.  A stream whose last
        sublayer is still to be normed and added (``PendingNormSum``) has that done in the same launch."""
        from .base import PendingNormSum

        dtype = getattr(x, "dtype", None) or x.narrow.dtype
        if isinstance(x, PendingNormSum) and not x.formed and x.eps == self.eps:
            return ops.layernorm_stream(dtype, pre=self.affine(), eps=self.eps, rows=rows, want_wide=False,
                                        **x.launch_terms())[0]
        return ops.layernorm_stream(dtype, x=x.wide, pre=self.affine(), eps=self.eps, rows=rows, want_wide=False)[0]

    def _wide_loads(self, x: torch.Tensor) -> bool:
        # bfloat16 rows of a width the sixteen-byte kernel takes: the one that also forms residual sums
        return x.dtype == torch.bfloat16 and ops.layernorm_sum_ok(self.hidden_size)

    def forward(self, x: torch.Tensor, rows: Optional[torch.Tensor] = None) -> torch.Tensor:
        if self._wide_loads(x):
            return ops.layernorm_sum([x], self.hidden_size, w=self.weight, b=self.bias, eps=self.eps, rows=rows,
                                     want_x=False)[1]
        return ops.layernorm(x, self.weight, self.bias, self.eps, rows=rows)

    def forward_pair(self, x: torch.Tensor, other: "Part"):
        """``(self(x), other(x))``; one pass over x when both are LayerNorms with one eps."""
        if isinstance(other, LayerNorm) and other.eps == self.eps:
            if self._wide_loads(x):
                return ops.layernorm_sum([x], self.hidden_size, w=self.weight, b=self.bias, eps=self.eps,
                                         w2=other.weight, b2=other.bias, want_x=False)[1:]
            return ops.layernorm(x, self.weight, self.bias, self.eps, w2=other.weight, b2=other.bias)
        return self.forward(x), other.forward(x)


    def forward_sum(self, total: ResidualSum, rows: Optional[torch.Tensor] = None, other: Optional["Part"] = None,
                    want_x: bool = True):
        """``(x, self(x), other(x))`` for the unformed sum ``total``: x is formed, rounded and normalised in
        one pass.  Falls back to forming the sum first where the fused kernel does not take the width."""
        pair = isinstance(other, LayerNorm) and other.eps == self.eps
        if total.features == self.hidden_size and ops.layernorm_sum_ok(self.hidden_size) and (other is None or pair):
            return ops.layernorm_sum(total.kernel_terms(), self.hidden_size, w=self.weight, b=self.bias, eps=self.eps,
                                     w2=other.weight if pair else None, b2=other.bias if pair else None, rows=rows,
                                     want_x=want_x)
        x = total.tensor()
        if other is None:
            return x, self.forward(x, rows=rows), None
        a, m = self.forward_pair(x, other)
        return x, a, m


class RMSNorm(Part):
    """``x / sqrt(mean(x^2) + eps) * (offset + w)`` in 32-bit, eps inside the root.  ``offset`` 1 is for a gain that
    is stored around zero, 0 for one stored as it is applied.  With ``groups`` > 1 a row is cut into that many equal
    parts, each divided by its own root mean square.  ``name`` is the weight's name in the file as it stands.

    The input may be 32-bit in a model whose compute type is narrower (a residual stream kept wide); the result
    comes in the compute type, and on request in 32-bit as well (``apply``)."""

    def __init__(self, name: str, size: int, eps: float, offset: float = 0.0, groups: int = 1):
        if groups < 1 or size % groups:
            raise ValueError(f"{name}: {size} features do not split into {groups} equal groups")
        self.name, self.size, self.eps, self.offset, self.groups = name, int(size), float(eps), float(offset), int(groups)
        self.weight: Optional[torch.Tensor] = None

    def tensor_specs(self) -> List[TensorSpec]:
        return [TensorSpec(self.name, (self.size,), VECTOR, INIT_ZERO_NOISE if self.offset else INIT_ONE_NOISE)]

    def load(self, tensors: Dict[str, torch.Tensor]) -> None:
        self.weight = tensors[self.name]

    def apply(self, x: torch.Tensor, dtype: torch.dtype, **how):
        """``ops.rmsnorm`` with this norm's weight and constants: ``(narrow, wide)``."""
        return ops.rmsnorm(x, self.weight, self.eps, dtype, offset=self.offset, groups=self.groups, **how)

    def forward(self, x: torch.Tensor, rows: Optional[torch.Tensor] = None) -> torch.Tensor:
        return self.apply(x, x.dtype, rows=rows)[0]

    def forward_wide(self, x, rows: Optional[torch.Tensor] = None) -> torch.Tensor:
        """The norm of a ``WideResidual``'s 32-bit side, in its compute type."""
        dtype = getattr(x, "dtype", None) or x.narrow.dtype  # (a sum that is not formed says its compute type itself)
        return self.apply(x.wide, dtype, rows=rows)[0]


register_part("norm", "layernorm", LayerNorm)
register_part("norm", "rmsnorm", RMSNorm)
