"""Mixing the residual streams of earlier layers into the one that goes on.

``DepthMix``: with X_0 the embedding's output and X_(j+1) what layer j leaves, the stream that goes on after
layer i is ``sum_j a[j] X_j`` over j = 0 .. i + 1, with one learned weight per earlier stream.  The streams of a
step are kept in one 32-bit buffer ``[layers + 1, tokens, features]`` (``StreamHistory``) that the blocks hand on
from one to the next; the sum is one pass over the planes filled so far, added in the order of j.
"""
from __future__ import annotations

from typing import Dict, List, Optional

import torch

from .. import ops
from ..engine.spec import INIT_ONE_NOISE, INIT_ZERO_NOISE, VECTOR, TensorSpec
from .base import Part, register_part


class StreamHistory:
    """The streams X_0 .. X_L of one step, ``planes[j]`` each, and how many are filled."""

    def __init__(self, depth: int, tokens: int, features: int, device):
        self.planes = torch.empty((depth + 1, tokens, features), dtype=torch.float32, device=device)
        self.filled = 0

    def next_plane(self) -> torch.Tensor:
        """The plane that the next stream is to be written into (by the kernel that forms it)."""
        if self.filled >= self.planes.shape[0]:
            raise RuntimeError("the stream history holds more layers than the model said it has")
        self.filled += 1
        return self.planes[self.filled - 1]


class DepthMix(Part):
    """The weights ``[index + 2]`` of the streams X_0 .. X_(index + 1) after layer ``index`` of ``depth`` layers.
    ``name`` is the tensor's name in the file as it stands."""

    def __init__(self, name: str, index: int, depth: int):
        if not (0 <= index < depth):
            raise ValueError(f"{name}: layer {index} of {depth}")
        self.name, self.index, self.depth = name, int(index), int(depth)
        self.weight: Optional[torch.Tensor] = None

    def tensor_specs(self) -> List[TensorSpec]:
        return [TensorSpec(self.name, (self.index + 2,), VECTOR, INIT_ONE_NOISE)]

    def load(self, tensors: Dict[str, torch.Tensor]) -> None:
        self.weight = tensors[self.name]

    def new_history(self, tokens: int, features: int, device) -> StreamHistory:
        return StreamHistory(self.depth, tokens, features, device)

    def fused(self, history: StreamHistory):
        """What ``ops.rmsnorm(mix=...)`` needs to form this sum in the launch that fills the last stream."""
        if history.filled != self.index + 2:
            raise RuntimeError(f"{self.name}: {history.filled} streams are filled, layer {self.index} mixes {self.index + 2}")
        return (history.planes, self.weight, history.filled)

    def forward(self, history: StreamHistory, dtype: torch.dtype):
        """``(narrow, wide)`` of the weighted sum of the streams filled so far, which must be X_0 .. X_(index + 1)."""
        if history.filled != self.index + 2:
            raise RuntimeError(f"{self.name}: {history.filled} streams are filled, layer {self.index} mixes {self.index + 2}")
        return ops.depth_mix(history.planes, self.weight, history.filled, dtype)


class LoopEntry(Part):
    """What a run of layers that runs ``times`` times in a row with the same weights adds to the stream in front of
    each pass t = 0, 1, ...: the embedding's output again (in front of every pass but the first; ``again=False``:
    never), then row t of a learned table ``[times, features]`` (``name`` is its name in the file as it stands).  The
    model keeps the embedding's 32-bit output for the step (``ModelSpec.keep_embedding_output``) in
    ``ctx.extras["embedding_output"]``; the block that a pass starts with adds the terms in its first launch."""

    def __init__(self, name: str, times: int, features: int, again: bool = True):
        if times < 1:
            raise ValueError(f"{name}: a loop of {times} passes")
        self.name, self.times, self.features, self.again = name, int(times), int(features), bool(again)
        self.steps: Optional[torch.Tensor] = None

    def tensor_specs(self) -> List[TensorSpec]:
        return [TensorSpec(self.name, (self.times, self.features), VECTOR, INIT_ZERO_NOISE)]

    def load(self, tensors: Dict[str, torch.Tensor]) -> None:
        self.steps = tensors[self.name]

    def terms(self, t: int, ctx):
        """``(tensor or None, vector)`` to add in front of pass ``t``, both 32-bit."""
        if not (0 <= t < self.times):
            raise RuntimeError(f"{self.name}: pass {t} of {self.times}")
        add = None
        if self.again and t > 0:
            add = ctx.extras.get("embedding_output")
            if add is None:
                raise RuntimeError(f"{self.name}: the model did not keep the embedding's output for the step")
        return add, self.steps[t]


register_part("stream", "loop_entry", LoopEntry)
register_part("stream", "depth_mix", DepthMix)
