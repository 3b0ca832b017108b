"""Feed-forward parts.  ``DenseFeedForward``: ``down(act(up(x)))``, no gate, no experts
(``FalconMLP`` src/transformers/models/falcon/modeling_falcon.py:565-578).  The activation is one of the
reference's by name (src/transformers/activations.py:200-220; ``gelu`` is the exact erf form, :59-78), applied
in 32-bit in the epilogue of the first product."""
from __future__ import annotations

from typing import Dict, List, Optional, Sequence

import torch

from .. import ops
from ..engine.spec import INIT_NORMAL, INIT_ONE_NOISE, INIT_ZERO_NOISE, MATRIX, VECTOR, TensorSpec
from .base import Part, StepContext, as_tensor, register_part
from .linear import Linear, PendingProjection


class DenseFeedForward(Part):
    def __init__(self, name: str, hidden_size: int, ffn_size: int, bias: bool, activation: str = "gelu",
                 up_name: str = "dense_h_to_4h", down_name: str = "dense_4h_to_h", bare_names: bool = False):
        """``bare_names``: the weight file holds the matrices as ``name.up_name`` and ``name.down_name`` themselves,
        with no ``.weight`` behind them."""
        if activation not in ops.ACT_CODES:
            raise ValueError(f"activation {activation!r} is not built; built: {sorted(k for k in ops.ACT_CODES if k)}")
        self.name = name
        self.activation = activation
        bare = (lambda n: n) if bare_names else (lambda n: None)
        self.up = Linear(f"{name}.{up_name}", hidden_size, ffn_size, bias, weight_name=bare(f"{name}.{up_name}"))
        self.down = Linear(f"{name}.{down_name}", ffn_size, hidden_size, bias, weight_name=bare(f"{name}.{down_name}"))

    def children(self) -> Sequence[Part]:
        return (self.up, self.down)

    can_defer = True

    def input_projection(self):
        """The first product of ``forward`` and how it is called (see ``AttentionMixer.input_projection``)."""
        return self.up, {"act": self.activation}

    def forward(self, x: torch.Tensor, ctx: StepContext, add1=None, add2=None, defer: bool = False, projected=None):
        """``down(act(up(x))) + add1 + add2``.  With ``defer`` the second product comes back not run
        (``PendingProjection``) and the caller sees to the additions."""
        h = projected if projected is not None else self.up(x, act=self.activation)
        if defer:
            return PendingProjection(self.down, h)
        return self.down(h, add1=as_tensor(add1), add2=as_tensor(add2))


class PolyNormFeedForward(Part):
    """``down(act(up(x)))`` without biases, with the activation PolyNorm: over a token's vector z of ``ffn_size`` values,
    ``a N(z) + b N(z^2) + c N(z^3) + e`` with powers element by element, ``N(v) = v / sqrt(mean(v^2) + eps)`` and four
    learned numbers (a, b, c, e).  The mean squares are 32-bit.  The file holds ``name.up``, ``name.down`` and the four
    numbers as ``name.act``."""

    def __init__(self, name: str, hidden_size: int, ffn_size: int, eps: float):
        self.name, self.eps, self.ffn_size = name, float(eps), int(ffn_size)
        self.up = Linear(f"{name}.up", hidden_size, ffn_size, False, weight_name=f"{name}.up")
        self.down = Linear(f"{name}.down", ffn_size, hidden_size, False, weight_name=f"{name}.down")
        self.coef: Optional[torch.Tensor] = None

    def children(self) -> Sequence[Part]:
        return (self.up, self.down)

    def tensor_specs(self) -> List[TensorSpec]:
        return [TensorSpec(f"{self.name}.act", (4,), VECTOR, INIT_ONE_NOISE)]

    def load(self, tensors: Dict[str, torch.Tensor]) -> None:
        self.coef = tensors[f"{self.name}.act"]

    def forward(self, x: torch.Tensor, ctx: StepContext, add1=None, add2=None):
        y = ops.polynorm(self.up(x), self.coef, self.eps)
        return self.down(y, add1=as_tensor(add1), add2=as_tensor(add2))


class XieluFeedForward(Part):
    """``down(act(up(x)))`` without biases, with the activation xIELU: with two learned numbers (p, q) and ``ap =
    softplus(p)``, ``an = 1/2 + softplus(q)``, element by element ``ap z^2 + z / 2`` for z > 0 and ``an (e^z - 1 - z) +
    z / 2`` else.  The two softplus and the activation are 32-bit.  The file holds ``name.up``, ``name.down`` and the two
    numbers as ``name.act``."""

    def __init__(self, name: str, hidden_size: int, ffn_size: int):
        self.name, self.ffn_size = name, int(ffn_size)
        self.up = Linear(f"{name}.up", hidden_size, ffn_size, False, weight_name=f"{name}.up")
        self.down = Linear(f"{name}.down", ffn_size, hidden_size, False, weight_name=f"{name}.down")
        self.coef: Optional[torch.Tensor] = None

    def children(self) -> Sequence[Part]:
        return (self.up, self.down)

    def tensor_specs(self) -> List[TensorSpec]:
        return [TensorSpec(f"{self.name}.act", (2,), VECTOR, INIT_ZERO_NOISE)]

    def load(self, tensors: Dict[str, torch.Tensor]) -> None:
        self.coef = tensors[f"{self.name}.act"]

    def forward(self, x: torch.Tensor, ctx: StepContext, add1=None, add2=None):
        y = ops.xielu(self.up(x), self.coef)
        return self.down(y, add1=as_tensor(add1), add2=as_tensor(add2))


class GatedFeedForward(Part):
    """A feed-forward with a gate: ``down(glu(gate(x), up(x)))``, no biases.  ``kind`` ``"silu"``: ``silu(gate) * up``;
    ``"clamped"``: with ``g = min(gate, limit)`` and ``u = clamp(up, -limit, limit)``, ``g * sigmoid(alpha * g) * (u +
    1)``.  The two input products run as one; the gate's arithmetic is 32-bit.  The file holds the matrices as
    ``name.gate``, ``name.up`` and ``name.down``."""

    def __init__(self, name: str, hidden_size: int, ffn_size: int, kind: str = "silu", alpha: float = 1.0,
                 limit: float = 0.0):
        if kind not in ops.GLU_CODES:
            raise ValueError(f"{name}: a gate of kind {kind!r} is not built; built: {sorted(ops.GLU_CODES)}")
        self.name, self.kind, self.alpha, self.limit = name, kind, float(alpha), float(limit)
        self.ffn_size = int(ffn_size)
        bare = lambda short, i, o: Linear(f"{name}.{short}", i, o, False, weight_name=f"{name}.{short}")
        self.gate = bare("gate", hidden_size, ffn_size)
        self.up = bare("up", hidden_size, ffn_size)
        self.down = bare("down", ffn_size, hidden_size)
        self.inp: Optional[Linear] = None

    def children(self) -> Sequence[Part]:
        return (self.gate, self.up, self.down)

    def after_load(self) -> None:
        self.inp = Linear.stacked(f"{self.name}.gate_up", [self.gate, self.up])

    def input_projection(self):
        """The first product of ``forward`` (see ``AttentionMixer.input_projection``)."""
        return self.inp, {}

    def forward(self, x: torch.Tensor, ctx: StepContext, add1=None, add2=None, projected=None):
        both = projected if projected is not None else self.inp(x)
        F = self.ffn_size
        y = ops.glu(both[:, :F], both[:, F:], self.kind, self.alpha, self.limit)
        return self.down(y, add1=as_tensor(add1), add2=as_tensor(add2))


def _stack_experts(experts: int, rows_each: Sequence[int]):
    """Pieces given expert by expert (each expert's matrices in turn) -> one tensor ``[experts, sum(rows), columns]``."""
    per = len(rows_each)

    def assemble(parts):
        return torch.stack([torch.cat(list(parts[e * per:(e + 1) * per]), dim=0) for e in range(experts)])

    return assemble


def _unstack_experts(rows_each: Sequence[int]):
    """The inverse of ``_stack_experts``: ``[experts, sum(rows), columns]`` -> the pieces, expert by expert."""

    def split(t):
        return [piece for e in range(t.shape[0]) for piece in torch.split(t[e], list(rows_each), dim=0)]

    return split


class RoutedFeedForward(Part):
    """A feed-forward of ``experts`` small gated feed-forwards of which each token uses ``top``:

        z = W_router x (32-bit), s = sigmoid(z) (or softmax(z)); the ``top`` largest s are taken;
        weight_e = s_e / (sum of the taken s + 1e-20) * scale     (``normalise=False``: s_e * scale)
        out = sum over the taken e of weight_e * down_e(act(gate_e x) * up_e(x))

    ``router_bias``: z has a learned bias added (``name.router.b`` in the file).  ``gate = (kind, alpha, limit)``: an
    expert's two input products meet as ``ops.glu`` of that kind says (``"clamped"``: ``g = min(gate, limit)``, ``u =
    clamp(up, -limit, limit)``, ``g * sigmoid(alpha g) * (u + 1)``) in place of ``act(gate) * up``.

    ``gated=False``: experts without a gate, ``down_e(act(up_e x))``.  ``groups = (count, keep)``: the experts form
    ``count`` equal groups of neighbours, a group's score is its largest s, and only experts of the ``keep`` best groups
    can be taken.  ``shared_ff`` > 0: one more expert of that size (``name.shared.up``, ``.down``; same form, no gate)
    runs for every token and is added, times ``sigmoid(W_sg x)`` (``name.shared.sg`` ``[1, hidden]``, one number a
    token, formed in 32-bit by the router's launch) if ``shared_gate``.

    The file holds ``name.router`` ``[experts, hidden]`` and per expert ``name.e<j>.gate``, ``.up`` ``[ff, hidden]``
    and ``.down`` ``[hidden, ff]``; on the device the experts' matrices are stacked (gate rows then up rows per
    expert, and the down matrices) and the router is 32-bit."""

    def __init__(self, name: str, hidden_size: int, ffn_size: int, experts: int, top: int, scale: float = 1.0,
                 score: str = "sigmoid", normalise: bool = True, act: str = "silu", router_bias: bool = False, gate=None,
                 gated: bool = True, groups=None, shared_ff: int = 0, shared_gate: bool = False):
        if gate is not None and gate[0] not in ops.GLU_CODES:
            raise ValueError(f"{name}: a gate of kind {gate[0]!r} is not built; built: {sorted(ops.GLU_CODES)}")
        if not (0 < top <= experts):
            raise ValueError(f"{name}: {top} of {experts} experts per token")
        if score not in ops.ROUTE_SCORE_CODES:
            raise ValueError(f"{name}: router scores of kind {score!r} are not built; built: {sorted(ops.ROUTE_SCORE_CODES)}")
        self.name, self.hidden_size, self.ffn_size = name, int(hidden_size), int(ffn_size)
        self.experts, self.top, self.scale = int(experts), int(top), float(scale)
        self.score, self.normalise, self.act = score, bool(normalise), act
        self.router_bias, self.gate = bool(router_bias), (None if gate is None else (gate[0], float(gate[1]), float(gate[2])))
        self.gated = bool(gated)
        if not self.gated and (gate is not None or act not in ops.ACT_CODES):
            raise ValueError(f"{name}: experts without a gate take an activation of {sorted(k for k in ops.ACT_CODES if k)}")
        self.groups = (1, 1) if groups is None else (int(groups[0]), int(groups[1]))
        count, keep = self.groups
        if count < 1 or experts % count or not (1 <= keep <= count) or keep * (experts // count) < top:
            raise ValueError(f"{name}: {experts} experts in {count} groups of which {keep} are kept do not give {top} a token")
        self.shared = None
        self.shared_gate = bool(shared_gate) and shared_ff > 0
        if shared_ff > 0:
            self.shared = DenseFeedForward(f"{name}.shared", hidden_size, int(shared_ff), False, act, "up", "down",
                                           bare_names=True)
        self.router = self.gate_up = self.down = self.bias = self.shared_gate_w = None

    def children(self) -> Sequence[Part]:
        return () if self.shared is None else (self.shared,)

    def tensor_specs(self) -> List[TensorSpec]:
        n, E, F, H = self.name, self.experts, self.ffn_size, self.hidden_size
        dn = tuple((f"{n}.e{e}.down", (H, F)) for e in range(E))
        bias = [TensorSpec(f"{n}.router.b", (E,), VECTOR, INIT_ZERO_NOISE)] if self.router_bias else []
        if self.shared_gate:
            bias.append(TensorSpec(f"{n}.shared.sg", (1, H), VECTOR, INIT_NORMAL))
        if self.gated:
            gu = tuple((f"{n}.e{e}.{m}", (F, H)) for e in range(E) for m in ("gate", "up"))
            first = TensorSpec(f"{n}.experts.gate_up", (E, 2 * F, H), MATRIX, INIT_NORMAL, pieces=gu,
                               assemble=_stack_experts(E, (F, F)), split=_unstack_experts((F, F)))
        else:
            up = tuple((f"{n}.e{e}.up", (F, H)) for e in range(E))
            first = TensorSpec(f"{n}.experts.up", (E, F, H), MATRIX, INIT_NORMAL, pieces=up,
                               assemble=_stack_experts(E, (F,)), split=_unstack_experts((F,)))
        return bias + [TensorSpec(f"{n}.router", (E, H), VECTOR, INIT_NORMAL), first,
                TensorSpec(f"{n}.experts.down", (E, H, F), MATRIX, INIT_NORMAL, pieces=dn, assemble=_stack_experts(E, (H,)),
                           split=_unstack_experts((H,)))]

    def load(self, tensors: Dict[str, torch.Tensor]) -> None:
        n = self.name
        self.router, self.down = tensors[f"{n}.router"], tensors[f"{n}.experts.down"]
        self.gate_up = tensors[f"{n}.experts.gate_up" if self.gated else f"{n}.experts.up"]
        self.bias = tensors[f"{n}.router.b"] if self.router_bias else None
        self.shared_gate_w = tensors[f"{n}.shared.sg"] if self.shared_gate else None

    def check_sizes(self) -> None:
        if self.top > 64 or self.experts > 2048 or self.groups[0] > 64:
            raise ValueError(f"{self.name}: the router takes at most 64 of at most 2048 experts in at most 64 groups")

    def forward(self, x: torch.Tensor, ctx: StepContext, add1=None, add2=None):
        routed = ops.moe_route(x, self.router, self.top, self.score, self.normalise, self.scale, bias=self.bias,
                               groups=self.groups[0], keep=self.groups[1], extra=self.shared_gate_w)
        ids, wts = routed[0], routed[1]
        extra = extra_gate = None
        if self.shared is not None:  # the expert of every token: added, times its gate, by the launch that sums the taken ones
            extra = self.shared.forward(x, ctx)
            extra_gate = routed[2] if self.shared_gate else torch.ones((x.shape[0], 1), dtype=torch.float32, device=x.device)
        out = ops.moe_experts(x, self.gate_up, self.down, ids, wts, self.act, gate=self.gate, gated=self.gated, extra=extra,
                              extra_gate=extra_gate)
        if add1 is None and add2 is None:
            return out
        return ops.epilogue_(out, None, None, as_tensor(add1), as_tensor(add2))


register_part("feed_forward", "dense", DenseFeedForward)
register_part("feed_forward", "gated", GatedFeedForward)
register_part("feed_forward", "polynorm", PolyNormFeedForward)
register_part("feed_forward", "xielu", XieluFeedForward)
register_part("feed_forward", "routed", RoutedFeedForward)
