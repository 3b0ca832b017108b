"""A plain, slow implementation of the Kekapel design in float64 on the CPU: one function per mechanism, written from
the equations in each docstring, sharing no code with the package.  A sequence is walked token by token; what a
sequence keeps between tokens is, per layer run, the list of the keys and values of its tokens so far.

``weights``: name -> float64 tensor, under the names of the weight file.  ``cfg``: the dict of ``config.json``.
"""
from __future__ import annotations

import math
from typing import Dict, List

import torch

F = torch.float64


def layer_norm(v: torch.Tensor, w: torch.Tensor, b: torch.Tensor, eps: float) -> torch.Tensor:
    """(v - mean) / sqrt(var + eps) * w + b over the last dimension; var is the mean squared deviation."""
    mu = v.mean(-1, keepdim=True)
    var = ((v - mu) ** 2).mean(-1, keepdim=True)
    return (v - mu) / torch.sqrt(var + eps) * w + b


def unit_rms(v: torch.Tensor, eps: float) -> torch.Tensor:
    """v / sqrt(mean(v^2) + eps) over the last dimension."""
    return v / torch.sqrt((v * v).mean(-1, keepdim=True) + eps)


def embed_token(w: Dict[str, torch.Tensor], cfg: dict, token: int, pos: int) -> torch.Tensor:
    """embed[token] * scale + pos[position]."""
    return w["embed"][token] * float(cfg["embedding"]["scale"]) + w["pos"][pos]


def visible(i: int, j: int, window: int) -> bool:
    """Whether position i sees position j: j <= i, and with a window i - j < window."""
    return j <= i and (window <= 0 or i - j < window)


def capped(s: torch.Tensor, cap: float) -> torch.Tensor:
    """cap * tanh(s / cap); no cap: s."""
    return cap * torch.tanh(s / cap) if cap > 0 else s


def attention_token(w, p: str, m: dict, eps: float, h: torch.Tensor, kept: List, pos: int) -> torch.Tensor:
    """One token through the mixer ``p``.  q = W_q h in H heads of ``dim``, k = W_k h in G heads, v = W_v h in G heads
    of ``vdim``; every query and key head divided by its root mean square and multiplied by the mixer's q / k norm
    weight; (k, v) joins ``kept``.  For every kept position j that ``pos`` sees and every head g:
    s_g(j) = capped(q_g . k_{g // (H/G)}(j) * scale); then t_h(j) = sum_g talk[h, g] s_g(j); weights = softmax of t_h
    over the seen j; head h's output is the weighted sum of v_{h // (H/G)}(j).  Output: W_o on the heads side by side."""
    H, G, d, dv = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    q = (w[p + ".q"] @ h).view(H, d)
    k = (w[p + ".k"] @ h).view(G, d)
    v = (w[p + ".v"] @ h).view(G, dv)
    q = unit_rms(q, eps) * w[p + ".q.norm"]
    k = unit_rms(k, eps) * w[p + ".k.norm"]
    kept.append((k, v))
    window = int((m.get("mask") or {}).get("size", 0))
    seen = [j for j in range(pos + 1) if visible(pos, j, window)]
    per = H // G
    s = torch.zeros(H, len(seen), dtype=F)
    for a, j in enumerate(seen):
        kj = kept[j][0]
        for g in range(H):
            s[g, a] = torch.dot(q[g], kj[g // per]) * float(m["scale"])
    s = capped(s, float(m.get("softcap") or 0.0))
    t = w[p + ".talk"] @ s
    a = torch.softmax(t, dim=-1)
    out = torch.zeros(H, dv, dtype=F)
    for hh in range(H):
        for n, j in enumerate(seen):
            out[hh] += a[hh, n] * kept[j][1][hh // per]
    return w[p + ".o"] @ out.reshape(-1)


def polynorm(z: torch.Tensor, coef: torch.Tensor, eps: float) -> torch.Tensor:
    """a N(z) + b N(z^2) + c N(z^3) + e with (a, b, c, e) = coef, powers element by element, N = unit_rms."""
    return coef[0] * unit_rms(z, eps) + coef[1] * unit_rms(z ** 2, eps) + coef[2] * unit_rms(z ** 3, eps) + coef[3]


def dense_ff(w, p: str, h: torch.Tensor, eps: float) -> torch.Tensor:
    """W_down polynorm(W_up h)."""
    return w[p + ".down"] @ polynorm(w[p + ".up"] @ h, w[p + ".act"], eps)


def expert(w, p: str, h: torch.Tensor, limit: float) -> torch.Tensor:
    """g = min(W_gate h, limit); u = clamp(W_up h, -limit, limit); W_down (g * sigmoid(1.702 g) * (u + 1))."""
    g = torch.clamp(w[p + ".gate"] @ h, max=limit)
    u = torch.clamp(w[p + ".up"] @ h, -limit, limit)
    return w[p + ".down"] @ (g * torch.sigmoid(1.702 * g) * (u + 1.0))


def route(w, p: str, h: torch.Tensor, top: int):
    """z = W_router h + bias; the ``top`` largest z (lower index first among equals); weights: softmax over those z."""
    z = w[p + ".router"] @ h + w[p + ".router.b"]
    order = sorted(range(z.shape[0]), key=lambda e: (-float(z[e]), e))[:top]
    wt = torch.softmax(torch.stack([z[e] for e in order]), dim=0)
    return order, wt


def moe_ff(w, p: str, mlp: dict, h: torch.Tensor) -> torch.Tensor:
    ids, wt = route(w, p, h, int(mlp["router"]["top"]))
    out = torch.zeros_like(h)
    for e, a in zip(ids, wt):
        out = out + a * expert(w, f"{p}.e{e}", h, float(mlp["expert"]["limit"]))
    return out


class PlainKekapel:
    def __init__(self, cfg: dict, weights: Dict[str, torch.Tensor]):
        self.cfg, self.w = cfg, weights
        self.eps = float(cfg["norm"]["eps"])
        self.m = float(cfg["residual_mult"])
        lp = cfg.get("loop") or {"start": 0, "stop": 0, "times": 1}
        self.loop = (int(lp["start"]), int(lp["stop"]), int(lp["times"]))
        self.streams: List[torch.Tensor] = []  # filled by ``token``: the stream after every layer run of the last token

    def runs(self):
        """(layer, pass whose first layer this is or None) for every layer run, in order."""
        a, b, t = self.loop
        n = len(self.cfg["layers"])
        out = [(i, None) for i in range(a)]
        for ps in range(t):
            out += [(i, ps if i == a else None) for i in range(a, b)]
        return out + [(i, None) for i in range(b, n)]

    def new_state(self):
        return [[] for _ in self.runs()]

    def layer(self, i: int, x: torch.Tensor, kept: List, pos: int) -> torch.Tensor:
        """x <- x + m * LN_1b(mixer(LN_1(x))); x <- x + m * LN_2b(ff(LN_2(x))) (the second only with a feed-forward)."""
        w, p, lay, eps = self.w, f"l{i}", self.cfg["layers"][i], self.eps
        ln = lambda v, n: layer_norm(v, w[f"{p}.{n}"], w[f"{p}.{n}.b"], eps)
        x = x + self.m * ln(attention_token(w, p + ".mix", lay["mixer"], eps, ln(x, "norm1"), kept, pos), "norm1b")
        mlp = lay.get("mlp")
        if mlp is not None:
            h = ln(x, "norm2")
            y = dense_ff(w, p + ".mlp", h, eps) if mlp["kind"] == "dense" else moe_ff(w, p + ".mlp", mlp, h)
            x = x + self.m * ln(y, "norm2b")
        return x

    def token(self, state, token: int, pos: int) -> torch.Tensor:
        """One token through the model; returns its logits.  In front of pass t of the loop: the embedding's output is
        added if t > 0, then row t of ``loop.step``."""
        x = e0 = embed_token(self.w, self.cfg, token, pos)
        self.streams = []
        for r, (i, ps) in enumerate(self.runs()):
            if ps is not None:
                if ps > 0:
                    x = x + e0
                x = x + self.w["loop.step"][ps]
            x = self.layer(i, x, state[r], pos)
            self.streams.append(x)
        return self.w["head"] @ layer_norm(x, self.w["final.norm"], self.w["final.norm.b"], self.eps)

    def logits(self, tokens: List[int]) -> torch.Tensor:
        state = self.new_state()
        return torch.stack([self.token(state, t, p) for p, t in enumerate(tokens)])

    def greedy(self, prompt: List[int], n: int) -> List[int]:
        state = self.new_state()
        for p, t in enumerate(prompt):
            last = self.token(state, t, p)
        out = []
        for _ in range(n):
            out.append(int(torch.argmax(last)))
            last = self.token(state, out[-1], len(prompt) + len(out) - 1)
        return out
