"""A plain, slow implementation of the Nopuzen design in float64 on the CPU: one function per mechanism, written from
the equations in each docstring, sharing no code with the package.  A sequence is walked token by token; what a
sequence keeps between tokens is, per layer, a list with one entry per token so far (latent attention: the normed
latent and the rotated shared key part; attention: the normed, rotated keys and the values).

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


def softplus(v: torch.Tensor) -> torch.Tensor:
    """ln(1 + e^v)."""
    return torch.log1p(torch.exp(v))


def sigmoid(v):
    return 1.0 / (1.0 + torch.exp(-v))


def rotary_frequencies(rot: dict) -> torch.Tensor:
    """f_i = base^(-2i/dims) for i < dims/2.  With ``scaling`` (factor, original, fast, slow): with dim(t) = dims *
    ln(original / (2 pi t)) / (2 ln base), lo = max(floor(dim(fast)), 0), hi = min(ceil(dim(slow)), dims - 1) and
    ramp_i = clamp((i - lo) / max(hi - lo, 0.001), 0, 1), the frequency is f_i / factor * ramp_i + f_i * (1 - ramp_i)."""
    dims, base = int(rot["dims"]), float(rot["base"])
    f = [base ** (-2.0 * i / dims) for i in range(dims // 2)]
    sc = rot.get("scaling")
    if sc:
        factor, original = float(sc["factor"]), float(sc["original"])

        def where(t):
            return dims * math.log(original / (2 * math.pi * t)) / (2 * math.log(base))

        lo = max(math.floor(where(float(sc["fast"]))), 0)
        hi = min(math.ceil(where(float(sc["slow"]))), dims - 1)
        for i in range(dims // 2):
            ramp = min(max((i - lo) / max(hi - lo, 0.001), 0.0), 1.0)
            f[i] = f[i] / factor * ramp + f[i] * (1 - ramp)
    return torch.tensor(f, dtype=F)


def rotary_magnitude(rot: dict) -> float:
    """What cosines and sines are multiplied by: 0.1 ln(factor) + 1 with a scaling, else 1."""
    sc = rot.get("scaling")
    return 0.1 * math.log(float(sc["factor"])) + 1.0 if sc else 1.0


def rotate(v: torch.Tensor, pos: int, rot: dict, layout: str) -> torch.Tensor:
    """The first ``dims`` elements of the last dimension turned by the position, the rest as they are.  Pairs: ``half``
    (i, i + dims/2), ``interleaved`` (2i, 2i + 1); no ``rot``: nothing turns; the pair (u, w) becomes (u cos a - w sin a, w cos a + u sin a), a =
    pos * f_i, cos and sin times the magnitude."""
    if not rot:
        return v
    dims = int(rot["dims"])
    f = rotary_frequencies(rot)
    a = pos * f
    c, s = torch.cos(a) * rotary_magnitude(rot), torch.sin(a) * rotary_magnitude(rot)
    out = v.clone()
    half = dims // 2
    for i in range(half):
        iu, iw = (i, i + half) if layout == "half" else (2 * i, 2 * i + 1)
        u, w = v[..., iu], v[..., iw]
        out[..., iu] = u * c[i] - w * s[i]
        out[..., iw] = w * c[i] + u * s[i]
    return out


def latent_attention_token(w, p: str, m: dict, eps: float, h: torch.Tensor, kept: List, pos: int) -> torch.Tensor:
    """One token through the latent attention mixer ``p``.  c_q = unit_rms(W_dq h) * dq.norm; q = W_uq c_q, per head
    [dim plain | rot_dim rotated].  d = W_dkv h: c = unit_rms(d[:rank]) * dkv.norm, r = rotate(d[rank:]) (one for all
    heads); (c, r) joins ``kept``.  For every kept j <= pos and head g: key_plain = (W_uk c_j)[g], value = (W_uv c_j)[g],
    s = (q_plain . key_plain + rotate(q_rot) . r_j) * scale; softmax over j; the heads side by side, times
    sigmoid(W_g h) element by element, through W_o."""
    H, d, dr, dv, R = m["heads"], m["dim"], m["rot_dim"], m["vdim"], m["kv_rank"]
    rot = dict(m["rot"])
    cq = unit_rms(w[p + ".dq"] @ h, eps) * w[p + ".dq.norm"]
    q = (w[p + ".uq"] @ cq).view(H, d + dr)
    q_plain, q_rot = q[:, :d], rotate(q[:, d:], pos, rot, "half")
    down = w[p + ".dkv"] @ h
    c = unit_rms(down[:R], eps) * w[p + ".dkv.norm"]
    r = rotate(down[R:], pos, rot, "half")
    kept.append((c, r))
    cs = torch.stack([e[0] for e in kept])          # [n, R]
    rs = torch.stack([e[1] for e in kept])          # [n, dr]
    keys = (cs @ w[p + ".uk"].T).view(-1, H, d)     # [n, H, d]
    vals = (cs @ w[p + ".uv"].T).view(-1, H, dv)
    s = (torch.einsum("hd,nhd->hn", q_plain, keys) + q_rot @ rs.T) * float(m["scale"])
    a = torch.softmax(s, dim=-1)
    o = torch.einsum("hn,nhv->hv", a, vals).reshape(H * dv)
    return w[p + ".o"] @ (o * sigmoid(w[p + ".g"] @ h))


def attention_token(w, p: str, m: dict, eps: float, h: torch.Tensor, kept: List, pos: int) -> torch.Tensor:
    """One token through the attention mixer ``p``.  q = W_q h + b_q in H heads of ``dim``, k = W_k h + b_k in G heads,
    v = W_v h + b_v in G heads of ``vdim``; every query and key head divided by its root mean square and multiplied by
    the q / k norm weight, then rotated (interleaved pairs); (k, v) joins ``kept``.  For every kept j <= pos and head
    g (on key head g // (H/G)): s = q_g . k(j) * scale * temp[g]; s <- softcap * tanh(s / softcap); the key's weight is
    sigmoid(s + pb[g]), not normalised over j.  Head g's weighted sum of values, times sigmoid(W_g h)[g]; the heads side
    by side through W_o, plus b_o."""
    H, G, d, dv = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    rot = m.get("rot")
    q = (w[p + ".q"] @ h + w[p + ".q.b"]).view(H, d)
    k = (w[p + ".k"] @ h + w[p + ".k.b"]).view(G, d)
    v = (w[p + ".v"] @ h + w[p + ".v.b"]).view(G, dv)
    q = rotate(unit_rms(q, eps) * w[p + ".q.norm"], pos, rot, "interleaved")
    k = rotate(unit_rms(k, eps) * w[p + ".k.norm"], pos, rot, "interleaved")
    kept.append((k, v))
    per = H // G
    ks = torch.stack([e[0] for e in kept])  # [n, G, d]
    vs = torch.stack([e[1] for e in kept])
    cap = float(m.get("softcap") or 0.0)
    gate = sigmoid(w[p + ".g"] @ h)
    out = torch.zeros(H, dv, dtype=F)
    for g in range(H):
        s = ks[:, g // per] @ q[g] * float(m["scale"]) * w[p + ".temp"][g]
        if cap > 0:
            s = cap * torch.tanh(s / cap)
        a = sigmoid(s + w[p + ".pb"][g])
        out[g] = (a[:, None] * vs[:, g // per]).sum(0) * gate[g]
    return w[p + ".o"] @ out.reshape(H * dv) + w[p + ".o.b"]


def xielu(z: torch.Tensor, act: torch.Tensor) -> torch.Tensor:
    """With (p, q) = act: z > 0: softplus(p) z^2 + z / 2; z <= 0: (1/2 + softplus(q)) (e^z - 1 - z) + z / 2."""
    ap, an = softplus(act[0]), 0.5 + softplus(act[1])
    return torch.where(z > 0, ap * z * z + 0.5 * z, an * (torch.expm1(torch.clamp(z, max=0.0)) - z) + 0.5 * z)


def dense_ff(w, p: str, h: torch.Tensor) -> torch.Tensor:
    """W_down xielu(W_up h)."""
    return w[p + ".down"] @ xielu(w[p + ".up"] @ h, w[p + ".act"])


def relu2_ff(w, p: str, h: torch.Tensor) -> torch.Tensor:
    """W_down relu(W_up h)^2."""
    return w[p + ".down"] @ torch.clamp(w[p + ".up"] @ h, min=0.0) ** 2


def route(w, p: str, r: dict, h: torch.Tensor):
    """s = softmax(W_router h) over all experts.  The experts form ``groups.count`` equal groups of neighbours, a
    group's score is its largest s, and only experts of the ``groups.keep`` best groups can be taken; of those the
    ``top`` with the largest s are taken, with the weights s * scale.  Returns [(expert, weight)]."""
    E, top = int(r["experts"]), int(r["top"])
    s = torch.softmax(w[p + ".router"] @ h, dim=-1)
    allowed = list(range(E))
    groups = r.get("groups")
    if groups:
        n, keep = int(groups["count"]), int(groups["keep"])
        size = E // n
        best = sorted(range(n), key=lambda g: -float(s[g * size:(g + 1) * size].max()))[:keep]
        allowed = [e for e in range(E) if e // size in best]
    taken = sorted(allowed, key=lambda e: -float(s[e]))[:top]
    return [(e, float(s[e]) * float(r["scale"])) for e in taken]


def moe_ff(w, p: str, mlp: dict, h: torch.Tensor) -> torch.Tensor:
    """The weighted sum of the taken experts' relu2_ff, plus (if the layer has one) the shared expert's relu2_ff times
    sigmoid(W_sg h)."""
    out = torch.zeros_like(h)
    for e, weight in route(w, p, mlp["router"], h):
        out = out + weight * relu2_ff(w, f"{p}.e{e}", h)
    if mlp.get("shared") is not None:
        out = out + relu2_ff(w, p + ".shared", h) * sigmoid(w[p + ".shared.sg"] @ h)
    return out


def feed_forward(w, p: str, mlp: dict, h: torch.Tensor) -> torch.Tensor:
    return dense_ff(w, p, h) if mlp["kind"] == "dense" else moe_ff(w, p, mlp, h)


class Sequence:
    """What one sequence keeps: per layer the list of its tokens' cache entries, and its length."""

    def __init__(self, cfg: dict):
        self.kept = [[] for _ in cfg["layers"]]
        self.length = 0


def step_token(w: Dict[str, torch.Tensor], cfg: dict, seq: Sequence, token: int, streams: List = None) -> torch.Tensor:
    """One token through the model: x = embed[token]; per layer x <- x + LN_1(mixer(x)), x <- x + LN_2(ff(x)) (no second
    step without a feed-forward); logits = embed . LN_final(x).  ``streams`` collects x after every layer."""
    eps = float(cfg["norm"]["eps"])
    pos = seq.length
    x = w["embed"][token].clone()
    for i, layer in enumerate(cfg["layers"]):
        p = f"l{i}"
        fn = latent_attention_token if layer["type"] == "latent_attention" else attention_token
        y = fn(w, p + ".mix", layer["mixer"], eps, x, seq.kept[i], pos)
        x = x + layer_norm(y, w[p + ".norm1"], w[p + ".norm1.b"], eps)
        if layer.get("mlp") is not None:
            y = feed_forward(w, p + ".mlp", layer["mlp"], x)
            x = x + layer_norm(y, w[p + ".norm2"], w[p + ".norm2.b"], eps)
        if streams is not None:
            streams.append(x.clone())
    seq.length += 1
    return w["embed"] @ layer_norm(x, w["final.norm"], w["final.norm.b"], eps)


def run_tokens(w, cfg: dict, tokens: List[int], seq: Sequence = None) -> torch.Tensor:
    """Logits [len(tokens), vocab] of a sequence fed token by token (on top of ``seq`` if given)."""
    seq = seq or Sequence(cfg)
    return torch.stack([step_token(w, cfg, seq, int(t)) for t in tokens])


def greedy(w, cfg: dict, prompt: List[int], new_tokens: int) -> List[int]:
    seq = Sequence(cfg)
    logits = run_tokens(w, cfg, prompt, seq)
    out = []
    for _ in range(new_tokens):
        out.append(int(torch.argmax(logits[-1])))
        logits = run_tokens(w, cfg, out[-1:], seq)
    return out
