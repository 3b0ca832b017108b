"""The Nopuzen design on the GPU against the plain implementation (``plain_nopuzen``): every mechanism alone, then whole
models of several shapes through the step function, the cache, captured decode steps and ``generate``.

The tests make their own small configurations and weights.  Sizes are chosen so that nothing is equal that need not be
(plain, rotated and value sizes of a head, heads and kv heads, the two latents, groups of experts and the cache's pages),
and a far key, a page's edge, a head's own number or a group that is not kept shows in the result instead of drowning in
averages.
"""
import json
import os

import pytest
import torch

import helpers
import plain_nopuzen as P
from test_gpu_bimepel import _bf16, _close, _load_part, _rand, _run_in_cuts, assert_model_close, load, write_model

pytestmark = pytest.mark.gpu

DTYPES = [("float32", 3e-5), ("bfloat16", 4e-2)]
TORCH = {"float32": torch.float32, "bfloat16": torch.bfloat16}
REL_BF16_MODEL = 0.1


# ---- configurations ---------------------------------------------------------------------------------------------
def rot(dims, base=10000.0, scaling=True):
    r = {"base": base, "dims": dims}
    if scaling:
        r["scaling"] = {"factor": 4.0, "original": 64, "fast": 8.0, "slow": 1.0}
    return r


def latent(heads=3, dim=24, rot_dim=8, vdim=20, kv_rank=40, q_rank=28, scale=0.25, base=10000.0, scaling=True):
    return {"type": "latent_attention", "mixer": {"heads": heads, "dim": dim, "rot_dim": rot_dim, "vdim": vdim,
                                                  "kv_rank": kv_rank, "q_rank": q_rank, "scale": scale,
                                                  "rot": rot(rot_dim, base, scaling)}}


def attn(heads=6, kv=2, dim=24, vdim=20, scale=0.3, softcap=6.0, dims=16, base=5000.0, scaling=False):
    m = {"heads": heads, "kv_heads": kv, "dim": dim, "vdim": vdim, "scale": scale}
    if softcap:
        m["softcap"] = softcap
    if dims:
        m["rot"] = rot(dims, base, scaling)
    return {"type": "attention", "mixer": m}


def dense(layer, ff=56):
    return dict(layer, mlp={"kind": "dense", "ff": ff})


def moe(layer, ff=24, experts=6, top=2, scale=1.5, groups=(3, 2), shared=40):
    mlp = {"kind": "moe", "expert": {"ff": ff}, "router": {"experts": experts, "top": top, "scale": scale}}
    if groups:
        mlp["router"]["groups"] = {"count": groups[0], "keep": groups[1]}
    if shared:
        mlp["shared"] = {"ff": shared}
    return dict(layer, mlp=mlp)


def bare(layer):
    return dict(layer, mlp=None)


def config(layers, vocab=131, width=48, eps=1e-5):
    return {"architecture": "Nopuzen", "vocab": vocab, "width": width, "layers": layers, "norm": {"eps": eps}}


CONFIGS = {
    # both mixers with every feed-forward and a layer without one; two latent shapes (two page pools), two attention shapes
    "mixed": config([dense(latent()), moe(attn()), moe(latent(2, 16, 16, 32, 24, 56, 0.2, 300.0, False), 16, 8, 2, 0.7, (4, 1), 0),
                     bare(attn(4, 4, 40, 8, 0.15, 0.0, 0)), dense(attn(5, 1, 16, 48, 0.2, 30.0, 8, 100.0, True), 40),
                     moe(latent(), 8, 5, 5, 1.0, None, 16)]),
    # one head, one expert of one, one group, factors of one, latents as wide as the model: the values that make indices vanish
    "ones": config([moe(latent(1, 16, 2, 16, 16, 16, 1.0), 8, 1, 1, 1.0, (1, 1), 8), dense(attn(1, 1, 16, 16, 1.0, 0.0, 2), 16)],
                   vocab=61, width=16),
    # attention only, heads of sizes the matrix-core kernels are built for, and experts that run on them
    "wide": config([moe(attn(8, 2, 32, 32, 0.18, 20.0, 32), 64, 8, 2, 2.0, (2, 1), 64), dense(attn(4, 4, 16, 16, 0.25, 4.0, 4), 96),
                    bare(attn(2, 1, 64, 48, 0.3, 5.0, 16))], vocab=97, width=64),
    # latent attention only
    "latent": config([moe(latent(4, 16, 16, 16, 32, 32, 0.3), 8, 4, 2, 0.3, (2, 2), 24), dense(latent(2, 40, 4, 12, 64, 8, 0.2), 24)],
                     vocab=77, width=40),
}


def make_weights(cfg, seed, std=0.3):
    """Random weights by the design's tensor names, rounded to bfloat16 (so that both compute types hold the same
    numbers), as float64.  Lively enough that layers matter: gains around one, numbers per head that differ, routers
    that spread their choices."""
    from pytorch_transformers_amd.config import AutoConfig
    from pytorch_transformers_amd.config.registry import lookup

    c = AutoConfig.from_dict(cfg)
    specs = lookup(c.model_type)[1](c).tensor_specs()
    g = torch.Generator().manual_seed(seed)
    w = {}
    for s in specs:
        names = [(s.name, s.shape)] if not s.pieces else list(s.pieces)
        for n, shape in names:
            if n == "head.weight":
                continue
            t = torch.randn(shape, generator=g)
            last = n.rsplit(".", 1)[-1]
            if last in ("norm1", "norm2"):
                t = 0.5 + 0.15 * t  # (every sublayer adds a normed vector to the stream, which the next reads as it is)
            elif last in ("norm", "temp"):
                t = 1.0 + 0.3 * t
            elif last in ("b", "pb", "act"):
                t = 0.3 * t
            elif last == "router":
                t = t * 0.4
            elif n != "embed":
                t = t * std * (48.0 / shape[-1]) ** 0.5
            w[n] = _bf16(t)
    return w


def plain_all(cfg, w, reqs):
    return {rid: P.run_tokens(w, cfg, toks).float() for rid, toks in reqs.items()}


def _part_weights(part, seed, std=0.3):
    g = torch.Generator().manual_seed(seed)
    w = {}
    for s in part.all_tensor_specs():
        for n, shape in ([(s.name, s.shape)] if not s.pieces else list(s.pieces)):
            t = torch.randn(shape, generator=g)
            if n.endswith((".norm", ".temp")):
                t = 1.0 + 0.3 * t
            else:
                t = t * (0.5 if len(shape) == 1 else std)
            w[n] = _bf16(t)
    return w


# ---- each mechanism alone ------------------------------------------------------------------------------------------------
@pytest.mark.parametrize("dtype,rel", DTYPES)
@pytest.mark.parametrize("width", [16, 48, 200, 1100])
def test_a_norm_on_a_sublayers_output_joins_the_stream(dtype, rel, width):
    """x + LN(y) * w + b in 32-bit, and its copy in the compute type for the next product."""
    from pytorch_transformers_amd.parts import LayerNorm

    dt, eps, rows = TORCH[dtype], 1e-5, 9
    x, y = _rand(rows, width, seed=1, scale=2.0), _bf16(_rand(rows, width, seed=2, scale=3.0) + 0.7)
    norm = LayerNorm("n", width, eps, weight_name="n", bias_name="n.b")
    w = {"n": _bf16(1.0 + 0.3 * _rand(width, seed=3)), "n.b": _bf16(0.3 * _rand(width, seed=4))}
    _load_part(norm, w, dt)
    narrow, wide = norm.apply(y.to(dt).cuda(), dt, residual=x.float().cuda(), want_wide=True)
    want = x.float().double() + P.layer_norm(y, w["n"], w["n.b"], eps)
    _close(wide, want, 3e-6, "the stream")
    assert narrow.dtype == dt
    _close(narrow, want, 1e-6 if dtype == "float32" else 5e-3, "the stream's copy")


@pytest.mark.parametrize("dtype,rel", DTYPES)
@pytest.mark.parametrize("ff,hidden,rows", [(56, 40, 7), (1, 8, 3), (300, 24, 40), (2048, 64, 300), (12, 8, 1)])
def test_feed_forward_with_xielu(dtype, rel, ff, hidden, rows):
    from pytorch_transformers_amd.parts import XieluFeedForward

    dt = TORCH[dtype]
    part = XieluFeedForward("f", hidden, ff)
    w = _part_weights(part, seed=ff)
    w["f.act"] = _bf16(torch.tensor([0.4, -1.2]))
    _load_part(part, w, dt)
    x = _bf16(_rand(rows, hidden, seed=1, scale=1.5))
    got = part.forward(x.to(dt).cuda(), None)
    want = torch.stack([P.dense_ff(w, "f", x[i]) for i in range(rows)])
    _close(got, want, rel, f"xielu feed-forward {ff}x{hidden}")


def test_xielu_alone_in_32_bit():
    """Both branches, the kink at zero, and coefficients on both sides of softplus's bend."""
    from pytorch_transformers_amd import ops

    z = torch.cat([torch.linspace(-30, 30, 601), torch.tensor([0.0, -0.0, 1e-6, -1e-6, 25.0, -80.0])]).view(1, -1)
    for p, q in ((0.4, -1.2), (-3.0, 2.5), (30.0, -30.0), (0.0, 0.0)):
        act = torch.tensor([p, q])
        got = ops.xielu(z.float().cuda().contiguous(), act.float().cuda())
        _close(got, P.xielu(z.float().double(), act.float().double()), 3e-6, f"xielu({p}, {q})")


@pytest.mark.parametrize("dtype,rel", DTYPES)
@pytest.mark.parametrize("experts,top,groups,shared,ff,hidden", [
    (6, 2, (3, 2), 40, 24, 40), (1, 1, (1, 1), 8, 8, 40), (8, 2, (4, 1), 0, 16, 40), (8, 8, None, 16, 16, 24),
    (12, 2, (6, 1), 64, 64, 64), (70, 5, (7, 3), 128, 64, 128), (18, 4, (3, 1), 20, 80, 64), (9, 3, (3, 3), 0, 128, 64)])
def test_routed_experts_with_groups_and_a_shared_expert(dtype, rel, experts, top, groups, shared, ff, hidden):
    """1 to 700 rows (a token's experts row by row, and tiles of an expert's tokens on the matrix cores where the sizes
    allow them): the experts the plain router takes, among the kept groups alone, and the weighted sum with the shared
    expert behind its gate."""
    from pytorch_transformers_amd import ops
    from pytorch_transformers_amd.parts import RoutedFeedForward

    dt = TORCH[dtype]
    mlp = moe({}, ff, experts, top, 1.5, groups, shared)["mlp"]
    part = RoutedFeedForward("f", hidden, ff, experts, top, 1.5, score="softmax", normalise=False, act="relu2", gated=False,
                             groups=groups, shared_ff=shared, shared_gate=bool(shared))
    w = _part_weights(part, seed=experts * 7 + top)
    w["f.router"] = _bf16(w["f.router"] * 4.0)  # scores far enough apart that no choice is a close call
    _load_part(part, w, dt)
    for rows in (1, 5, 16, 17, 700):
        x = _bf16(_rand(rows, hidden, seed=rows, scale=1.2))
        got = part.forward(x.to(dt).cuda(), None)
        want = torch.stack([P.moe_ff(w, "f", mlp, x[i]) for i in range(rows)])
        _close(got, want, rel, f"{experts} experts, top {top}, groups {groups}, {rows} rows")
        routed = ops.moe_route(x.to(dt).cuda(), part.router, top, "softmax", False, 1.5, groups=part.groups[0], keep=part.groups[1])
        for i in range(min(rows, 40)):
            taken = P.route(w, "f", mlp["router"], x[i])
            assert sorted(routed[0][i].tolist()) == sorted(e for e, _ in taken), f"row {i}: experts taken"
            assert abs(float(routed[1][i].sum()) - sum(wt for _, wt in taken)) < 1e-4


def test_only_experts_of_the_kept_groups_are_taken():
    """The best expert of a group that is not kept loses to a worse one of the kept group."""
    from pytorch_transformers_amd import ops

    hidden = 8
    router = torch.zeros(6, hidden)
    for e, z in enumerate([1.0, 3.0, 2.5, 0.2, 0.1, 2.9]):  # groups {0,1}, {2,3}, {4,5}; group maxima 3.0, 2.5, 2.9
        router[e, 0] = z
    x = torch.zeros(2, hidden)
    x[:, 0] = 1.0
    ids, wts = ops.moe_route(x.cuda(), router.cuda(), 3, "softmax", False, 1.0, groups=3, keep=2)
    assert sorted(ids[0].tolist()) == [0, 1, 5], "groups 0 and 2 are kept; expert 2 of group 1 must not be taken"
    s = torch.softmax(router[:, 0].double(), 0)
    assert abs(float(wts[0].sum()) - float(s[0] + s[1] + s[5])) < 1e-6
    ids, _ = ops.moe_route(x.cuda(), router.cuda(), 3, "softmax", False, 1.0)
    assert sorted(ids[0].tolist()) == [1, 2, 5]


# ---- the two mixers alone -------------------------------------------------------------------------------------------------
def _latent_mixer(hidden, m, eps=1e-5):
    from pytorch_transformers_amd.engine.nopuzen import _positions
    from pytorch_transformers_amd.parts import LatentAttentionMixer

    return LatentAttentionMixer("a", hidden, m["heads"], m["dim"], m["rot_dim"], m["vdim"], m["kv_rank"], m["scale"], eps,
                                _positions(m["rot"], m["rot_dim"], "half"), q_rank=m["q_rank"], gate=True)


def _attention_mixer(hidden, m, eps=1e-5):
    from pytorch_transformers_amd.engine.nopuzen import _positions
    from pytorch_transformers_amd.parts import GatedAttentionMixer

    return GatedAttentionMixer("a", hidden, m["heads"], m["kv_heads"], m["dim"], m["vdim"], m["scale"], eps,
                               _positions(m.get("rot"), m["dim"], "interleaved"), v_norm=False, gate=True,
                               softcap=float(m.get("softcap") or 0.0), bias=True, head_scale=True, weights="sigmoid",
                               gate_per_head=True)


def _group(mixer):
    from pytorch_transformers_amd.engine.spec import CACHE_FULL, CacheGroupSpec

    if hasattr(mixer, "cache_row"):
        return CacheGroupSpec("kv", CACHE_FULL, 1, 1, mixer.cache_row, values=False)
    return CacheGroupSpec("kv", CACHE_FULL, 1, mixer.kv_heads, mixer.frame)


def _plain_mixer(kind, w, m, x, eps=1e-5):
    kept = []
    fn = P.latent_attention_token if kind == "latent_attention" else P.attention_token
    return torch.stack([fn(w, "a", m, eps, x[pos], kept, pos) for pos in range(x.shape[0])])


def _make_mixer(shape, hidden):
    return (_latent_mixer if shape["type"] == "latent_attention" else _attention_mixer)(hidden, shape["mixer"])


SHAPES = [latent(), latent(2, 16, 16, 32, 24, 56, 0.2, 300.0, False), latent(1, 16, 2, 16, 16, 16, 0.5), latent(5, 8, 4, 72, 130, 9, 0.3),
          latent(16, 32, 32, 16, 64, 32, 0.15), attn(), attn(4, 1, 16, 32, 0.2, 3.0, 8, 100.0, True), attn(2, 2, 40, 8, 0.15, 0.0, 0),
          attn(5, 5, 8, 8, 0.5, 10.0, 8), attn(3, 1, 72, 130, 0.1, 30.0, 72), attn(20, 4, 16, 16, 0.3, 4.0, 2),
          attn(8, 2, 64, 64, 0.2, 15.0, 32), attn(1, 1, 24, 24, 0.3, 5.0, 24)]


@pytest.mark.parametrize("dtype,rel", DTYPES)
@pytest.mark.parametrize("shape", SHAPES, ids=lambda s: s["type"][:3] + "-".join(str(v) for v in s["mixer"].values() if isinstance(v, int)))
def test_mixer_alone(dtype, rel, shape):
    """Whole, token by token, in portions down to two tokens and across page borders, four sequences a step, and once
    more on slots and pages that were given back."""
    from pytorch_transformers_amd.engine.spec import LayerCall

    m, hidden, dt = shape["mixer"], 32, TORCH[dtype]
    mixer = _make_mixer(shape, hidden)
    w = _part_weights(mixer, seed=5)
    _load_part(mixer, w, dt)
    call = LayerCall(0, "kv", 0)
    cuts = [[150], [64, 1, 1, 62, 2, 20], [1] * 20 + [130], [63, 2, 85]]
    xs = [_bf16(_rand(150, hidden, seed=40 + i)) for i in range(4)]
    outs = _run_in_cuts(lambda x, ctx: mixer.forward(x, ctx, call), [_group(mixer)], dt, xs, cuts, free_and_again=True)
    for i in range(4):
        _close(outs[i], _plain_mixer(shape["type"], w, m, xs[i]), rel, f"{shape['type']} {m} sequence {i}")


@pytest.mark.parametrize("dtype,rel", DTYPES)
def test_a_heads_own_numbers_are_that_heads(dtype, rel):
    """Two heads with the same queries, keys and values: what differs between their outputs is their own score factor,
    score bias and gate; swapping the two heads' numbers swaps their outputs."""
    from pytorch_transformers_amd.engine.spec import LayerCall

    m, hidden, dt = attn(2, 1, 16, 16, 0.8, 6.0, 8)["mixer"], 32, TORCH[dtype]
    outs = []
    for swap in (False, True):
        mixer = _attention_mixer(hidden, m)
        w = _part_weights(mixer, seed=9, std=0.5)
        w["a.q"][16:] = w["a.q"][:16]
        w["a.q.b"][16:] = w["a.q.b"][:16]
        w["a.temp"] = _bf16(torch.tensor([0.5, 1.5]))
        w["a.pb"] = _bf16(torch.tensor([-2.0, 0.5]))
        w["a.g"] = _bf16(torch.stack([w["a.g"][0], -w["a.g"][0]]))
        if swap:
            for n in ("a.temp", "a.pb", "a.g"):
                w[n] = w[n].flip(0)
        _load_part(mixer, w, dt)
        x = _bf16(_rand(40, hidden, seed=1))
        got = _run_in_cuts(lambda t, ctx: mixer.forward(t, ctx, LayerCall(0, "kv", 0)), [_group(mixer)], dt, [x], [[30] + [1] * 10])[0]
        _close(got, _plain_mixer("attention", w, m, x), rel, "two heads with numbers of their own")
        bias = w["a.o.b"]
        outs.append(((got.double() - bias) @ torch.linalg.pinv(w["a.o"]).T).view(40, 2, 16))  # undo W_o: the heads side by side
    tol = (0.05 if dtype == "bfloat16" else 1e-4) * float(outs[0].abs().max())
    assert float((outs[0][:, 0] - outs[1][:, 1]).abs().max()) < tol and float((outs[0][:, 1] - outs[1][:, 0]).abs().max()) < tol
    assert float((outs[0][:, 0] - outs[0][:, 1]).abs().max()) > 10 * tol


def _loud_weights(kind, mixer, m, hidden):
    """Weights under which a token whose first half of the input repeats an earlier token's gives that token's key a
    score that stands out: queries and keys read the first half of the input, values the second."""
    w = _part_weights(mixer, seed=6)
    half = hidden // 2
    if kind == "attention":
        d = m["dim"]
        w["a.q"][:, half:] = 0
        w["a.k"][:, half:] = 0
        w["a.v"][:, :half] = 0
        w["a.q"][d:] = w["a.q"][:d]
        w["a.k"] = w["a.q"][:d].clone()  # the key of a token points where its heads' queries point
        for n in ("a.q.b", "a.k.b"):
            w[n] = torch.zeros_like(w[n])
        w["a.q.norm"] = w["a.k.norm"] = torch.ones(d, dtype=torch.float64)
        w["a.temp"] = torch.ones(m["heads"], dtype=torch.float64)
        w["a.pb"] = torch.full((m["heads"],), -14.0, dtype=torch.float64)  # quiet keys weigh next to nothing
    else:
        R, d, dr, H = m["kv_rank"], m["dim"], m["rot_dim"], m["heads"]
        # the first half of the latent reads the input's first half and makes the keys, the second half makes the values
        w["a.dkv"][:R // 2, half:] = 0
        w["a.dkv"][R // 2:R, :half] = 0
        w["a.dkv"][R:] = 0  # no rotated part of the keys
        w["a.dq"] = w["a.dkv"][:R].clone()
        w["a.dq"][R // 2:] = 0
        w["a.dq.norm"] = w["a.dkv.norm"] = torch.ones(R, dtype=torch.float64)
        w["a.uk"][:, R // 2:] = 0
        w["a.uv"][:, :R // 2] = 0
        uq = torch.zeros(H, d + dr, R, dtype=torch.float64)
        uq[:, :d] = w["a.uk"].view(H, d, R)  # a head's plain query is that head's key of the same token
        w["a.uq"] = uq.view(H * (d + dr), R)
    return w


@pytest.mark.parametrize("dtype,rel", DTYPES)
@pytest.mark.parametrize("kind", ["attention", "latent_attention"])
@pytest.mark.parametrize("query,key", [(500, 0), (500, 1), (500, 63), (500, 64), (500, 137), (200, 199), (200, 201), (191, 127),
                                       (192, 128), (64, 63), (64, 65), (63, 0), (9, 8), (2, 0), (1, 0), (300, 302)])
def test_one_loud_key_is_seen_from_wherever_it_lies_behind(dtype, rel, kind, query, key):
    """One key far back among hundreds, at a page's first and last place, among a sequence's first tokens, right behind
    the query, and ahead of it (where it must not be seen): fed whole and with the query decoded alone.  The plain side
    checks that the loud key shows exactly where it is visible."""
    from pytorch_transformers_amd.engine.spec import LayerCall

    hidden, dt = 32, TORCH[dtype]
    shape = attn(2, 1, 24, 20, 0.7, 25.0, 0) if kind == "attention" else latent(2, 24, 8, 20, 32, 32, 0.6)
    m = shape["mixer"]
    mixer = _make_mixer(shape, hidden)
    w = _loud_weights(kind, mixer, m, hidden)
    _load_part(mixer, w, dt)
    n = max(query, key) + 2
    x = _bf16(_rand(n, hidden, seed=7))
    loud = _bf16(_rand(16, seed=8) * 3.0)
    x[key, :16] = loud
    x[query, :16] = loud
    want = _plain_mixer(kind, w, m, x)
    quiet = x.clone()
    quiet[key, :16] = x[next(i for i in range(n) if i not in (key, query)), :16]
    moved = float((_plain_mixer(kind, w, m, quiet)[query] - want[query]).abs().max()) > 0.2 * float(want[query].abs().max())
    assert moved == (key < query), "the test's loud key does not show where it should"
    call = LayerCall(0, "kv", 0)
    first = min(key, query)
    for cuts in ([[n]], [[query, 1, n - query - 1]], [[first + 1, query - first - 1, 1, n - query - 1]] if query - first > 1 else [[1] * n]):
        got = _run_in_cuts(lambda t, ctx: mixer.forward(t, ctx, call), [_group(mixer)], dt, [x], [[c for c in cuts[0] if c]])[0]
        _close(got, want, rel, f"{kind}: query {query}, loud key {key}, cuts {cuts}")


def test_sigmoid_weights_are_not_normalised():
    """Twice the same keys and values give twice the output (a softmax would give the same)."""
    from pytorch_transformers_amd.engine.spec import LayerCall

    m, hidden = attn(2, 1, 16, 16, 0.5, 0.0, 0)["mixer"], 32
    mixer = _attention_mixer(hidden, m)
    w = _part_weights(mixer, seed=3)
    w["a.o.b"] = torch.zeros_like(w["a.o.b"])
    w["a.g"] = torch.zeros_like(w["a.g"])  # gates of one half: the output is half the heads' sums through W_o
    _load_part(mixer, w, torch.float32)
    x = _bf16(_rand(1, hidden, seed=2)).repeat(20, 1)
    got = _run_in_cuts(lambda t, ctx: mixer.forward(t, ctx, LayerCall(0, "kv", 0)), [_group(mixer)], torch.float32, [x], [[20]])[0]
    _close(got, _plain_mixer("attention", w, m, x), 3e-5, "equal tokens")
    _close(got[9], got[4].double() * 2.0, 1e-4, "ten equal keys against five")


# ---- whole models ------------------------------------------------------------------------------------------------------
@pytest.mark.parametrize("dtype,rel", [("float32", helpers.REL_F32), ("bfloat16", REL_BF16_MODEL)])
@pytest.mark.parametrize("name", sorted(CONFIGS))
def test_schedules_give_the_plain_logits(tmp_path, name, dtype, rel):
    """Whole prompts, prompt then token by token, unequal batches decoded together, requests that join and leave with
    prompts in portions down to one token: all the plain logits, with slots and pages freed and used again."""
    from pytorch_transformers_amd.engine.replay import Replayer

    cfg = CONFIGS[name]
    w = make_weights(cfg, seed=11)
    model = load(write_model(tmp_path / name, cfg, w), dtype)
    reqs = helpers.make_requests(cfg["vocab"], [9, 70, 131, 1, 64, 65, 2, 300], seed=3)
    want = plain_all(cfg, w, reqs)
    rp = Replayer(model, 1024, max_slots=8)
    for label, records in (("whole", helpers.schedule_whole(reqs)), ("tail", helpers.schedule_tail(reqs, 40)),
                           ("batches", helpers.schedule_batches(reqs, 3)),
                           ("staggered", helpers.schedule_staggered(reqs, chunks=(None, 2, 19, 1))),
                           ("batches again", helpers.schedule_batches(reqs, 4, decode=(1, 30, 2, 5)))):
        got = helpers.run_schedule(rp, records)
        for rid in reqs:
            assert_model_close(got[rid], want[rid], rel, f"{name} {dtype} {label} {rid}")
        assert not rp.cache.live_slots()


def test_the_stream_after_every_layer(tmp_path):
    """The 32-bit stream after every layer, last token of a prompt, against the plain model's."""
    cfg = CONFIGS["mixed"]
    w = make_weights(cfg, seed=17)
    model = load(write_model(tmp_path / "m", cfg, w), "float32")
    toks = helpers.make_requests(cfg["vocab"], [75], seed=2)["r0"]
    seen = {}
    model.layer_hook = lambda i, x: seen.__setitem__(i, x[-1].double().cpu())
    cache = model.new_cache(256)
    model.step(cache, [cache.alloc()], [toks], "last")
    seq, streams = P.Sequence(cfg), []
    for t in toks:
        streams = []
        P.step_token(w, cfg, seq, t, streams)
    assert len(seen) == len(streams) == len(cfg["layers"])
    for i, want in enumerate(streams):
        _close(seen[i], want, 2e-5, f"stream after layer {i}")


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_captured_decode_steps_equal_direct_ones(tmp_path, dtype):
    """Decode steps replayed from a captured graph give the bits of the same steps launched one by one, with batches
    that are padded to the captured size."""
    from pytorch_transformers_amd.engine.replay import Replayer

    cfg = CONFIGS["mixed"]
    folder = write_model(tmp_path / "m", cfg, make_weights(cfg, seed=12))
    reqs = helpers.make_requests(cfg["vocab"], [9, 30, 70, 3, 41, 12, 25, 8, 19, 33, 50], seed=4)
    records = helpers.schedule_batches(reqs, 3, decode=(5, 2, 8)) + \
        [dict(r, step=r["step"] + 1000) for r in helpers.schedule_batches(reqs, 11, decode=(2, 9, 4))]
    outs = {}
    for graphs in (False, True):
        model = load(folder, dtype)
        assert model.use_graphs
        model.use_graphs = graphs
        rp = Replayer(model, 2048, max_slots=16)
        outs[graphs] = [rp.run(rec) for rec in records]
        torch.cuda.synchronize()
    for rec, a, b in zip(records, outs[False], outs[True]):
        assert (a is None) == (b is None)
        if a is not None:
            assert torch.equal(a, b), f"step {rec['step']}: a captured step differs from the same step launched directly"


@pytest.mark.parametrize("dtype,rel", [("float32", helpers.REL_F32), ("bfloat16", REL_BF16_MODEL)])
def test_long_decoding_and_a_loud_far_token(tmp_path, dtype, rel):
    """300 tokens decoded one by one after a short prompt, with a token near the start whose embedding is loud: every
    layer keeps seeing it over hundreds of steps and several pages."""
    from pytorch_transformers_amd.engine.replay import Replayer

    cfg = CONFIGS["mixed"]
    w = make_weights(cfg, seed=13)
    w["embed"][7] = _bf16(w["embed"][7] * 6.0)
    model = load(write_model(tmp_path / "m", cfg, w), dtype)
    toks = [t if t != 7 else 8 for t in helpers.make_requests(cfg["vocab"], [330], seed=5)["r0"]]
    toks[2] = 7
    reqs = {"long": toks}
    want = plain_all(cfg, w, reqs)
    got = helpers.run_schedule(Replayer(model, 1024, max_slots=2), helpers.schedule_tail(reqs, 300))
    assert_model_close(got["long"], want["long"], rel, f"long decoding {dtype}")


def test_greedy_generation_follows_the_plain_model(tmp_path):
    cfg = CONFIGS["mixed"]
    w = make_weights(cfg, seed=14)
    model = load(write_model(tmp_path / "m", cfg, w), "float32")
    reqs = helpers.make_requests(cfg["vocab"], [5, 17, 2], seed=6)
    out = model.generate(list(reqs.values()), max_new_tokens=12, do_sample=False, eos_token_id=None)
    for seq, toks in zip(out, reqs.values()):
        assert list(seq) == list(toks) + P.greedy(w, cfg, list(toks), 12)


def test_random_weights_from_a_configuration_run(tmp_path):
    """The framework's own random-weights mode writes the design's tensor names, and what it writes loads and steps."""
    from safetensors import safe_open

    from pytorch_transformers_amd import AutoModelForCausalLM
    from pytorch_transformers_amd.config import AutoConfig
    from pytorch_transformers_amd.weights import write_random_model

    cfg = AutoConfig.from_dict(CONFIGS["mixed"])
    folder = write_random_model(str(tmp_path / "r"), cfg, seed=1, std=0.1)
    with safe_open(os.path.join(folder, "model.safetensors"), framework="pt") as f:
        names = set(f.keys())
    assert {"embed", "final.norm", "final.norm.b", "l0.norm1.b", "l0.mix.dq", "l0.mix.dq.norm", "l0.mix.uq", "l0.mix.dkv",
            "l0.mix.dkv.norm", "l0.mix.uk", "l0.mix.uv", "l0.mix.g", "l0.mix.o", "l0.mlp.act", "l0.mlp.up", "l1.mix.q.b",
            "l1.mix.k.norm", "l1.mix.temp", "l1.mix.pb", "l1.mix.o.b", "l1.mlp.router", "l1.mlp.e5.up", "l1.mlp.e0.down",
            "l1.mlp.shared.up", "l1.mlp.shared.down", "l1.mlp.shared.sg", "l4.norm2"} <= names
    assert not any(n.startswith(("l3.mlp", "l3.norm2", "l2.mlp.shared")) or ".experts." in n or n.endswith((".weight", ".bias", ".gate"))
                   for n in names)
    for dtype in ("bfloat16", "float32"):
        model = AutoModelForCausalLM.from_pretrained(folder, dtype=dtype)
        cache = model.new_cache(256)
        logits = model.step(cache, [cache.alloc()], [[1, 2, 3]], "all")
        assert logits.shape == (3, cfg.vocab) and torch.isfinite(logits).all()


def test_the_command_line_generates_from_a_model_folder(tmp_path, capsys):
    """``run_generation`` on a folder of this design: greedy tokens as the plain model chooses them."""
    from pytorch_transformers_amd import run_generation

    cfg = CONFIGS["latent"]
    w = make_weights(cfg, seed=15)
    folder = write_model(tmp_path / "m", cfg, w)
    rc = run_generation.main(["--model_name_or_path", folder, "--model_type", "nopuzen", "--prompt_ids", "3,1,4,1,5",
                              "--length", "6", "--greedy", "--dtype", "float32"])
    assert rc == 0
    printed = [ln for ln in capsys.readouterr().out.splitlines() if ln and ln[0].isdigit()]
    assert [int(t) for t in printed[-1].split(",")] == [3, 1, 4, 1, 5] + P.greedy(w, cfg, [3, 1, 4, 1, 5], 6)


# ---- configurations drawn at random --------------------------------------------------------------------------------------
def draw_config(seed):
    import random

    r = random.Random(seed)
    layers = []
    for _ in range(r.randint(1, 4)):
        if r.random() < 0.5:
            dr = r.choice([2, 4, 8, 16])
            a = latent(r.choice([1, 2, 3, 8]), r.choice([8, 12, 16, 40]), dr, r.choice([8, 20, 32, 48]), r.choice([8, 24, 64]),
                       r.choice([8, 12, 48]), r.choice([0.1, 0.3]), r.choice([100.0, 10000.0]), r.random() < 0.5)
        else:
            kv, d = r.choice([1, 2, 3]), r.choice([8, 12, 16, 40])
            a = attn(kv * r.choice([1, 2, 4]), kv, d, r.choice([8, 20, 32, 48]), r.choice([0.1, 0.3]), r.choice([0.0, 2.0, 15.0]),
                     r.choice([0, 2, d // 2 // 2 * 2, d]), r.choice([100.0, 10000.0]), r.random() < 0.3)
        kind = r.choice(["dense", "moe", "none"])
        if kind == "dense":
            a = dense(a, r.choice([8, 30, 64]))
        elif kind == "moe":
            count = r.choice([1, 2, 3])
            size = r.choice([1, 2, 4])
            keep = r.randint(1, count)
            a = moe(a, r.choice([8, 20, 64]), count * size, r.randint(1, keep * size), r.choice([0.3, 1.0, 2.5]),
                    r.choice([None, (count, keep)]) if keep == count else (count, keep), r.choice([0, 8, 33]))
        else:
            a = bare(a)
        layers.append(a)
    return config(layers, vocab=r.choice([50, 101]), width=r.choice([16, 24, 64, 72]), eps=r.choice([1e-5, 1e-6, 1e-3]))


@pytest.mark.parametrize("seed", range(10))
def test_configurations_drawn_at_random(tmp_path, seed):
    from pytorch_transformers_amd.engine.replay import Replayer

    cfg = draw_config(seed)
    w = make_weights(cfg, seed=seed)
    reqs = helpers.make_requests(cfg["vocab"], [70, 3, 130], seed=seed)
    want = plain_all(cfg, w, reqs)
    folder = write_model(tmp_path / "m", cfg, w)
    for dtype, rel in (("float32", helpers.REL_F32), ("bfloat16", REL_BF16_MODEL)):
        rp = Replayer(load(folder, dtype), 512, max_slots=4)
        for label, records in (("whole", helpers.schedule_whole(reqs)), ("batches", helpers.schedule_batches(reqs, 3, decode=(4, 1, 7)))):
            got = helpers.run_schedule(rp, records)
            for rid in reqs:
                assert_model_close(got[rid], want[rid], rel, f"{json.dumps(cfg)} {dtype} {label} {rid}")


def draw_larger_config(seed):
    """Sizes that the matrix-core kernels and the products for batches of rows take: heads of 32 to 128 elements, latents of
    64 to 256, experts of 64 and 128 rows on widths that are multiples of 64."""
    import random

    r = random.Random(1000 + seed)
    layers = []
    for i in range(r.randint(2, 3)):
        if (i + seed) % 2 == 0:
            dr = r.choice([16, 32, 64])
            a = latent(r.choice([4, 6, 12]), r.choice([32, 64, 96, 128]), dr, r.choice([32, 64, 128]), r.choice([64, 96, 256]),
                       r.choice([64, 160]), r.choice([0.08, 0.12]), r.choice([10000.0, 500000.0]), r.random() < 0.7)
        else:
            kv, d = r.choice([1, 2, 4]), r.choice([32, 48, 64, 128])
            a = attn(kv * r.choice([1, 2, 4]), kv, d, r.choice([32, 64, 80]), r.choice([0.1, 0.15]), r.choice([0.0, 12.0, 30.0]),
                     r.choice([d // 2, d]), r.choice([10000.0, 1000000.0]), r.random() < 0.3)
        kind = r.choice(["dense", "moe"])
        if kind == "dense":
            a = dense(a, r.choice([192, 448]))
        else:
            count, size = r.choice([2, 4]), r.choice([2, 6])
            keep = r.randint(1, count)
            a = moe(a, r.choice([64, 128]), count * size, r.randint(1, min(6, keep * size)), r.choice([1.0, 2.5]), (count, keep),
                    r.choice([0, 64, 192]))
        layers.append(a)
    return config(layers, vocab=r.choice([300, 513]), width=r.choice([128, 192, 320]), eps=r.choice([1e-5, 1e-6]))


@pytest.mark.parametrize("seed", range(6))
def test_larger_configurations_drawn_at_random(tmp_path, seed):
    from pytorch_transformers_amd.engine.replay import Replayer

    cfg = draw_larger_config(seed)
    w = make_weights(cfg, seed=seed)
    reqs = helpers.make_requests(cfg["vocab"], [150, 9, 40, 70], seed=seed)
    want = plain_all(cfg, w, reqs)
    folder = write_model(tmp_path / "m", cfg, w)
    for dtype, rel in (("float32", helpers.REL_F32), ("bfloat16", REL_BF16_MODEL)):
        rp = Replayer(load(folder, dtype), 1024, max_slots=4)
        for label, records in (("whole", helpers.schedule_whole(reqs)), ("tail", helpers.schedule_tail(reqs, 20)),
                               ("batches", helpers.schedule_batches(reqs, 4, decode=(4, 1, 7)))):
            got = helpers.run_schedule(rp, records)
            for rid in reqs:
                assert_model_close(got[rid], want[rid], rel, f"{json.dumps(cfg)} {dtype} {label} {rid}")
