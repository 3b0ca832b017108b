"""The Kekapel design on the GPU against the plain implementation (``plain_kekapel``): every mechanism alone, then whole
models of several shapes through the step function, the cache, captured decode steps and ``generate``.

The tests make their own small configurations and weights.  Sizes are chosen so that nothing is equal that need not be
(key and value sizes of a head, heads and kv heads, windows and the cache's pages), and a far key, a window's edge or a
pass's stale cache shows in the result instead of drowning in averages.
"""
import json
import os

import pytest
import torch

import helpers
import plain_kekapel as P
from test_gpu_bimepel import _bf16, _close, _load_part, _rand, _run_in_cuts, assert_model_close, load, write_model

pytestmark = pytest.mark.gpu

DTYPES = [("float32", 3e-5), ("bfloat16", 4e-2)]
TORCH = {"float32": torch.float32, "bfloat16": torch.bfloat16}
REL_BF16_MODEL = 0.1


# ---- configurations ---------------------------------------------------------------------------------------------
def attn(heads=6, kv=2, dim=24, vdim=20, scale=0.3, softcap=6.0, mask=40):
    m = {"heads": heads, "kv_heads": kv, "dim": dim, "vdim": vdim, "scale": scale}
    if softcap:
        m["softcap"] = softcap
    if mask:
        m["mask"] = {"size": mask}
    return {"type": "attention", "mixer": m}


def dense(layer, ff=56):
    return dict(layer, mlp={"kind": "dense", "ff": ff})


def moe(layer, ff=24, experts=5, top=2, limit=0.8):
    return dict(layer, mlp={"kind": "moe", "expert": {"ff": ff, "limit": limit}, "router": {"experts": experts, "top": top}})


def bare(layer):
    return dict(layer, mlp=None)


def config(layers, loop=None, vocab=131, width=48, eps=1e-5, mult=0.6, scale=2.5, positions=512):
    c = {"architecture": "Kekapel", "vocab": vocab, "width": width, "max_positions": positions, "embedding": {"scale": scale},
         "layers": layers, "norm": {"eps": eps}, "residual_mult": mult}
    if loop is not None:
        c["loop"] = {"start": loop[0], "stop": loop[1], "times": loop[2]}
    return c


CONFIGS = {
    # every feed-forward and a layer without one, four shapes of attention (windows of less than a page, more than one,
    # none; with and without a cap), a loop of two layers in the middle that runs twice
    "mixed": config([dense(attn()), moe(attn(4, 1, 16, 32, 0.2, 3.0, 70), 16, 7, 3, 0.5), bare(attn(2, 2, 40, 8, 0.15, 0.0, 0)),
                     dense(attn(5, 5, 8, 8, 0.5, 10.0, 7), 40)], loop=(1, 3, 2)),
    # one head, one expert of one, one pass, a window of one token, factors of one: the values that make indices vanish
    "ones": config([moe(attn(1, 1, 16, 16, 0.25, 2.0, 1), 8, 1, 1, 1.0), dense(attn(1, 1, 16, 16, 0.25, 0.0, 3), 16)],
                   loop=(0, 1, 1), vocab=61, width=16, mult=1.0, scale=1.0, positions=400),
    # the whole model as one loop of three passes; windows of one page, of less and of a size that no page shares
    "loop": config([dense(attn(4, 2, 32, 32, 0.18, 20.0, 64)), moe(attn(4, 4, 16, 24, 0.25, 4.0, 17), 32, 4, 4, 2.0),
                    bare(attn(8, 2, 8, 16, 0.3, 5.0, 130))], loop=(0, 3, 3), vocab=97, width=64, mult=0.5, scale=3.5),
    # no loop at all
    "flat": config([moe(attn(3, 1, 20, 12, 0.2, 8.0, 33), 8, 3, 2, 0.3), dense(attn(2, 1, 12, 28, 0.3, 0.0, 65), 24)], vocab=77,
                   width=40, mult=0.9, scale=0.7),
}


def make_weights(cfg, seed, std=0.3):
    """Random weights by the design's tensor names, rounded to bfloat16 (so that both compute types hold the same
    numbers), as float64.  Lively enough that layers matter: gains around one, head mixes that are no unit matrix,
    routers that spread their choices."""
    from pytorch_transformers_amd.config import AutoConfig
    from pytorch_transformers_amd.config.registry import lookup

    c = AutoConfig.from_dict(cfg)
    specs = lookup(c.model_type)[1](c).tensor_specs()
    g = torch.Generator().manual_seed(seed)
    w = {}
    for s in specs:
        names = [(s.name, s.shape)] if not s.pieces else list(s.pieces)
        for n, shape in names:
            t = torch.randn(shape, generator=g)
            last = n.rsplit(".", 1)[-1]
            if last in ("norm1", "norm2", "norm1b", "norm2b", "norm"):
                t = 1.0 + 0.3 * t
            elif last == "b":
                t = 0.2 * t
            elif last == "talk":
                t = torch.eye(shape[0]) + 0.4 * t
            elif last == "act":
                t = torch.tensor([0.9, 0.5, 0.3, 0.1]) + 0.2 * t
            elif last == "router":
                t = t * 0.8
            elif n == "pos":
                t = t * 0.5
            elif n == "loop.step":
                t = t * 0.4
            elif n != "embed":
                t = t * std * (48.0 / shape[-1]) ** 0.5
            w[n] = _bf16(t)
    return w


def plain_all(cfg, w, reqs):
    model = P.PlainKekapel(cfg, w)
    return {rid: model.logits(toks).float() for rid, toks in reqs.items()}


def _part_weights(part, seed, std=0.3):
    g = torch.Generator().manual_seed(seed)
    w = {}
    for s in part.all_tensor_specs():
        for n, shape in ([(s.name, s.shape)] if not s.pieces else list(s.pieces)):
            t = torch.randn(shape, generator=g)
            if n.endswith(".talk"):
                t = torch.eye(shape[0]) + 0.4 * t
            elif n.endswith(".norm"):
                t = 1.0 + 0.3 * t
            else:
                t = t * (0.5 if len(shape) == 1 else std)
            w[n] = _bf16(t)
    return w


# ---- each mechanism alone ------------------------------------------------------------------------------------------------
@pytest.mark.parametrize("dtype,rel", DTYPES)
@pytest.mark.parametrize("width", [16, 48, 200, 1100])
def test_norms_around_the_stream(dtype, rel, width):
    """Every combination of the launch's terms: the stream alone, a sublayer's output normed, scaled and added, a second
    tensor and a vector added, the norm of the sum, and a gather of rows."""
    from pytorch_transformers_amd import ops

    dt, eps, mult, rows = TORCH[dtype], 1e-5, 0.6, 9
    x, y, add = (_rand(rows, width, seed=s, scale=2.0) for s in (1, 2, 3))
    y = _bf16(y)
    vec, w1, b1, w2, b2 = (_rand(width, seed=s) for s in (4, 5, 6, 7, 8))
    dev = lambda t: t.float().cuda()
    post, pre = (dev(w1), dev(b1)), (dev(w2), dev(b2))
    s_want = x.double() + mult * P.layer_norm(y, w1.double(), b1.double(), eps)
    # the first launch of a block: the stream as it is, normed
    h, wide = ops.layernorm_stream(dt, x=dev(x), pre=pre, eps=eps, want_wide=False)
    assert wide is None
    _close(h, P.layer_norm(x.double(), w2.double(), b2.double(), eps), rel, "norm of the stream")
    # between two sublayers
    h, wide = ops.layernorm_stream(dt, x=dev(x), y=y.to(dt).cuda(), post=post, mult=mult, pre=pre, eps=eps)
    _close(wide, s_want, 1e-6, "stream plus a normed sublayer")
    _close(h, P.layer_norm(s_want, w2.double(), b2.double(), eps), rel, "its norm")
    # at the start of a pass of a loop, with the last sublayer still to add; then without a norm; then on three rows
    full = s_want + add.double() + vec.double()
    h, wide = ops.layernorm_stream(dt, x=dev(x), y=y.to(dt).cuda(), post=post, mult=mult, add=dev(add), vec=dev(vec), pre=pre, eps=eps)
    _close(wide, full, 1e-6, "with a tensor and a vector added")
    _close(h, P.layer_norm(full, w2.double(), b2.double(), eps), rel, "its norm")
    h, wide = ops.layernorm_stream(dt, x=dev(x), vec=dev(vec), eps=eps)
    assert h is None
    _close(wide, x.double() + vec.double(), 1e-6, "a vector alone")
    take = torch.tensor([7, 0, 3], dtype=torch.int32).cuda()
    h, _ = ops.layernorm_stream(dt, x=dev(x), y=y.to(dt).cuda(), post=post, mult=mult, pre=pre, eps=eps, rows=take, want_wide=False)
    _close(h, P.layer_norm(s_want, w2.double(), b2.double(), eps)[[7, 0, 3]], rel, "three rows of it")


@pytest.mark.parametrize("dtype,rel", DTYPES)
def test_scaled_embedding_with_learned_positions(dtype, rel):
    from pytorch_transformers_amd import ops

    dt = TORCH[dtype]
    table, pos = _bf16(_rand(50, 24, seed=1)), _bf16(_rand(30, 24, seed=2))
    ids = torch.tensor([3, 49, 0, 3], dtype=torch.int32)
    at = torch.tensor([0, 29, 7, 8], dtype=torch.int32)
    got = ops.embed_pos(table.to(dt).cuda(), ids.cuda(), 2.5, pos.to(dt).cuda(), at.cuda())
    assert got.dtype == torch.float32
    _close(got, table[ids.long()] * 2.5 + pos[at.long()], 1e-6, "embedding")


@pytest.mark.parametrize("dtype,rel", DTYPES)
@pytest.mark.parametrize("ff,hidden", [(56, 40), (1, 8), (300, 24), (2048, 64), (8200, 16), (12, 8)])
def test_feed_forward_with_polynorm(dtype, rel, ff, hidden):
    from pytorch_transformers_amd.parts import PolyNormFeedForward

    dt = TORCH[dtype]
    part = PolyNormFeedForward("f", hidden, ff, 1e-5)
    w = _part_weights(part, seed=3)
    w["f.act"] = _bf16(torch.tensor([0.9, -0.5, 0.3, 0.2]))
    _load_part(part, w, dt)
    for rows in (1, 9, 300):
        x = _bf16(_rand(rows, hidden, seed=rows))
        want = torch.stack([P.dense_ff(w, "f", x[i], 1e-5) for i in range(rows)])
        _close(part.forward(x.to(dt).cuda(), None), want, rel, f"PolyNorm feed-forward {ff} rows {rows}")


def test_polynorm_alone_in_32_bit():
    from pytorch_transformers_amd import ops

    z = _rand(5, 77, seed=1, scale=1.5)
    coef = torch.tensor([0.7, -1.1, 0.4, 0.25])
    got = ops.polynorm(z.cuda(), coef.cuda(), 1e-5)
    _close(got, P.polynorm(z.double(), coef.double(), 1e-5), 1e-5, "PolyNorm")


@pytest.mark.parametrize("dtype,rel", DTYPES)
@pytest.mark.parametrize("experts,top,limit,ff,hidden", [(5, 2, 0.8, 24, 40), (1, 1, 1.0, 8, 40), (7, 7, 0.2, 16, 40),
                                                         (70, 3, 5.0, 40, 40),
                                                         # sizes that the matrix-core launches take (steps of many tokens)
                                                         (5, 2, 0.7, 64, 64), (9, 3, 1.5, 192, 128)])
def test_routed_experts_with_a_router_bias_and_a_clamped_gate(dtype, rel, experts, top, limit, ff, hidden):
    from pytorch_transformers_amd import ops
    from pytorch_transformers_amd.parts import RoutedFeedForward

    dt = TORCH[dtype]
    part = RoutedFeedForward("f", hidden, ff, experts, top, 1.0, score="softmax", normalise=True, router_bias=True,
                             gate=("clamped", 1.702, limit))
    w = _part_weights(part, seed=13, std=0.4)
    w["f.router.b"] = _bf16(_rand(experts, seed=2) * 2.0)  # a bias that decides choices
    _load_part(part, w, dt)
    mlp = {"router": {"experts": experts, "top": top}, "expert": {"ff": ff, "limit": limit}}
    for rows in (1, 7, 17, 150):
        x = _bf16(_rand(rows, hidden, seed=14 + rows))
        want = torch.stack([P.moe_ff(w, "f", mlp, x[i]) for i in range(rows)])
        _close(part.forward(x.to(dt).cuda(), None), want, rel, f"routed feed-forward {experts} experts top {top} rows {rows}")
        ids, wts = ops.moe_route(x.to(dt).cuda(), part.router, top, "softmax", True, 1.0, bias=part.bias)
        for i in range(rows):
            want_ids, want_w = P.route(w, "f", x[i], top)
            assert ids[i].tolist() == want_ids
            _close(wts[i], want_w, 1e-5, "the taken experts' weights")
    if experts > top:  # without the bias other experts are taken: the bias is what the test sees
        x = _bf16(_rand(40, hidden, seed=3))
        ids_b, _ = ops.moe_route(x.to(dt).cuda(), part.router, top, "softmax", True, 1.0, bias=part.bias)
        ids_0, _ = ops.moe_route(x.to(dt).cuda(), part.router, top, "softmax", True, 1.0)
        assert not torch.equal(ids_b, ids_0)


def _attention_mixer(hidden, m, eps=1e-5, talk=True):
    from pytorch_transformers_amd.parts import GatedAttentionMixer, NoPositions

    return GatedAttentionMixer("a", hidden, m["heads"], m["kv_heads"], m["dim"], m["vdim"], m["scale"], eps, NoPositions(),
                               window=(m.get("mask") or {}).get("size", 0), v_norm=False, gate=False,
                               softcap=float(m.get("softcap") or 0.0), talk=talk)


def _plain_attention(w, m, x, eps=1e-5):
    kept = []
    return torch.stack([P.attention_token(w, "a", m, eps, x[pos], kept, pos) for pos in range(x.shape[0])])


def _window_group(mixer):
    from pytorch_transformers_amd.engine.spec import CACHE_FULL, CACHE_WINDOW, CacheGroupSpec

    return CacheGroupSpec("kv", CACHE_WINDOW if mixer.window else CACHE_FULL, 1, mixer.kv_heads, mixer.frame,
                          window=mixer.window or None)


@pytest.mark.parametrize("dtype,rel", DTYPES)
@pytest.mark.parametrize("shape", [attn(), attn(4, 1, 16, 32, 0.2, 3.0, 64), attn(2, 2, 40, 8, 0.15, 0.0, 0),
                                   attn(5, 5, 8, 8, 0.5, 10.0, 7), attn(3, 1, 72, 130, 0.1, 30.0, 100),
                                   attn(20, 4, 16, 16, 0.3, 4.0, 65), attn(1, 1, 24, 24, 0.3, 5.0, 1)])
def test_attention_mixer_alone(dtype, rel, shape):
    """Whole, token by token, in portions down to two tokens and across page borders, four sequences a step, and once
    more on slots and pages that were given back."""
    from pytorch_transformers_amd.engine.spec import LayerCall

    m, hidden, dt = shape["mixer"], 32, TORCH[dtype]
    mixer = _attention_mixer(hidden, m)
    w = _part_weights(mixer, seed=5)
    _load_part(mixer, w, dt)
    call = LayerCall(0, "kv", 0)
    cuts = [[150], [64, 1, 1, 62, 2, 20], [1] * 20 + [130], [63, 2, 85]]
    xs = [_bf16(_rand(150, hidden, seed=40 + i)) for i in range(4)]
    outs = _run_in_cuts(lambda x, ctx: mixer.forward(x, ctx, call), [_window_group(mixer)], dt, xs, cuts, free_and_again=True)
    for i in range(4):
        _close(outs[i], _plain_attention(w, m, xs[i]), rel, f"attention {m} sequence {i}")


@pytest.mark.parametrize("dtype,rel", DTYPES)
def test_the_heads_mix_is_applied_row_by_row(dtype, rel):
    """A mix that hands head 1 the scores of head 0 and nothing else: head 1 then weighs its own values as head 0 does.
    (The transposed mix would leave head 1 with no scores at all, that is with even weights.)"""
    from pytorch_transformers_amd.engine.spec import LayerCall

    m, hidden, dt = attn(2, 2, 16, 16, 0.6, 0.0, 0)["mixer"], 32, TORCH[dtype]
    mixer = _attention_mixer(hidden, m)
    w = _part_weights(mixer, seed=9, std=0.5)
    w["a.talk"] = torch.tensor([[1.0, 0.0], [1.0, 0.0]], dtype=torch.float64)
    w["a.v"][16:] = w["a.v"][:16]  # both heads hold the same values: equal weights give equal outputs
    _load_part(mixer, w, dt)
    x = _bf16(_rand(40, hidden, seed=1))
    want = _plain_attention(w, m, x)
    got = _run_in_cuts(lambda t, ctx: mixer.forward(t, ctx, LayerCall(0, "kv", 0)), [_window_group(mixer)], dt, [x], [[30] + [1] * 10])[0]
    _close(got, want, rel, "a mix that copies a head's scores")
    heads = (got.to(torch.float64) @ torch.linalg.pinv(w["a.o"]).T).view(40, 2, 16)  # undo W_o: the heads side by side
    assert float((heads[:, 0] - heads[:, 1]).abs().max()) < (0.05 if dtype == "bfloat16" else 1e-4) * float(heads.abs().max())


@pytest.mark.parametrize("dtype,rel", DTYPES)
@pytest.mark.parametrize("window,query,key", [(64, 200, 136), (64, 200, 137), (64, 200, 199), (96, 300, 204), (96, 300, 205),
                                              (0, 500, 0), (0, 500, 63), (0, 500, 64), (50, 149, 99), (50, 149, 100),
                                              (50, 127, 78), (50, 128, 79), (50, 128, 78), (130, 191, 62), (130, 192, 63),
                                              (130, 192, 62), (2, 9, 8), (2, 9, 7), (70, 69, 0), (70, 70, 0), (70, 70, 1)])
def test_attention_sees_one_loud_key_inside_its_window_only(dtype, rel, window, query, key):
    """One key far back, at the window's first place, or just outside it, also where the edge lies on a page border
    and among a sequence's first tokens, with a score that stands out: queries and keys read one half of the input and
    values the other, and the query's token repeats the loud key's first half.  Fed whole and with the query decoded
    alone.  The plain side checks that the loud key shows exactly where it is visible."""
    from pytorch_transformers_amd.engine.spec import LayerCall

    m, hidden, dt = attn(2, 1, 24, 20, 2.0, 25.0, window)["mixer"], 32, TORCH[dtype]
    mixer = _attention_mixer(hidden, m)
    w = _part_weights(mixer, seed=6)
    w["a.q"][:, 16:] = 0
    w["a.k"][:, 16:] = 0
    w["a.v"][:, :16] = 0
    w["a.q"][24:] = w["a.q"][:24]
    w["a.k"] = w["a.q"][:24].clone()  # the key of a token points where its heads' queries point
    w["a.q.norm"] = w["a.k.norm"] = torch.ones(24, dtype=torch.float64)
    w["a.talk"] = torch.tensor([[1.0, 0.25], [-0.25, 1.0]], dtype=torch.float64)
    _load_part(mixer, w, dt)
    n = query + 3
    x = _bf16(_rand(n, hidden, seed=7))
    loud = _bf16(_rand(16, seed=8) * 3.0)
    x[key, :16] = loud
    x[query, :16] = loud
    want = _plain_attention(w, m, x)
    quiet = x.clone()
    quiet[key, :16] = x[key - 1 if key else 1, :16]
    visible = window == 0 or query - key < window
    moved = float((_plain_attention(w, m, quiet)[query] - want[query]).abs().max()) > 0.3 * float(want[query].abs().max())
    assert moved == (visible and key != query), "the test's loud key does not show where it should"
    call = LayerCall(0, "kv", 0)
    for cuts in ([[n]], [[query, 1, 2]], [[key + 1, query - key - 1, 1, 1, 1]] if query - key > 1 else [[key, 1, 1, 1, 1]]):
        got = _run_in_cuts(lambda t, ctx: mixer.forward(t, ctx, call), [_window_group(mixer)], dt, [x], cuts)[0]
        _close(got, want, rel, f"window {window}, query {query}, loud key {key}, cuts {cuts}")


def test_a_cap_flattens_a_loud_score():
    """With a small cap two loud keys of different loudness weigh alike; without it the louder one takes all."""
    from pytorch_transformers_amd.engine.spec import LayerCall

    hidden = 32
    outs = {}
    for cap in (1.0, 0.0):
        m = attn(1, 1, 16, 16, 4.0, cap, 0)["mixer"]
        mixer = _attention_mixer(hidden, m)
        w = _part_weights(mixer, seed=3)
        w["a.talk"] = torch.ones(1, 1, dtype=torch.float64)
        _load_part(mixer, w, torch.float32)
        x = _bf16(_rand(20, hidden, seed=2))
        want = _plain_attention(w, m, x)
        got = _run_in_cuts(lambda t, ctx: mixer.forward(t, ctx, LayerCall(0, "kv", 0)), [_window_group(mixer)], torch.float32,
                           [x], [[20]])[0]
        _close(got, want, 3e-5, f"cap {cap}")
        outs[cap] = got
    assert float((outs[1.0] - outs[0.0]).abs().max()) > 0.05 * float(outs[0.0].abs().max())


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


def test_the_stream_after_every_layer_run(tmp_path):
    """The 32-bit stream after every entry of the run order (passes of the loop each on their own), last token of a
    prompt, against the plain model's."""
    cfg = CONFIGS["mixed"]
    w = make_weights(cfg, seed=17)
    model = load(write_model(tmp_path / "m", cfg, w), "float32")
    toks = helpers.make_requests(cfg["vocab"], [75], seed=2)["r0"]
    seen = {}
    model.layer_hook = lambda i, x: seen.__setitem__(i, x[-1].double().cpu())
    cache = model.new_cache(256)
    model.step(cache, [cache.alloc()], [toks], "last")
    plain = P.PlainKekapel(cfg, w)
    plain.logits(toks)
    assert len(seen) == len(plain.streams) == 6
    for i, want in enumerate(plain.streams):
        _close(seen[i], want, 2e-5, f"stream after layer run {i}")


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
    """300 tokens decoded one by one after a short prompt (pages handed back as the windows move on, over hundreds of
    steps), with a token near the start whose embedding is loud: the layer without a window keeps seeing it."""
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


def test_a_sequence_longer_than_the_position_table_is_refused(tmp_path):
    cfg = config([bare(attn(2, 1, 8, 8, 0.3, 0.0, 4))], vocab=20, width=16, positions=12)
    model = load(write_model(tmp_path / "m", cfg, make_weights(cfg, seed=1)), "float32")
    cache = model.new_cache(128)
    slot = cache.alloc()
    model.step(cache, [slot], [[1] * 12], "last")
    with pytest.raises(ValueError, match="positions"):
        model.step(cache, [slot], [[1, 2]], "last")


def test_greedy_generation_follows_the_plain_model(tmp_path):
    cfg = CONFIGS["mixed"]
    w = make_weights(cfg, seed=14)
    model = load(write_model(tmp_path / "m", cfg, w), "float32")
    reqs = helpers.make_requests(cfg["vocab"], [5, 17, 2], seed=6)
    out = model.generate(list(reqs.values()), max_new_tokens=12, do_sample=False, eos_token_id=None)
    plain = P.PlainKekapel(cfg, w)
    for seq, toks in zip(out, reqs.values()):
        assert list(seq) == list(toks) + plain.greedy(list(toks), 12)


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
    assert {"embed", "pos", "head", "loop.step", "final.norm", "final.norm.b", "l0.norm1b.b", "l0.mix.q.norm", "l0.mix.talk",
            "l0.mlp.act", "l0.mlp.up", "l1.mlp.router", "l1.mlp.router.b", "l1.mlp.e4.up", "l1.mlp.e6.down", "l3.norm2b"} <= names
    assert not any(n.startswith(("l2.mlp", "l2.norm2")) or ".experts." in n or n.endswith((".weight", ".bias")) for n in names)
    for dtype in ("bfloat16", "float32"):
        model = AutoModelForCausalLM.from_pretrained(folder, dtype=dtype)
        cache = model.new_cache(256)
        logits = model.step(cache, [cache.alloc()], [[1, 2, 3]], "all")
        assert logits.shape == (3, cfg.vocab) and torch.isfinite(logits).all()


def test_the_command_line_generates_from_a_model_folder(tmp_path, capsys):
    """``run_generation`` on a folder of this design: greedy tokens as the plain model chooses them."""
    from pytorch_transformers_amd import run_generation

    cfg = CONFIGS["flat"]
    w = make_weights(cfg, seed=15)
    folder = write_model(tmp_path / "m", cfg, w)
    rc = run_generation.main(["--model_name_or_path", folder, "--model_type", "kekapel", "--prompt_ids", "3,1,4,1,5",
                              "--length", "6", "--greedy", "--dtype", "float32"])
    assert rc == 0
    printed = [ln for ln in capsys.readouterr().out.splitlines() if ln and ln[0].isdigit()]
    assert [int(t) for t in printed[-1].split(",")] == [3, 1, 4, 1, 5] + P.PlainKekapel(cfg, w).greedy([3, 1, 4, 1, 5], 6)


# ---- configurations drawn at random --------------------------------------------------------------------------------------
def draw_config(seed):
    import random

    r = random.Random(seed)
    layers = []
    for _ in range(r.randint(1, 4)):
        kv = r.choice([1, 2, 3])
        a = attn(kv * r.choice([1, 2, 4]), kv, r.choice([8, 12, 16, 40]), r.choice([8, 20, 32, 48]), r.choice([0.1, 0.3]),
                 r.choice([0.0, 2.0, 15.0]), r.choice([0, 1, 5, 63, 64, 65, 100]))
        kind = r.choice(["dense", "moe", "none"])
        if kind == "dense":
            a = dense(a, r.choice([8, 30, 64]))
        elif kind == "moe":
            e = r.choice([1, 3, 6])
            a = moe(a, r.choice([8, 20]), e, r.randint(1, e), r.choice([0.3, 1.0, 4.0]))
        else:
            a = bare(a)
        layers.append(a)
    loop = None
    if r.random() < 0.7:
        a = r.randint(0, len(layers) - 1)
        loop = (a, r.randint(a, len(layers)), r.randint(1, 3))
    return config(layers, loop, vocab=r.choice([50, 101]), width=r.choice([16, 24, 72]), eps=r.choice([1e-5, 1e-6, 1e-3]),
                  mult=r.choice([0.4, 1.0, 1.3]), scale=r.choice([1.0, 3.0]), positions=256)


@pytest.mark.parametrize("seed", range(10))
def test_configurations_drawn_at_random(tmp_path, seed):
    from pytorch_transformers_amd.engine.replay import Replayer

    cfg = draw_config(seed)
    w = make_weights(cfg, seed=100 + seed)
    reqs = helpers.make_requests(cfg["vocab"], [70, 3, 140], seed=seed)
    want = plain_all(cfg, w, reqs)
    folder = write_model(tmp_path / "m", cfg, w)
    for dtype, rel in (("float32", helpers.REL_F32), ("bfloat16", REL_BF16_MODEL)):
        rp = Replayer(load(folder, dtype), 1024, max_slots=4)
        for records in (helpers.schedule_batches(reqs, 3, decode=(20, 1, 70)), helpers.schedule_staggered(reqs, chunks=(7, None, 2))):
            got = helpers.run_schedule(rp, records)
            for rid in reqs:
                assert_model_close(got[rid], want[rid], rel, f"seed {seed} {dtype} {rid}: {json.dumps(cfg)[:300]}")
