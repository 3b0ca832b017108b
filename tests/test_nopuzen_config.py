"""The Nopuzen design's configuration, tensor names and cache groups (no GPU)."""
import pytest

from pytorch_transformers_amd.config import AutoConfig, ConfigError


def _rot(dims, scaling=True):
    r = {"base": 10000.0, "dims": dims}
    if scaling:
        r["scaling"] = {"factor": 4.0, "original": 64, "fast": 8.0, "slow": 1.0}
    return r


def _mlp(kind):
    return {"dense": {"kind": "dense", "ff": 32},
            "moe": {"kind": "moe", "expert": {"ff": 8}, "router": {"experts": 6, "top": 2, "scale": 1.5,
                                                                   "groups": {"count": 3, "keep": 2}}, "shared": {"ff": 12}},
            None: None}[kind]


def _latent(mlp="dense", **over):
    m = {"heads": 3, "dim": 24, "rot_dim": 8, "vdim": 20, "kv_rank": 40, "q_rank": 28, "scale": 0.2, "rot": _rot(8)}
    m.update(over)
    return {"type": "latent_attention", "mixer": m, "mlp": _mlp(mlp)}


def _attn(mlp="dense", **over):
    m = {"heads": 4, "kv_heads": 2, "dim": 24, "vdim": 20, "scale": 0.2, "softcap": 9.0, "rot": _rot(16, False)}
    m.update(over)
    return {"type": "attention", "mixer": m, "mlp": _mlp(mlp)}


def _cfg(layers, **more):
    return dict({"architecture": "Nopuzen", "vocab": 50, "width": 32, "norm": {"eps": 1e-5}, "layers": layers}, **more)


def test_the_architecture_key_chooses_the_design():
    cfg = AutoConfig.from_dict(_cfg([_latent(), _attn("moe")]))
    assert type(cfg).__name__ == "NopuzenConfig" and cfg.model_type == "nopuzen" and cfg.vocab_size == 50 and cfg.eps == 1e-5
    again = AutoConfig.from_dict(cfg.to_dict())
    assert again.layers == cfg.layers


def _moe_with(**router):
    mlp = _mlp("moe")
    mlp["router"].update(router)
    return dict(_attn(), mlp=mlp)


@pytest.mark.parametrize("layers,more,word", [
    ([dict(_attn(), type="conv")], {}, "type"),
    ([_attn(kv_heads=3)], {}, "multiple"),
    ([_attn(softcap=-1.0)], {}, "softcap"),
    ([_attn(rot=_rot(26, False))], {}, "dims"),
    ([_attn(rot=_rot(7, False))], {}, "dims"),
    ([_latent(rot=_rot(10))], {}, "dims"),
    ([_latent(q_rank=0)], {}, "q_rank"),
    ([{"type": "latent_attention", "mixer": {"heads": 2}, "mlp": None}], {}, "lacks"),
    ([dict(_attn(), mlp={"kind": "glu", "ff": 8})], {}, "kind"),
    ([_moe_with(top=5)], {}, "top"),
    ([_moe_with(groups={"count": 4, "keep": 1})], {}, "groups"),
    ([_moe_with(groups={"count": 3, "keep": 4})], {}, "groups"),
    ([_moe_with(scale="big")], {}, "scale"),
    ([_attn()], {"norm": {}}, "eps"),
    ([], {}, "layers"),
])
def test_configurations_that_cannot_be_built_are_refused_by_name(layers, more, word):
    with pytest.raises(ConfigError, match=word):
        AutoConfig.from_dict(_cfg(layers, **more))


def _spec(cfg):
    from pytorch_transformers_amd.config.registry import lookup

    c = AutoConfig.from_dict(cfg)
    spec = lookup(c.model_type)[1](c)
    spec.validate()
    return spec


def test_tensor_names_and_shapes_follow_the_design():
    spec = _spec(_cfg([_latent(), _attn("moe", heads=6, kv_heads=3, dim=8, vdim=16, rot=None), _latent(None)]))
    shapes = {}
    for s in spec.tensor_specs():
        for n, shape in ([(s.name, s.shape)] if not s.pieces else s.pieces):
            shapes[n] = tuple(shape)
    assert shapes["embed"] == (50, 32) and shapes["final.norm"] == shapes["final.norm.b"] == (32,)
    for n in ("norm1", "norm1.b", "norm2", "norm2.b"):
        assert shapes[f"l0.{n}"] == (32,)
    assert shapes["l0.mix.dq"] == (28, 32) and shapes["l0.mix.dq.norm"] == (28,) and shapes["l0.mix.uq"] == (96, 28)
    assert shapes["l0.mix.dkv"] == (48, 32) and shapes["l0.mix.dkv.norm"] == (40,)
    assert shapes["l0.mix.uk"] == (72, 40) and shapes["l0.mix.uv"] == (60, 40)
    assert shapes["l0.mix.g"] == (60, 32) and shapes["l0.mix.o"] == (32, 60)
    assert shapes["l0.mlp.up"] == (32, 32) and shapes["l0.mlp.down"] == (32, 32) and shapes["l0.mlp.act"] == (2,)
    assert shapes["l1.mix.q"] == (48, 32) and shapes["l1.mix.q.b"] == (48,) and shapes["l1.mix.k"] == (24, 32)
    assert shapes["l1.mix.v"] == (48, 32) and shapes["l1.mix.v.b"] == (48,) and shapes["l1.mix.o"] == (32, 96)
    assert shapes["l1.mix.o.b"] == (32,) and shapes["l1.mix.g"] == (6, 32)
    assert shapes["l1.mix.q.norm"] == shapes["l1.mix.k.norm"] == (8,) and shapes["l1.mix.temp"] == shapes["l1.mix.pb"] == (6,)
    assert shapes["l1.mlp.router"] == (6, 32) and shapes["l1.mlp.e5.up"] == (8, 32) and shapes["l1.mlp.e0.down"] == (32, 8)
    assert shapes["l1.mlp.shared.up"] == (12, 32) and shapes["l1.mlp.shared.down"] == (32, 12)
    assert shapes["l1.mlp.shared.sg"] == (1, 32)
    assert not any(n.startswith(("l2.mlp", "l2.norm2")) or n.endswith((".gate", ".q", ".weight")) and n.startswith("l0") for n in shapes)


def test_layers_that_keep_the_same_rows_share_a_page_pool():
    spec = _spec(_cfg([_latent(), _attn("moe"), _latent(None, heads=5, vdim=8), _latent(kv_rank=24), _attn(None, dim=40, vdim=8),
                       _attn(heads=8, kv_heads=2, dim=20, vdim=32)]))
    runs = [(c.block, c.cache_group, c.cache_layer) for c in spec.order]
    assert [r[0] for r in runs] == list(range(6)) and len(set(r[1:] for r in runs)) == 6
    groups = {g.name: g for g in spec.cache_groups}
    assert len(groups) == 4 and all(g.kind == "full" for g in groups.values())
    a, b = groups[runs[0][1]], groups[runs[3][1]]
    assert runs[0][1] == runs[2][1] and not a.values and a.kv_heads == 1 and a.head_dim == 48 and a.num_layers == 2
    assert not b.values and b.head_dim == 32 and b.num_layers == 1
    c, d = groups[runs[1][1]], groups[runs[4][1]]
    assert runs[1][1] == runs[5][1] and c.values and c.kv_heads == 2 and c.head_dim == 32 and c.num_layers == 2
    assert d.values and d.head_dim == 48 and d.num_layers == 1


@pytest.mark.parametrize("dims,base,scaling", [(8, 10000.0, None), (16, 50.0, {"factor": 4.0, "original": 64, "fast": 8.0, "slow": 1.0}),
                                               (64, 500000.0, {"factor": 16.0, "original": 4096, "fast": 32.0, "slow": 1.0}),
                                               (2, 100.0, {"factor": 2.0, "original": 8, "fast": 1.0, "slow": 1.0}),
                                               (12, 10000.0, {"factor": 8.0, "original": 100000, "fast": 64.0, "slow": 0.5})])
def test_the_builders_frequencies_are_the_plain_ones(dims, base, scaling):
    """The table a mixer rotates by, and what its cosines and sines are multiplied by, against the plain formulas: no
    ramp, a ramp inside the table, a ramp that is clamped at either end."""
    import plain_nopuzen as P
    from pytorch_transformers_amd.engine.nopuzen import _positions

    rot = {"base": base, "dims": dims}
    if scaling:
        rot["scaling"] = scaling
    for pairing in ("half", "interleaved"):
        r = _positions(rot, dims + 4, pairing).rotation()
        want = P.rotary_frequencies(rot)
        assert r.rotary_dim == dims and r.pairing == pairing
        assert float((r.inv_freq.double() - want).abs().max()) <= 1e-7 * float(want.abs().max())
        assert abs(r.scale - P.rotary_magnitude(rot)) < 1e-12
    assert _positions(None, 16, "half").rotation() is None
