"""Tekezen's configuration reader, checkpoint names and cache shapes (no GPU), and the float64
reference against itself: a prompt's logits do not depend on what follows a position, a key
outside every window and not among the kept first tokens does not matter, the hashed pair rows,
and the frequency tables the framework builds equal the reference's."""
import pytest
import torch

from tests import tekezen_oracle as R
from vllm_legacy_amd.model.registry import resolve, supported_architectures
from vllm_legacy_amd.model.tekezen import TekezenConfig, TekezenForCausalLM

YARN = {"factor": 8.0, "original": 64, "fast": 16.0, "slow": 2.0}


def small():
    return R.make_config([
        R.attention_layer(4, 2, 8, vdim=12, window=5, keep_first=2, rot_dims=4, factor=4.0, softcap=15.0, v_mix=True,
                          mlp=R.dense_mlp(40, 1.5)),
        R.latent_layer(3, 8, 4, 12, 10, window=7, scaling=YARN, mlp=R.moe_mlp(3, 2, 10, 2.5, 6, 0.5)),
        R.attention_layer(2, 2, 8, vdim=12, v_mix=True, mlp=None)], vocab=50, width=32, buckets=17, mul_prev=3, mul_cur=11)


def test_registry_and_config():
    assert "Tekezen" in supported_architectures()
    model_cls, config_cls = resolve("Tekezen")
    assert model_cls is TekezenForCausalLM and config_cls is TekezenConfig
    cfg = TekezenConfig.from_dict(small())
    a, l, b = (layer.mixer for layer in cfg.layers)
    assert (a.heads, a.kv_heads, a.dim, a.vdim, a.window, a.keep_first, a.rot_dims) == (4, 2, 8, 12, 5, 2, 4)
    assert (a.softcap, a.rot_factor, a.v_mix, a.scale) == (15.0, 4.0, True, 8**-0.5)
    assert (l.heads, l.dim, l.rot_dim, l.vdim, l.kv_rank, l.window, l.rot_dims) == (3, 8, 4, 12, 10, 7, 4)
    assert l.rot_scaling == YARN
    # what a config does not mention does not exist: no window, no kept tokens, no cap, factor 1
    assert (b.window, b.keep_first, b.softcap, b.rot_factor, b.rot_dims) == (0, 0, 0.0, 1.0, 8)
    d, m = cfg.layers[0].mlp, cfg.layers[1].mlp
    assert (d.kind, d.ff, d.limit) == ("dense", 40, 1.5) and cfg.layers[2].mlp is None
    assert (m.kind, m.experts, m.top, m.ff, m.limit, m.shared_ff, m.shared_limit) == ("moe", 3, 2, 10, 2.5, 6, 0.5)
    assert (cfg.buckets, cfg.mul_prev, cfg.mul_cur, cfg.vocab, cfg.width) == (17, 3, 11, 50, 32)


def test_checkpoint_names_and_cache_shapes():
    raw = small()
    cfg = TekezenConfig.from_dict(raw)
    model = TekezenForCausalLM(cfg, torch.float32, "cpu")
    W = R.random_tensors(raw, 0)
    assert {k: tuple(v.shape) for k, v in W.items()} == model.tensor_shapes()
    assert model.load_weights(W) == len(W)
    assert set(model.random_weights(1)) == set(W)
    # the first blending layer is the one the others read; the stream norms hold 1 + w
    assert [layer.blends for layer in model.layers if layer.spec.type == "attention"] == [False, True]
    assert torch.equal(model.layers[0].norm1.data, 1.0 + W["l0.norm1"].float())
    caches = model.allocate_caches(5, 4, 2)
    assert caches[0]["keys"].shape == (5, 4, 2, 8) and caches[0]["values"].shape == (5, 4, 2, 12)
    assert caches[1]["latent"].shape == (5, 4, 14) and set(caches[1]) == {"latent"}
    assert caches[3]["last_token"].shape == (2, ) and caches[3]["last_token"].dtype == torch.int64
    del W["l1.mlp.shared.gate"]
    with pytest.raises(KeyError):
        model.load_weights(W)


def test_bad_configs_are_refused():
    raw = small()
    raw["layers"][0]["type"] = "lstm"
    with pytest.raises(ValueError):
        TekezenConfig.from_dict(raw)
    raw = small()
    raw["layers"][1]["mlp"]["router"]["top"] = 9
    with pytest.raises(ValueError):
        TekezenConfig.from_dict(raw)
    raw = small()
    raw["layers"][0]["mixer"]["kv_heads"] = 3
    with pytest.raises(ValueError):
        TekezenConfig.from_dict(raw)
    raw = small()
    raw["layers"][2]["mixer"]["vdim"] = 8        # blending layers must agree on their values' shape
    with pytest.raises(ValueError):
        TekezenConfig.from_dict(raw)
    raw = small()
    raw["layers"][0]["mlp"]["limit"] = 0.0
    with pytest.raises(ValueError):
        TekezenConfig.from_dict(raw)


def test_frequency_tables_match_the_reference():
    from vllm_legacy_amd.attention.backends.latent_kv import yarn_frequencies
    from vllm_legacy_amd.attention.backends.rotary_kv import inverse_frequencies
    for dims, base, sc in ((8, 10000.0, None), (32, 1e6, {"factor": 4.0, "original": 2048, "fast": 32.0, "slow": 1.0}),
                           (6, 300.0, YARN), (64, 5e5, {"factor": 40.0, "original": 4096, "fast": 32.0, "slow": 1.0})):
        rot = {"dims": dims, "base": base, **({"scaling": sc} if sc else {})}
        f, mag = yarn_frequencies(dims, base, sc)
        want_f, want_mag = R.yarn_frequencies(rot)
        assert torch.equal(f, want_f.to(torch.float32)) and abs(mag - want_mag) < 1e-12
    for dims, base, factor in ((8, 10000.0, 1.0), (6, 300.0, 4.0), (32, 5e5, 2.0)):
        assert torch.equal(inverse_frequencies(base, dims, None, factor),
                           (R.plain_frequencies(dims, base) / factor).to(torch.float32))


def test_pair_rows():
    assert R.pair_rows([3, 0, 7, 7], 10, 4, 3) == [10, (3 * 4) % 10, (0 * 4 + 7 * 3) % 10, (7 * 4 + 7 * 3) % 10]
    assert R.pair_rows([5], 10, 4, 3) == [10]


def test_reference_is_causal_and_windowed():
    raw = small()
    W = R.random_tensors(raw, 1)
    toks = torch.randint(0, 50, (12, ), generator=torch.Generator().manual_seed(0)).tolist()
    full = R.forward(raw, W, toks)
    part = R.forward(raw, W, toks[:7])
    assert float((full[:7] - part).abs().max()) < 1e-9
    # visibility: window 3 with two kept tokens
    vis = R.visible(8, 3, 2)
    assert vis[7].tolist() == [True, True, False, False, False, True, True, True]
    assert vis[2].tolist() == [True, True, True, False, False, False, False, False]
    assert R.visible(8, 0)[5].tolist() == [True] * 6 + [False] * 2
    # one layer: a key outside the window and not kept has no say
    q, k, v = (torch.randn(9, 2, 4, dtype=R.F, generator=torch.Generator().manual_seed(s)) for s in (1, 2, 3))
    base = R.attention_core(q, k, v, 0.5, 10.0, 3, 2)
    k2, v2 = k.clone(), v.clone()
    k2[4] += 5.0
    v2[4] -= 3.0
    moved = R.attention_core(q, k2, v2, 0.5, 10.0, 3, 2)
    assert float((moved[7:] - base[7:]).abs().max()) == 0.0 and float((moved[4:7] - base[4:7]).abs().max()) > 1e-3
