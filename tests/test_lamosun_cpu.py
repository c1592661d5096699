"""Lamosun's configuration reader, checkpoint names and cache shapes (no GPU), and the float64
reference against itself: a prompt's logits do not depend on what follows a position, and the
frequency table the framework builds equals the reference's."""
import pytest
import torch

from tests import lamosun_oracle as R
from vllm_legacy_amd.model.lamosun import LamosunConfig, LamosunForCausalLM
from vllm_legacy_amd.model.registry import resolve, supported_architectures

YARN = {"factor": 8.0, "original": 64, "fast": 16.0, "slow": 2.0}


def small():
    return R.make_config([R.rglru_layer(24, 2, conv=3, mlp=R.dense_mlp(40)),
                          R.latent_layer(4, 8, 4, 12, 10, 6, scaling=YARN, mlp=R.moe_mlp(3, 2, 10)),
                          R.delta_layer(4, 2, 8, vdim=12, conv=2, mlp=None)], vocab=50, width=32, side_dim=5)


def test_registry_and_config():
    assert "Lamosun" in supported_architectures()
    model_cls, config_cls = resolve("Lamosun")
    assert model_cls is LamosunForCausalLM and config_cls is LamosunConfig
    cfg = LamosunConfig.from_dict(small())
    g, a, d = (layer.mixer for layer in cfg.layers)
    assert (g.width, g.blocks, g.taps) == (24, 2, 3)
    assert (a.heads, a.dim, a.rot_dim, a.vdim, a.kv_rank, a.q_rank, a.rot_dims) == (4, 8, 4, 12, 10, 6, 4)
    assert a.rot_scaling == YARN and (d.heads, d.kv_heads, d.dim, d.vdim, d.taps) == (4, 2, 8, 12, 2)
    m = cfg.layers[1].mlp
    assert (m.kind, m.experts, m.top, m.ff) == ("moe", 3, 2, 10) and cfg.layers[2].mlp is None
    assert (cfg.alpha, cfg.embed_scale, cfg.side_dim, cfg.softcap) == (1.5, 3.0, 5, 20.0)
    raw = small()
    del raw["token_side"], raw["logit_softcap"], raw["embedding"]
    cfg = LamosunConfig.from_dict(raw)
    assert (cfg.embed_scale, cfg.side_dim, cfg.softcap) == (1.0, 0, 0.0)


def test_checkpoint_names_and_cache_shapes():
    raw = small()
    cfg = LamosunConfig.from_dict(raw)
    model = LamosunForCausalLM(cfg, torch.float32, "cpu")
    W = R.random_tensors(raw, 0)
    assert {k: tuple(v.shape) for k, v in W.items()} == model.tensor_shapes()
    assert model.load_weights(W) == len(W)
    assert set(model.random_weights(1)) == set(W)
    caches = model.allocate_caches(5, 4, 2)
    assert caches[0]["state"].shape == (2, 24) and caches[0]["conv"].shape == (2, 2, 24)
    assert caches[1]["latent"].shape == (5, 4, 14) and set(caches[1]) == {"latent"}
    assert caches[2]["state"].shape == (2, 4, 12, 8) and caches[2]["conv"].shape == (2, 1, 2 * 2 * 8 + 4 * 12)
    del W["l1.mlp.router.b"]
    with pytest.raises(KeyError):
        model.load_weights(W)


def test_bad_configs_are_refused():
    raw = small()
    raw["layers"][0]["type"] = "lstm"
    with pytest.raises(ValueError):
        LamosunConfig.from_dict(raw)
    raw = small()
    raw["layers"][1]["mlp"]["router"]["top"] = 9
    with pytest.raises(ValueError):
        LamosunConfig.from_dict(raw)
    raw = small()
    raw["layers"][2]["mixer"]["kv_heads"] = 3
    with pytest.raises(ValueError):
        LamosunConfig.from_dict(raw)
    raw = small()
    raw["layers"][0]["mixer"]["blocks"] = 5
    with pytest.raises(ValueError):
        LamosunConfig.from_dict(raw)


def test_frequency_table_matches_the_reference():
    from vllm_legacy_amd.attention.backends.latent_kv import yarn_frequencies
    for dims, base, sc in ((8, 10000.0, None), (32, 1e6, {"factor": 4.0, "original": 2048, "fast": 32.0, "slow": 1.0}),
                           (6, 300.0, YARN), (64, 5e5, {"factor": 40.0, "original": 4096, "fast": 32.0, "slow": 1.0})):
        rot = {"dims": dims, "base": base, **({"scaling": sc} if sc else {})}
        f, mag = yarn_frequencies(dims, base, sc)
        want_f, want_mag = R.yarn_frequencies(rot)
        assert torch.equal(f, want_f.to(torch.float32)) and abs(mag - want_mag) < 1e-12
        if sc:      # the fastest pair keeps its frequency, the slowest is divided by the factor
            assert float(f[0]) == 1.0 and abs(float(f[-1]) * sc["factor"] / base**(-(dims - 2) / dims) - 1) < 1e-6


def test_reference_is_causal():
    raw = small()
    W = R.random_tensors(raw, 1)
    toks = torch.randint(0, 50, (12, ), generator=torch.Generator().manual_seed(0)).tolist()
    full = R.forward(raw, W, toks)
    part = R.forward(raw, W, toks[:7])
    assert float((full[:7] - part).abs().max()) < 1e-9
