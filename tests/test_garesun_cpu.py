"""Host side of the Garesun model package (no GPU): config parsing and its refusals, the registry lookup by config.json, the
hybrid pool's page / slot bookkeeping, weight packing, and the plain oracle against itself (a prompt fed in pieces gives
what the whole prompt gives - the property the device tests then demand of the kernels)."""
import numpy as np
import pytest
import torch

from tests import garesun_helpers as H
from tests import garesun_oracle as O


def test_config_reads_every_size_and_refuses_what_the_design_does_not_have():
    from mlx_vlm_amd.models.garesun import ModelConfig

    cfg = H.config(H.MIXED, vocab=123, width=56, side=5, scale=1.5, eps=3e-4)
    mc = ModelConfig.from_dict(cfg)
    assert (mc.vocab, mc.width, mc.side_dim, mc.embedding_scale, mc.norm_eps, len(mc.layers)) == (123, 56, 5, 1.5, 3e-4, 6)
    assert mc.layers[4].mlp is None and mc.layers[4].experts == 0
    assert (mc.layers[5].top, mc.layers[5].shared_ff, mc.layers[0].shared_ff) == (1, 0, 16)
    no_side = dict(cfg)
    del no_side["token_side"]
    assert ModelConfig.from_dict(no_side).side_dim == 0
    bad = H.config([H.layer("retention")])
    bad["layers"][0]["type"] = "convolution"
    with pytest.raises(ValueError):
        ModelConfig.from_dict(bad)
    for layers in ([H.layer("latent_attention", kv_from=0)],                                   # names itself
                   [H.layer("mlstm"), H.layer("latent_attention", kv_from=0)],                 # not an attention layer
                   [H.layer("latent_attention"), H.layer("latent_attention", kv_from=0, kv_rank=48)],
                   [H.layer("latent_attention"), H.layer("latent_attention", kv_from=0), H.layer("latent_attention", kv_from=1)]):
        with pytest.raises(ValueError):
            ModelConfig.from_dict(H.config(layers))
    with pytest.raises(ValueError):
        ModelConfig.from_dict(H.config([H.layer("retention", heads=3, decay=[0.9, 0.8])]))
    with pytest.raises(ValueError):
        ModelConfig.from_dict(H.config([H.layer("mlstm", experts=2, top=3)]))


def test_registry_finds_the_package_by_architecture():
    from mlx_vlm_amd.utils import get_model_and_args

    arch, name = get_model_and_args({"architecture": "Garesun"})
    assert name == "garesun" and hasattr(arch, "Model") and hasattr(arch, "ModelConfig")
    with pytest.raises(ValueError):
        get_model_and_args({})


def test_hybrid_pool_gives_pages_and_slots_back():
    from mlx_vlm_amd.models.cache import PAGE, HybridPool, PagedSequence

    pool = HybridPool(3, {1: 12}, {0: (2, 4, 5, True), 2: (3, 4, 6, False)}, max_tokens=4 * PAGE, max_seqs=2, device="cpu",
                      dtype=torch.float32)
    assert pool.rows[1].shape == (4, PAGE, 12) and pool.state[0].shape == (2, 2, 4, 5) and list(pool.scalar) == [0]
    a, b = PagedSequence(pool), PagedSequence(pool)
    a.reserve(PAGE + 1)
    b.reserve(2 * PAGE)
    assert pool.free_pages == 0 and sorted(a.pages + b.pages) == [0, 1, 2, 3]
    with pytest.raises(RuntimeError):
        a.reserve(2 * PAGE + 1)
    with pytest.raises(RuntimeError):
        PagedSequence(pool)
    assert pool.block_table[a.seq, :2].tolist() == a.pages
    pa = list(a.pages)
    a.release()
    c = PagedSequence(pool)
    c.reserve(2 * PAGE)
    assert c.seq == a.seq and sorted(c.pages) == sorted(pa)         # the freed slot and pages are used again


def test_weight_packing_aligns_sections():
    from mlx_vlm_amd.models.garesun.language import _pack_cols, _pack_rows

    a, b = torch.ones(5, 6), 2 * torch.ones(3, 6)
    m, off = _pack_rows([("a", a), ("b", b)], torch.float32, "cpu")
    assert off == {"a": 0, "b": 8} and m.shape == (16, 6) and m[5:8].abs().sum() == 0 and m[8:11].eq(2).all()
    m, off = _pack_cols([("a", a.T), ("b", b.T)], torch.float32, "cpu")
    assert off == {"a": 0, "b": 8} and m.shape == (6, 16) and m[:, 11:].abs().sum() == 0


def test_oracle_is_consistent_under_cuts():
    cfg = H.config(H.MIXED)
    W = H.weights(cfg, seed=5)
    ids = np.random.default_rng(0).integers(0, cfg["vocab"], 40)
    whole = O.Oracle(cfg, W, torch.float64).forward(ids)
    o = O.Oracle(cfg, W, torch.float64)
    parts = torch.cat([o.forward(ids[:7]), o.forward(ids[7:9]), o.forward(ids[9:39]), o.forward(ids[39:])])
    assert (parts - whole).abs().max() < 1e-9
    # rotations: both pairings are norm-preserving and differ
    x = torch.randn(3, 2, 8, dtype=torch.float64)
    pos = torch.tensor([0, 5, 77])
    for f in (O.rope_half, O.rope_interleaved):
        y = f(x, pos, 6, 100.0)
        assert torch.allclose(y.norm(dim=-1), x.norm(dim=-1)) and torch.equal(y[0], x[0]) and torch.equal(y[..., 6:], x[..., 6:])
    assert not torch.allclose(O.rope_half(x, pos, 6, 100.0), O.rope_interleaved(x, pos, 6, 100.0))
