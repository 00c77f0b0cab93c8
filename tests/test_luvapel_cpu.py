"""Host side of the Luvapel model package (no GPU): config parsing and its refusals, the registry lookup by config.json,
the hybrid pool's typed row caches and auxiliary state, weight loading and its shape checks on the CPU device, and the
plain oracle against itself (causality, the window's edge, the convolution's reach, shared layer weights)."""
import numpy as np
import pytest
import torch

from tests import luvapel_helpers as H
from tests import luvapel_oracle as O

F64 = torch.float64


def test_config_reads_every_size_and_refuses_what_the_design_does_not_have():
    from mlx_vlm_amd.models.luvapel import ModelConfig

    cfg = H.config(H.mixed_layers(), vocab=123, width=56, scale=1.5, eps=3e-4)
    mc = ModelConfig.from_dict(cfg)
    assert (mc.vocab, mc.width, mc.embedding_scale, mc.norm_eps, len(mc.layers)) == (123, 56, 1.5, 3e-4, 6)
    assert mc.layers[2].mlp is None and mc.layers[4].weights_of == 1 and mc.layers[0].weights_of is None
    assert mc.layers[3].mixer["left"]["mask"]["size"] == 70 and mc.layers[3].mixer["right"]["conv"] == 2
    bad = H.config([H.general()])
    bad["layers"][0]["type"] = "convolution"
    with pytest.raises(ValueError):
        ModelConfig.from_dict(bad)
    L = H.mixed_layers()
    fwd = ModelConfig.from_dict(H.config([H.shared(L, 1), L[1], dict(H.shared(L, 1), weights_of=0), L[0]]))
    assert [l.weights_of for l in fwd.layers] == [1, None, 1, None]               # a later source; a borrowing source is followed
    for layers in ([H.shared(L, 0)],                                              # names itself
                   [L[0], dict(H.shared(L, 0), weights_of=7)],                                      # no such layer
                   [dict(H.shared(L, 1), weights_of=1), dict(H.shared(L, 1), weights_of=0)],  # no layer with tensors of its own
                   [L[0], dict(H.shared(L, 1), weights_of=0)],                    # another entry than the layer it names
                   [H.parallel(heads=5, kv_heads=2)], [H.parallel(rheads=5, rkv=2)], [H.parallel(rot_dims=5)],
                   [H.parallel(dim=8, rot_dims=10)], [H.parallel(window=0)], [H.parallel(conv=0)]):
        with pytest.raises(ValueError):
            ModelConfig.from_dict(H.config(layers))
    moe = H.config([H.general()])
    moe["layers"][0]["mlp"]["kind"] = "moe"
    with pytest.raises(ValueError):
        ModelConfig.from_dict(moe)
    uneq = H.config([H.parallel()])
    uneq["layers"][0]["mixer"]["left"]["vdim"] = 8                                # the values are the keys
    with pytest.raises(ValueError):
        ModelConfig.from_dict(uneq)


def test_registry_finds_the_package_by_architecture():
    from mlx_vlm_amd.utils import get_model_and_args

    arch, name = get_model_and_args({"architecture": "Luvapel"})
    assert name == "luvapel" and hasattr(arch, "Model") and hasattr(arch, "ModelConfig")


def test_hybrid_pool_typed_rows_and_auxiliary_state():
    from mlx_vlm_amd.models.cache import PAGE, HybridPool, PagedSequence, RecurrentCache

    pool = HybridPool(2, {(1, "k"): (12, torch.float32), (1, "v"): 12, 0: 6}, {0: (2, 4, 5, False), 1: (3, 4, 6, False)},
                      max_tokens=3 * PAGE, max_seqs=2, device="cpu", dtype=torch.bfloat16, aux_layers={1: (3, 20)})
    assert pool.rows[(1, "k")].dtype == torch.float32 and pool.rows[(1, "v")].dtype == torch.bfloat16 and pool.rows[0].shape == (3, PAGE, 6)
    assert pool.aux[1].shape == (2, 3, 20) and pool.aux[1].dtype == torch.float32
    s = PagedSequence(pool)
    st = RecurrentCache(s, 1).state
    assert [tuple(t.shape) for t in st] == [(3, 4, 6), (3, 20)] and not RecurrentCache(s, 1).is_trimmable()
    assert pool.nbytes == sum(t.numel() * t.element_size() for t in list(pool.rows.values()) + list(pool.state.values()) + [pool.aux[1]])
    s.reserve(2 * PAGE + 1)
    assert pool.free_pages == 0
    s.release()
    assert pool.free_pages == 3


def test_weights_load_on_the_host_and_wrong_shapes_are_refused():
    from mlx_vlm_amd.models.luvapel import LanguageModel, ModelConfig

    cfg = H.config(H.mixed_layers())
    W = H.weights(cfg, seed=1)
    lm = LanguageModel(ModelConfig.from_dict(cfg), device="cpu", dtype="float32", kv_pool_tokens=256, max_seqs=3).load_weights(W)
    assert lm._L[4].wproj is lm._L[1].wproj and lm._L[4].off == lm._L[1].off         # shared tensors
    assert sorted(lm.pool.state) == [0, 1, 2, 3, 4, 5] and sorted(lm.pool.aux) == [1, 3, 4]
    assert lm.pool.rows[(4, "k")] is not lm.pool.rows[(1, "k")] and lm.pool.aux[4].shape == (3, 3, 2 * 3 * 16 + 6 * 24)
    assert all(o % 8 == 0 for ns in lm._L for o in ns.off.values())
    assert lm._L[1].normw.shape == (6 * 24,) and torch.equal(lm._L[1].normw[:24], lm._L[1].normw[24:48])
    assert len(lm.make_cache()) == 6 and lm.STATEFUL
    for name in ("l1.mix.left.k", "l0.mix.w2", "l3.mix.right.v.conv", "head"):
        bad = dict(W)
        bad[name] = W[name][:-1]
        with pytest.raises(ValueError):
            LanguageModel(ModelConfig.from_dict(cfg), device="cpu", dtype="float32", kv_pool_tokens=64, max_seqs=1).load_weights(bad)
    missing = {k: v for k, v in W.items() if k != "l5.mix.r"}
    with pytest.raises(KeyError):
        LanguageModel(ModelConfig.from_dict(cfg), device="cpu", dtype="float32", kv_pool_tokens=64, max_seqs=1).load_weights(missing)
    assert not any(k.startswith("l4.") for k in W)
    # a borrowing layer may stand before its source
    L = H.mixed_layers()
    cfg2 = H.config([H.shared(L, 1), L[1], L[0]])
    lm2 = LanguageModel(ModelConfig.from_dict(cfg2), device="cpu", dtype="float32", kv_pool_tokens=64, max_seqs=1).load_weights(H.weights(cfg2))
    assert lm2._L[0].wproj is lm2._L[1].wproj and lm2._L[0].type == "parallel" and lm2._L[2].type == "general_delta"


def test_oracle_is_causal_and_its_edges_sit_where_they_should():
    cfg = H.config(H.mixed_layers())
    W = H.weights(cfg, seed=5)
    ids = np.random.default_rng(0).integers(0, cfg["vocab"], 60)
    o = O.Oracle(cfg, W, F64)
    whole = o.forward(ids)
    assert (o.forward(ids[:31]) - whole[:31]).abs().max() < 1e-9                 # a prefix does not see what follows
    # window: query i sees exactly keys i - size + 1 .. i
    m = H.parallel(window=5)["mixer"]["left"]
    cfg1 = H.config([H.parallel(window=5)])
    W1 = {k: v.double() for k, v in H.weights(cfg1, seed=2).items()}
    h = torch.randn(20, cfg1["width"], dtype=F64)
    base = O.window_attention(h, W1, "l0.mix.left.", m, 1e-5)
    for j, seen in ((15, True), (14, False), (19, True)):
        h2 = h.clone()
        h2[j] += 1.0
        d = (O.window_attention(h2, W1, "l0.mix.left.", m, 1e-5)[19] - base[19]).abs().max()
        assert (d > 1e-9) == seen, j
    # convolution: taps tokens back and no further; the last column is the current token's
    x = torch.zeros(10, 3, dtype=F64)
    x[4] = 1.0
    w = torch.tensor([[1.0, 2.0, 3.0, 4.0]] * 3, dtype=F64)
    y = O.short_conv_silu(x, w)
    silu = torch.nn.functional.silu
    assert torch.allclose(y[:, 0], silu(torch.tensor([0, 0, 0, 0, 4.0, 3.0, 2.0, 1.0, 0, 0], dtype=F64)))
    # pair rotation keeps norms and leaves the dimensions past `dims` alone
    v = torch.randn(3, 2, 8, dtype=F64)
    r = O.rotate_pairs(v, torch.tensor([0, 5, 77]), 6, 100.0)
    assert torch.allclose(r.norm(dim=-1), v.norm(dim=-1)) and torch.equal(r[0], v[0]) and torch.equal(r[..., 6:], v[..., 6:])
    assert torch.allclose(r[1, 0, 0], v[1, 0, 0] * np.cos(5.0) - v[1, 0, 1] * np.sin(5.0))


def test_delta_rules_replace_what_the_state_returned():
    """one key written twice with full strength: the second value replaces the first (a plain sum would return both)"""
    D = 4
    k = torch.zeros(D, dtype=F64)
    k[1] = 1.0
    S = torch.zeros(D, 3, dtype=F64)
    for v in (torch.tensor([1.0, 2.0, 3.0], dtype=F64), torch.tensor([-5.0, 0.5, 7.0], dtype=F64)):
        S = S + torch.outer(k, 1.0 * (v - S.T @ k))
    assert torch.allclose(S.T @ k, torch.tensor([-5.0, 0.5, 7.0], dtype=F64))
    # the general form with removal rate 1 and no decay forgets the old value along the unit key before it writes
    S = torch.outer(k, torch.tensor([1.0, 2.0, 3.0], dtype=F64))
    u = O.unit(k)
    S = S - torch.outer(1.0 * u, S.T @ u) + torch.outer(k, torch.tensor([9.0, 9.0, 9.0], dtype=F64))
    assert torch.allclose(S.T @ k, torch.tensor([9.0, 9.0, 9.0], dtype=F64), atol=1e-5)
