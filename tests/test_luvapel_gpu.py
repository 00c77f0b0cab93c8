"""Luvapel on MI355X against the plain restatement in tests/luvapel_oracle.py (float64 on the CPU, token by token).

Small random checkpoints with unequal sizes (tests/luvapel_helpers.py) are written to disk and loaded through
`utils.load_model` (registry by config.json, safetensors reader, weight packing).  float32 serving is compared tightly,
bfloat16 within the rounding of a 16-bit projection chain.  Covered: every mechanism alone (operator level and as a one-
layer model); whole prompts against portions of several sizes (down to two tokens) and against token-by-token decoding;
batches of unequal requests against each alone; pages and state slots freed and used again; attention keys at page, tile
and window borders, just inside and just outside the window, in prompts and decoding, with one score made to stand out;
associations far back in the recurrent state; the first tokens (shorter than the convolution and the window); long
decoding; sizes that are equal or 1 elsewhere (kv_heads = heads, one tap, window 1, no rotation, no feed-forward, shared
layer weights); greedy generation through generate_step and the continuous batch generator; captured decode steps."""
import numpy as np
import pytest
import torch

from tests import luvapel_helpers as H
from tests import luvapel_oracle as O

pytestmark = pytest.mark.gpu
F64 = torch.float64
TOL = {"float32": 2e-5, "bfloat16": 4e-2}


def _close(got, want, dtype):
    """float32: every row within TOL.  bfloat16: nine rows in ten within TOL and none beyond 2.5 TOL - a row whose softmax or
    unit vector sits on a near tie of the random test weights amplifies the rounding of a 16-bit projection"""
    if dtype == "float32":
        return H.rel_rms(got, want) < TOL[dtype]
    return H.rel_rms(got, want, 0.9) < TOL[dtype] and H.rel_rms(got, want) < 2.5 * TOL[dtype]


def _load(tmp_path, cfg, W, dtype, tokens=4096, seqs=6, name="m"):
    from mlx_vlm_amd.utils import load_model

    return load_model(H.write_checkpoint(str(tmp_path / name), cfg, W), dtype=dtype, kv_pool_tokens=tokens, max_seqs=seqs)


def _ids(n, vocab, seed):
    return torch.randint(0, vocab, (n,), generator=torch.Generator().manual_seed(seed)).numpy().astype(np.int32)


def _whole(lm, ids):
    c = lm.make_cache()
    lg = lm.step([(c[0]._seq, ids)], want="all").cpu()
    c[0]._seq.release()
    return lg


def _portions(lm, ids, sizes):
    """the prompt in portions of the given sizes (cycled), every row's logits"""
    c, out, o, j = lm.make_cache(), [], 0, 0
    while o < len(ids):
        n = min(sizes[j % len(sizes)], len(ids) - o)
        out.append(lm.step([(c[0]._seq, ids[o:o + n])], want="all").cpu())
        o, j = o + n, j + 1
    c[0]._seq.release()
    return torch.cat(out)


# ------------------------------------------------------------------------------------------------ operators
def test_stream_operators_of_the_gated_normed_residual():
    from mlx_vlm_amd import ops

    g = torch.Generator().manual_seed(2)
    for T in (torch.float32, torch.bfloat16):
        tol = 1e-5 if T == torch.float32 else 1e-2
        x = torch.randn(7, 50, generator=g)
        a, b, gate = (torch.randn(7, 60, generator=g).to(T) for _ in range(3))            # views with a pitch of 60
        w, wa, wb, gb = (torch.randn(50, generator=g).to(T) for _ in range(4))
        d = lambda t: t.double()[:, :50] if t.dim() == 2 else t.double()                      # noqa: E731
        for two in (False, True):
            y = d(a) if not two else 0.5 * (O.rms(d(a), 1e-5) * d(wa) + O.rms(d(b), 1e-5) * d(wb))
            want = x.double() + O.rms(y * torch.sigmoid(d(gate) + d(gb)), 1e-5) * d(w)
            xs, h = x.clone().cuda(), torch.empty(7, 50, dtype=T, device="cuda")
            kw = dict(b=b.cuda()[:, :50], wa=wa.cuda(), wb=wb.cuda()) if two else {}
            ops.gated_rms_add_(xs, a.cuda()[:, :50], w.cuda(), 1e-5, gate=gate.cuda()[:, :50], gate_bias=gb.cuda(), h=h, **kw)
            assert (xs.cpu().double() - want).abs().max() < tol * 10, (T, two)
            assert torch.equal(h.cpu(), xs.cpu().to(T))
        wn = torch.randn(50, generator=g).to(T)
        got = ops.rms_rows(x.cuda(), wn.cuda(), 1e-5).float().cpu()
        assert (got.double() - O.rms(x.double(), 1e-5) * wn.double()).abs().max() < tol * 5
        assert torch.equal(ops.stream_cast(x.cuda(), T).cpu(), x.to(T))
        up = torch.randn(5, 33, generator=g).to(T)
        assert (ops.relu2_rows(up.cuda()[:, :30]).float().cpu() - torch.relu(up.float()[:, :30]) ** 2).abs().max() < tol * 10


@pytest.mark.parametrize("D", [20, 24])
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_window_attention_both_forms_against_a_dense_softmax(dtype, D):
    """two sequences at different offsets on scattered pages (one 1890 tokens deep: the decode form walks more than one chunk
    of keys), query blocks that end inside a key tile, grouped heads, windows shorter and longer than the cached prefix, per-
    head score multipliers, elementwise output gate.  D = 24 takes the decode form with 16-byte loads, D = 20 the plain one."""
    from mlx_vlm_amd import ops
    from mlx_vlm_amd.models.cache import PAGE

    Hh, G = 6, 2
    g = torch.Generator().manual_seed(9)
    bt = torch.zeros(3, 32, dtype=torch.int32)
    bt[1, :31] = torch.randperm(31, generator=g).to(torch.int32) + 1
    bt[2, :1] = 0
    kpool = torch.randn(32, PAGE, G * D, generator=g) * 0.7
    vpool = torch.randn(32, PAGE, G * D, generator=g).to(dtype)
    tok_seq = torch.tensor([1] * 37 + [2] * 5, dtype=torch.int32)
    tok_pos = torch.tensor(list(range(1890, 1927)) + list(range(5)), dtype=torch.int32)
    q = torch.randn(42, Hh * D, generator=g)
    gate = torch.randn(42, Hh * D + 8, generator=g).to(dtype)
    temp = (1 + 0.3 * torch.randn(Hh, generator=g)).to(dtype)
    qb_start = torch.tensor([0, 16, 32, 37], dtype=torch.int32).cuda()
    qb_count = torch.tensor([16, 16, 5, 5], dtype=torch.int32).cuda()
    rows = {sq: (kpool[bt[sq].long()].reshape(-1, G, D).double(), vpool[bt[sq].long()].reshape(-1, G, D).double()) for sq in (1, 2)}
    for window in (0, 1, 3, 16, 17, 37, 64, 65, 500, 1024, 1025, 1800):
        want = torch.zeros(42, Hh, D, dtype=F64)
        for t in range(42):
            sq, pos = int(tok_seq[t]), int(tok_pos[t])
            lo = max(0, pos - window + 1) if window > 0 else 0
            for h in range(Hh):
                kh = h // (Hh // G)
                ks, vs = rows[sq][0][lo:pos + 1, kh], rows[sq][1][lo:pos + 1, kh]
                w = torch.softmax(ks @ q[t, h * D:(h + 1) * D].double() * 0.3 * temp[h].double(), 0)
                want[t, h] = (w @ vs) * torch.sigmoid(gate[t, h * D:(h + 1) * D].double())
        args = (tok_seq.cuda(), tok_pos.cuda(), bt.cuda(), Hh, G, D, D, 0.3)
        a = torch.zeros(42, Hh * D, dtype=dtype, device="cuda")
        b = torch.zeros(42, Hh * D, dtype=dtype, device="cuda")
        ops.window_attn_rows(q.cuda(), kpool.cuda(), vpool.cuda(), *args, a, temp=temp.cuda(), window=window, gate=gate.cuda()[:, : Hh * D])
        ops.window_attn_blocks(q.cuda(), kpool.cuda(), vpool.cuda(), qb_start, qb_count, *args, b, temp=temp.cuda(), window=window,
                               gate=gate.cuda()[:, : Hh * D])
        tol = 2e-5 if dtype == torch.float32 else 2e-2
        assert (a.cpu().double().view(42, Hh, D) - want).abs().max() < tol, window
        assert (b.cpu().double().view(42, Hh, D) - want).abs().max() < tol, window


def test_headnorm_rope_rows_dense_and_paged():
    from mlx_vlm_amd import ops
    from mlx_vlm_amd.models.cache import PAGE

    g = torch.Generator().manual_seed(4)
    Hh, D, dims = 3, 14, 6
    x = torch.randn(9, Hh * D + 5, generator=g)
    w = torch.randn(D, generator=g)
    pos = torch.tensor([0, 1, 63, 64, 65, 700, 5, 6, 7], dtype=torch.int32)
    seq = torch.tensor([0] * 6 + [1] * 3, dtype=torch.int32)
    bt = torch.zeros(2, 12, dtype=torch.int32)
    bt[0] = torch.arange(12, dtype=torch.int32).flip(0) + 1
    bt[1, 0] = 0
    inv = torch.tensor([500.0 ** (-2 * i / dims) for i in range(dims // 2)])
    want = O.rotate_pairs(O.rms(x[:, : Hh * D].double().view(9, Hh, D), 1e-5) * w.double(), pos, dims, 500.0)
    dense = torch.zeros(9, Hh * D, device="cuda")
    ops.headnorm_rope_rows(x.cuda()[:, : Hh * D], Hh, D, w.cuda(), 1e-5, dims, inv.cuda(), pos.cuda(), dense)
    assert (dense.cpu().double().view(9, Hh, D) - want).abs().max() < 2e-4              # fp32 angles at position 700
    kp, vp = torch.zeros(13, PAGE, Hh * D, device="cuda"), torch.zeros(13, PAGE, Hh * D, device="cuda")
    ops.headnorm_rope_rows(x.cuda()[:, : Hh * D], Hh, D, w.cuda(), 1e-5, dims, inv.cuda(), pos.cuda(), kp, tok_seq=seq.cuda(),
                           block_table=bt.cuda(), raw_pool=vp)
    for t in range(9):
        page, slot = int(bt[seq[t], pos[t] // PAGE]), int(pos[t]) % PAGE
        assert torch.equal(kp[page, slot].cpu(), dense[t].cpu()) and torch.equal(vp[page, slot].cpu(), x[t, : Hh * D])


# ------------------------------------------------------------------------------------------------ one-layer models
ONE = {"general": [H.general()], "general_wide": [H.general(heads=2, dim=72, ff=0)], "general_many_small": [H.general(heads=7, dim=8)],
       "parallel": [H.parallel()], "parallel_equal_heads_one_tap": [H.parallel(heads=3, kv_heads=3, rheads=2, rkv=2, conv=1, window=1, ff=0)],
       "parallel_no_rotation_wide": [H.parallel(heads=2, kv_heads=1, dim=72, rot_dims=0, rheads=4, rkv=1, rdim=136, rvdim=80, conv=5, window=200)],
       "parallel_full_rotation": [H.parallel(dim=16, rot_dims=16, rheads=2, rkv=2, rdim=8, rvdim=72, conv=2, window=33)]}


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("kind", sorted(ONE))
def test_each_mixer_alone(tmp_path, kind, dtype):
    cfg = H.config(ONE[kind])
    W = H.weights(cfg, seed=3)
    ids = _ids(150, cfg["vocab"], 5)
    got = _whole(_load(tmp_path, cfg, W, dtype, tokens=512).language_model, ids)
    assert _close(got, O.Oracle(cfg, W, F64).forward(ids), dtype)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_layers_match_layer_by_layer(tmp_path, dtype):
    cfg = H.config(H.mixed_layers())
    W = H.weights(cfg, seed=11)
    ids = _ids(90, cfg["vocab"], 6)
    lm = _load(tmp_path, cfg, W, dtype, tokens=512).language_model
    lm._trace = []
    c = lm.make_cache()
    lm.step([(c[0]._seq, ids)], want="all")
    ref = []
    O.Oracle(cfg, W, F64).forward(ids, ref)
    assert len(lm._trace) == len(ref) == 6
    for i, (a, b) in enumerate(zip(lm._trace, ref)):
        assert _close(a.cpu(), b, dtype), i
    lm._trace = None
    c[0]._seq.release()


# ------------------------------------------------------------------------------------------------ schedules
@pytest.fixture(scope="module")
def mixed32(tmp_path_factory):
    cfg = H.config(H.mixed_layers())
    W = H.weights(cfg, seed=21)
    model = _load(tmp_path_factory.mktemp("mixed32"), cfg, W, "float32", tokens=1024, seqs=4)
    return cfg, W, model.language_model


def test_portions_and_token_by_token_equal_the_whole_prompt(mixed32):
    cfg, W, lm = mixed32
    ids = _ids(200, cfg["vocab"], 7)
    whole = _whole(lm, ids)
    assert H.rel_rms(whole, O.Oracle(cfg, W, F64).forward(ids)) < TOL["float32"]
    for sizes in ([1], [2], [3, 1, 2], [37], [61, 2, 1], [63], [64], [65, 1, 1, 1, 2], [9, 70]):
        assert torch.equal(_portions(lm, ids, sizes), whole), sizes           # float32 serving: one summation order per token


def test_bf16_portions_and_decode(tmp_path):
    cfg = H.config(H.mixed_layers())
    W = H.weights(cfg, seed=22)
    lm = _load(tmp_path, cfg, W, "bfloat16", tokens=1024).language_model
    ids = _ids(140, cfg["vocab"], 8)
    want = O.Oracle(cfg, W, F64).forward(ids)
    for sizes in ([1], [2], [5, 1, 1, 40], [64, 3]):
        assert _close(_portions(lm, ids, sizes), want, "bfloat16"), sizes


def test_unequal_batch_equals_each_alone_and_slots_are_reused(mixed32):
    cfg, W, lm = mixed32
    rng = np.random.default_rng(3)
    reqs = [_ids(n, cfg["vocab"], 30 + n) for n in (130, 2, 75, 1, 64, 199, 33)]
    alone = [_whole(lm, r) for r in reqs]
    free0 = lm.pool.free_pages
    live, waiting, got = {}, list(range(len(reqs))), {i: [] for i in range(len(reqs))}
    used_slots = []
    while waiting or live:
        while waiting and len(live) < 4:
            i = waiting.pop(0)
            live[i] = [lm.make_cache(), 0]
            used_slots.append(live[i][0][0]._seq.seq)
        entries, who = [], []
        for i, (c, o) in live.items():
            if rng.random() < 0.25 and len(live) > 1:
                continue                                                     # left out of this step
            n = min(int(rng.choice([1, 1, 2, 3, 17, 64, 70])), len(reqs[i]) - o)
            entries.append((c[0]._seq, reqs[i][o:o + n]))
            who.append((i, n))
        if not entries:
            continue
        lg = lm.step(entries, want="all").cpu()
        o = 0
        for i, n in who:
            got[i].append(lg[o:o + n])
            o += n
            live[i][1] += n
            if live[i][1] == len(reqs[i]):
                live.pop(i)[0][0]._seq.release()
    for i in range(len(reqs)):
        assert torch.equal(torch.cat(got[i]), alone[i]), i
    assert lm.pool.free_pages == free0 and len(set(used_slots)) < len(used_slots)      # pages came back, slots were used again


def test_pool_exhaustion_is_an_error_not_a_fault(tmp_path):
    cfg = H.config([H.parallel()])
    lm = _load(tmp_path, cfg, H.weights(cfg, seed=1), "float32", tokens=128, seqs=2).language_model
    c = lm.make_cache()
    lm.step([(c[0]._seq, _ids(128, cfg["vocab"], 1))])
    with pytest.raises(RuntimeError):
        lm.step([(c[0]._seq, _ids(1, cfg["vocab"], 2))])
    c[0]._seq.release()
    c = lm.make_cache()
    lm.step([(c[0]._seq, _ids(100, cfg["vocab"], 3))])
    c[0]._seq.release()


# ------------------------------------------------------------------------------------------------ edges made visible
def _window_probe(window, D=16):
    """one attention layer whose query / key maps read one stream direction each, so that the score of a chosen earlier token
    towers over all others: the output then equals that token's value if and only if it is inside the window"""
    cfg = H.config([H.parallel(heads=2, kv_heads=1, dim=D, window=window, rot_dims=0, scale=1.0, ff=0)], width=48, vocab=64)
    W = H.weights(cfg, seed=5)
    return cfg, W


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("window", [1, 2, 16, 17, 64, 65, 130])
def test_window_edge_in_prompt_and_decoding(tmp_path, window, dtype):
    """token `mark` appears once, at distance window - 1 (just inside) or window (just outside) of the asked position; the
    embedding of `mark` and of the asking token are made so that their score stands out.  Whole prompt, portions cut at the
    edge, and decoding token by token must agree with the oracle."""
    cfg, W = _window_probe(window)
    emb = W["embed"].float()
    emb[:, :2] = 0
    emb[1], emb[2] = 0, 0
    emb[1, 0], emb[2, 1] = 4.0, 4.0                       # `mark` = 1 lives on direction 0, the asking token 2 on direction 1
    W["embed"] = emb.to(torch.bfloat16)
    k, q = W["l0.mix.left.k"].float(), W["l0.mix.left.q"].float()
    k[:, 0], q[:, 1] = 0, 0
    k[:16, 0] = 3.0                                       # key of `mark`: large along every head dimension
    q[:, 1] = 3.0                                         # query of the asking token: the same direction, both heads
    W["l0.mix.left.k"], W["l0.mix.left.q"] = k.to(torch.bfloat16), q.to(torch.bfloat16)
    W["l0.mix.left.k.norm"] = torch.full((16,), 1.5).to(torch.bfloat16)
    W["l0.mix.left.q.norm"] = torch.full((16,), 1.5).to(torch.bfloat16)
    lm = _load(tmp_path, cfg, W, dtype, tokens=1024).language_model
    orc = O.Oracle(cfg, W, F64)
    n = 2 * window + 70
    for ask in (window + 3, n - 1):
        for dist in (window - 1, window):
            if ask - dist < 0:
                continue
            ids = 3 + _ids(n, cfg["vocab"] - 3, 40 + ask + dist)
            ids[ask - dist], ids[ask] = 1, 2
            want = orc.forward(ids)
            if 0 < dist < window:                         # the probe is sharp: with and without `mark` in view differ widely
                other = ids.copy()
                other[ask - dist] = 5
                assert H.rel_rms(orc.forward(other)[ask:ask + 1], want[ask:ask + 1]) > 0.05
            for sizes in ([n], [ask - dist + 1, 1000], [ask, 1], [ask - 1, 2], [ask - dist, 1, 1000], [3, 1]):
                got = _portions(lm, ids, sizes)
                assert H.rel_rms(got[ask:ask + 1], want[ask:ask + 1]) < (2.5 if dtype == "bfloat16" else 1) * TOL[dtype], (ask, dist, sizes)
                assert _close(got, want, dtype), (ask, dist, sizes)


@pytest.mark.parametrize("kind", ["general", "parallel"])
def test_far_association_through_the_recurrent_state(tmp_path, kind):
    """decays and removal rates set close to "keep everything": what the state took in at tokens 40..43 of a long prompt still
    moves the logits hundreds of tokens later (far outside the attention window) - in a whole prompt, in portions and decoded"""
    layers = [H.general(heads=2, dim=32)] if kind == "general" else [H.parallel(window=8, rheads=2, rkv=1, rdim=64, rvdim=32)]
    cfg = H.config(layers + [H.shared(layers, 0)])
    W = H.weights(cfg, seed=13, gain=1.5)
    if kind == "general":
        W["l0.mix.w0"], W["l0.mix.a.b"] = torch.full_like(W["l0.mix.w0"], -8.0), torch.full_like(W["l0.mix.a.b"], -6.0)
    else:
        W["l0.mix.right.A_log"] = torch.full_like(W["l0.mix.right.A_log"], -8.0)
    n = 700 if kind == "general" else 330
    lm = _load(tmp_path, cfg, W, "float32", tokens=1024).language_model
    ids = _ids(n, cfg["vocab"], 77)
    want = O.Oracle(cfg, W, F64).forward(ids)
    other = ids.copy()
    other[40:44] = (other[40:44] + 1) % cfg["vocab"]
    assert H.rel_rms(O.Oracle(cfg, W, F64).forward(other)[n - 50:], want[n - 50:]) > 1e-2       # the early tokens still matter at the end
    whole = _whole(lm, ids)
    assert H.rel_rms(whole, want) < TOL["float32"]
    assert H.rel_rms(whole[n - 50:], want[n - 50:]) < TOL["float32"]
    assert torch.equal(_portions(lm, ids, [n - 100, 1]), whole) and torch.equal(_portions(lm, ids, [64, 63, 2]), whole)


def test_first_tokens_and_a_one_token_request(mixed32):
    cfg, W, lm = mixed32
    for n in (1, 2, 3, 4, 5):                                       # shorter than the convolutions (4 and 2 taps) and the windows
        ids = _ids(n, cfg["vocab"], 90 + n)
        want = O.Oracle(cfg, W, F64).forward(ids)
        assert H.rel_rms(_whole(lm, ids), want) < TOL["float32"]
        assert H.rel_rms(_portions(lm, ids, [1]), want) < TOL["float32"]


def test_long_decoding_keeps_state_conv_inputs_and_window(tmp_path):
    cfg = H.config([H.parallel(window=70, conv=4), H.general(), H.parallel(window=5, conv=3, rheads=2, rkv=1)])
    W = H.weights(cfg, seed=17)
    lm = _load(tmp_path, cfg, W, "float32", tokens=1024).language_model
    ids = _ids(400, cfg["vocab"], 19)
    want = O.Oracle(cfg, W, F64).forward(ids)
    got = _portions(lm, ids, [20] + [1] * 380)
    assert H.rel_rms(got, want) < TOL["float32"]
    assert H.rel_rms(got[-1:], want[-1:]) < TOL["float32"]


def test_other_sizes(tmp_path):
    """widths and head sizes that are not multiples of 8 or 64, a vocabulary that is odd, heads wider than 128"""
    layers = [H.general(heads=1, dim=136, ff=24), H.parallel(heads=5, kv_heads=1, dim=12, rot_dims=2, window=1000, rheads=3, rkv=3, rdim=20,
                                                              rvdim=70, conv=7, ff=16), H.general(heads=3, dim=20, ff=0)]
    cfg = H.config(layers, vocab=301, width=60, scale=0.7, eps=3e-4)
    W = H.weights(cfg, seed=23)
    ids = _ids(100, cfg["vocab"], 29)
    want = O.Oracle(cfg, W, F64).forward(ids)
    for dtype in ("float32", "bfloat16"):
        lm = _load(tmp_path, cfg, W, dtype, tokens=256, name=dtype).language_model
        assert _close(_whole(lm, ids), want, dtype), dtype
        assert _close(_portions(lm, ids, [50, 1, 2]), want, dtype), dtype


def test_borrowed_weights_before_their_source_and_with_constants_of_their_own(tmp_path):
    """a layer that uses a LATER layer's tensors, and borrowing layers whose window, score scale and rotation (which are no
    tensors) differ from their source's"""
    src = H.parallel(window=9, rot_dims=16, base=10000.0)
    early, late = H.shared([src], 0), H.shared([src], 0)
    early["weights_of"], late["weights_of"] = 1, 1
    early["mixer"]["left"].update(mask=dict(size=3), scale=0.31, rot=dict(base=50.0, dims=8))
    del late["mixer"]["left"]["mask"], late["mixer"]["left"]["rot"]                # an entry without them: every earlier key, no rotation
    cfg = H.config([early, src, H.general(), late], vocab=97, width=48, scale=1.3, eps=2e-5)
    W = H.weights(cfg, seed=31)
    assert not any(k.startswith(("l0.", "l3.")) for k in W)
    ids = _ids(90, cfg["vocab"], 37)
    want = O.Oracle(cfg, W, F64).forward(ids)
    same = O.Oracle(H.config([H.shared([src], 0) | dict(weights_of=1), src, H.general(), H.shared([src], 0) | dict(weights_of=1)],
                             vocab=97, width=48, scale=1.3, eps=2e-5), W, F64).forward(ids)
    assert H.rel_rms(same, want) > 1e-2                                          # the constants of their own matter
    for dtype in ("float32", "bfloat16"):
        lm = _load(tmp_path, cfg, W, dtype, tokens=256, name=dtype).language_model
        assert _close(_whole(lm, ids), want, dtype), dtype
        assert _close(_portions(lm, ids, [7, 1, 30, 2]), want, dtype), dtype


# ------------------------------------------------------------------------------------------------ generation
def _greedy_oracle(cfg, W, prompt, n):
    orc, ids, toks, margins = O.Oracle(cfg, W, F64), list(prompt), [], []
    for _ in range(n):
        lg = orc.forward(np.asarray(ids))[-1]
        top = torch.topk(lg, 2).values
        toks.append(int(lg.argmax()))
        margins.append(float((top[0] - top[1]) / lg.std()))
        ids.append(toks[-1])
    return toks, margins


def test_greedy_generation_through_generate_step_and_the_batch_generator(tmp_path):
    from mlx_vlm_amd.batch import BatchGenerator
    from mlx_vlm_amd.generate import generate_step

    cfg = H.config(H.mixed_layers()[:4])
    W = H.weights(cfg, seed=51)
    W["head"] = (W["head"].float() * 6).to(torch.bfloat16)          # wide margins: greedy choices survive bf16 logits
    model = _load(tmp_path, cfg, W, "float32", tokens=2048, seqs=8)
    prompts = [_ids(n, cfg["vocab"], 60 + n) for n in (9, 70, 33)]
    refs = [_greedy_oracle(cfg, W, p, 12) for p in prompts]

    def agree(got, ref):
        toks, margins = ref
        for a, b, m in zip(got, toks, margins):
            if a != b:
                assert m < 0.05, (got, toks, margins)            # a tie within the bf16 rounding of the sampler's logits
                return
    for p, ref in zip(prompts, refs):
        got = [t for t, _ in generate_step(p[None], model, None, None, max_tokens=12, temperature=0.0)]
        assert len(got) == 12
        agree(got, ref)
    gen = BatchGenerator(model, None, max_tokens=12, completion_batch_size=2, prefill_batch_size=2, compute_logprobs=True)
    uids = gen.insert([p for p in prompts])
    out = {u: [] for u in uids}
    while gen.has_work:
        _, rs = gen.next()
        for r in rs:
            out[r.uid].append(r.token)
    gen.close()
    for u, ref in zip(uids, refs):
        assert len(out[u]) == 12
        agree(out[u], ref)
    assert len(model.language_model.pool._free_seqs) >= 7         # rows gave their slots back (the scratch row keeps one)


def test_trace_session_replays_mixed_steps(tmp_path):
    from mlx_vlm_amd.batch import TraceSession

    cfg = H.config(H.mixed_layers()[:3])
    W = H.weights(cfg, seed=61)
    model = _load(tmp_path, cfg, W, "float32", tokens=256, seqs=4)
    a, b = _ids(100, cfg["vocab"], 1), _ids(30, cfg["vocab"], 2)
    wa, wb = O.Oracle(cfg, W, F64).forward(a), O.Oracle(cfg, W, F64).forward(b)
    s = TraceSession(model)
    assert s.step([("a", a[:64].tolist(), [])]) is None
    lg = s.step([("a", a[64:99].tolist(), [0, 34]), ("b", b[:29].tolist(), [28])])
    assert H.rel_rms(lg, torch.stack([wa[64], wa[98], wb[28]])) < TOL["float32"]
    lg = s.step([("b", b[29:].tolist(), [0]), ("a", a[99:].tolist(), [0])], end=["a", "b"])
    assert H.rel_rms(lg, torch.stack([wb[29], wa[99]])) < TOL["float32"]
    assert model.language_model.pool.free_pages == 4


def test_captured_decode_steps_equal_eager_ones(tmp_path):
    """a captured decode step is replayed many times, with eager work (another request's prompt, a release, synchronisations)
    between the replays; every replay's logits and token must equal the eager step's"""
    from mlx_vlm_amd.sample_utils import make_sampler

    cfg = H.config(H.mixed_layers())
    W = H.weights(cfg, seed=71)
    lm = _load(tmp_path, cfg, W, "bfloat16", tokens=2048, seqs=6).language_model
    sargs = make_sampler().engine_args()
    prompts = [_ids(n, cfg["vocab"], 80 + n) for n in (40, 7, 66)]

    def run(use_graph):
        caches = lm.make_cache_batch(3)
        lg = lm.prefill(torch.cat([torch.as_tensor(p) for p in prompts]).cuda().reshape(-1, 1), None, caches, [len(p) for p in prompts])
        st = lm.decode_begin(caches, lg.argmax(-1), np.zeros((3, 1)), max_new_tokens=80)
        out = []
        for i in range(70):                                          # crosses a page border and the windows in every row
            lm.decode_run(st, 1, sargs, use_graph=use_graph)
            out.append((st.tok.cpu().clone(), st.logits.float().cpu().clone()))
            if i % 9 == 4:                                           # eager work between replays
                other = lm.make_cache()
                lm.step([(other[0]._seq, _ids(30 + i, cfg["vocab"], i))])
                torch.cuda.synchronize()
                other[0]._seq.release()
        for c in caches:
            c[0]._seq.release()
        return out
    eager, graph = run(False), run(True)
    assert any(isinstance(v, tuple) for v in lm._graphs.values())            # a graph was captured and used
    for i, ((t0, l0), (t1, l1)) in enumerate(zip(eager, graph)):
        assert torch.equal(t0, t1) and torch.equal(l0, l1), i


def test_sampled_generation_uses_the_device_sampler_and_refuses_what_is_not_built(tmp_path):
    from mlx_vlm_amd.generate import generate_step

    cfg = H.config(H.mixed_layers()[:3])
    model = _load(tmp_path, cfg, H.weights(cfg, seed=91), "bfloat16", tokens=1024, seqs=4)
    p = _ids(20, cfg["vocab"], 5)
    runs = [[t for t, _ in generate_step(p[None], model, None, None, max_tokens=16, temperature=0.8, top_p=0.9, seed=7)] for _ in range(2)]
    assert runs[0] == runs[1] and len(runs[0]) == 16 and all(0 <= t < cfg["vocab"] for t in runs[0])
    with pytest.raises(NotImplementedError):
        list(generate_step(p[None], model, None, None, max_tokens=4, repetition_penalty=1.3))
    assert len(model.language_model.pool._free_seqs) == 4           # every generation gave its slot back
