"""Garesun on MI355X against the plain restatement in tests/garesun_oracle.py (float64 on the CPU, token by token).

Small random checkpoints with unequal sizes (tests/garesun_helpers.py) are written to disk and loaded through
`utils.load_model` (registry by config.json, safetensors reader, weight packing).  float32 serving is compared tightly,
bfloat16 within the rounding of a 16-bit projection chain.  Covered: every mechanism alone (operator level and as a one-
layer model); whole prompts against portions of several sizes (down to two tokens) and against token-by-token decoding;
batches of unequal requests against each alone; pages and state slots freed and used again; attention keys far back, at
page and tile borders, in prompts and decoding, with one score made to stand out; the first tokens; long decoding; sizes
that are equal or 1 elsewhere (top = 1, no shared expert, no feed-forward, no token input, partial rotation, shared
latent cache); greedy generation through generate_step and the continuous batch generator."""
import numpy as np
import pytest
import torch

from tests import garesun_helpers as H
from tests import garesun_oracle as O

pytestmark = pytest.mark.gpu
F64 = torch.float64


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


TOL = {"float32": 2e-5, "bfloat16": 4e-2}
Q = {"float32": 1.0, "bfloat16": 0.8}         # bf16: see garesun_helpers.rel_rms


# ------------------------------------------------------------------------------------------------ operators
def test_linear_any_all_formats_and_batched():
    from mlx_vlm_amd import ops

    g = torch.Generator().manual_seed(1)
    for M in (1, 3, 8, 9, 70):
        a, w = torch.randn(M, 37, generator=g), torch.randn(29, 37, generator=g)
        for ta in (torch.float32, torch.bfloat16):
            for tw in (torch.float32, torch.bfloat16):
                for tc in (torch.float32, torch.bfloat16):
                    A, Wt = a.to(ta).cuda(), w.to(tw).cuda()
                    got = ops.linear_any(A, Wt, out_dtype=tc).float().cpu()
                    want = (A.double().cpu() @ Wt.double().cpu().T)
                    tol = 1e-5 if tc == torch.float32 else 1e-2
                    assert (got.double() - want).abs().max() <= tol * want.abs().max(), (M, ta, tw, tc)
    # accumulate onto an fp32 stream; rows do not depend on their neighbours
    a, w = torch.randn(40, 24, generator=g).cuda(), torch.randn(16, 24, generator=g).cuda()
    x = torch.ones(40, 16, device="cuda")
    ops.linear_any(a, w, out=x, accumulate=True)
    assert torch.allclose(x.cpu(), 1 + a.cpu() @ w.cpu().T, atol=1e-5)
    assert torch.equal(ops.linear_any(a[:20], w), ops.linear_any(a, w)[:20])
    # per-head maps inside wider rows
    Hh, D, R, X = 3, 5, 7, 2
    q = torch.randn(11, Hh * (D + X), generator=g).cuda()
    wk = torch.randn(Hh, R, D, generator=g).cuda()
    out = torch.zeros(11, Hh * (R + X), device="cuda")
    ops.linear_any(q, wk.view(Hh * R, D), out=out, M=11, N=R, K=D, batch=Hh, stride_a=D + X, stride_w=R * D, stride_c=R + X)
    want = torch.einsum("thd,hrd->thr", q.view(11, Hh, D + X)[..., :D], wk)
    assert torch.allclose(out.view(11, Hh, R + X)[..., :R], want, atol=1e-5)
    assert out.view(11, Hh, R + X)[..., R:].abs().max() == 0


def test_stream_row_operators():
    from mlx_vlm_amd import ops

    g = torch.Generator().manual_seed(2)
    x = (torch.randn(9, 50, generator=g) * 3 + 1.5)
    w = torch.randn(50, generator=g)
    got = ops.layernorm_nobias(x.cuda(), w.cuda(), 1e-5).cpu()
    assert torch.allclose(got.double(), O.layer_norm_nobias(x.double(), w.double(), 1e-5), atol=1e-5)
    y = torch.randn(9, 50, generator=g)
    xs = x.clone().cuda()
    ops.unit_rms_add_(xs, y.cuda(), w.cuda(), 1e-5)
    assert torch.allclose(xs.cpu().double(), x.double() + O.unit_rms(y.double(), 1e-5) * w.double(), atol=1e-5)
    ids = torch.tensor([3, 0, 6, 6, 1, 2, 5, 4, 3], dtype=torch.int32)
    table = torch.randn(7, 12, generator=g)
    gate = torch.randn(9, 4, generator=g)
    got = ops.gelu_tanh_gate_rows(gate.cuda(), table.cuda(), ids.cuda(), 8).cpu()
    assert torch.allclose(got.double(), O.gelu_tanh(gate.double()) * table.double()[ids.long()][:, 8:12], atol=1e-6)
    emb = ops.embed_scale_f32(ids.cuda(), table.to(torch.bfloat16).cuda(), 2.5).cpu()
    assert torch.equal(emb, table.to(torch.bfloat16).float()[ids.long()] * 2.5)


@pytest.mark.parametrize("E,top", [(5, 2), (8, 8), (70, 1), (130, 6)])
def test_moe_route_top_k_and_softmax_over_chosen(E, top):
    from mlx_vlm_amd import ops

    z = torch.randn(33, E, generator=torch.Generator().manual_seed(E))
    z[0, :] = 0.25                                    # all equal: the lowest indices win
    gate, idx, wgt = (t.cpu() for t in ops.moe_route(z.cuda(), top))
    val, ref_idx = torch.topk(z[1:], top, dim=-1)
    assert torch.equal(idx[1:].long(), ref_idx)
    assert torch.allclose(wgt[1:], torch.softmax(val, -1), atol=1e-6)
    assert sorted(idx[0].tolist()) == list(range(top))
    dense = torch.zeros(33, E).scatter_(1, idx.long(), wgt)
    assert torch.equal(gate, dense)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("kind", ["retention", "mlstm", "latent_attention"])
def test_each_mixer_alone_and_each_feed_forward_shape(tmp_path, kind, dtype):
    for j, kw in enumerate((dict(mlp=None), dict(), dict(top=1, shared_ff=0), dict(experts=3, top=3))):
        cfg = H.config([H.layer(kind, **kw)], side=(0 if j == 0 else 8))
        W = H.weights(cfg, seed=10 + j)
        lm = _load(tmp_path, cfg, W, dtype, name=f"{kind}{j}").language_model
        ids = _ids(50, cfg["vocab"], j)
        want = O.Oracle(cfg, W, F64).forward(ids)
        assert H.rel_rms(_whole(lm, ids), want, Q[dtype]) < TOL[dtype], (kind, kw)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_layers_match_layer_by_layer(tmp_path, dtype):
    cfg = H.config(H.MIXED)
    W = H.weights(cfg, seed=3)
    lm = _load(tmp_path, cfg, W, dtype).language_model
    ids = _ids(70, cfg["vocab"], 5)
    orc = O.Oracle(cfg, W, F64)
    orc.forward(ids)
    lm._trace = []
    try:
        _whole(lm, ids)
        for i, (got, want) in enumerate(zip(lm._trace, orc.trace)):
            err = H.rel_rms(got.cpu(), want, Q[dtype])
            assert err < (1e-5 if dtype == "float32" else 2e-2), (i, cfg["layers"][i]["type"], float(err))
    finally:
        lm._trace = None


# ------------------------------------------------------------------------------------------------ schedules
@pytest.fixture(scope="module")
def mixed32(tmp_path_factory):
    cfg = H.config(H.MIXED)
    W = H.weights(cfg, seed=7)
    lm = _load(tmp_path_factory.mktemp("g32"), cfg, W, "float32", tokens=1024, seqs=4).language_model
    return cfg, W, lm


def _portions(lm, ids, sizes):
    """feed ids in portions of the given sizes (cycled), every row's logits"""
    c = lm.make_cache()
    out, o, j = [], 0, 0
    while o < len(ids):
        n = min(sizes[j % len(sizes)], len(ids) - o)
        out.append(lm.step([(c[0]._seq, ids[o:o + n])], want="all").cpu())
        o, j = o + n, j + 1
    c[0]._seq.release()
    return torch.cat(out)


def test_portions_and_token_by_token_equal_the_whole_prompt(mixed32):
    cfg, W, lm = mixed32
    ids = _ids(150, cfg["vocab"], 11)          # crosses two page borders and the recurrence's 16-token staging blocks
    whole = _whole(lm, ids)
    assert H.rel_rms(whole, O.Oracle(cfg, W, F64).forward(ids)) < TOL["float32"]
    for sizes in ([2], [3, 61, 2, 64], [37, 2, 3], [64], [63, 1, 1, 65], [1]):
        got = _portions(lm, ids, sizes)
        assert torch.equal(got, whole), sizes               # float32 serving: the same bits however the prompt is cut


def test_bf16_portions_and_decode(tmp_path):
    cfg = H.config(H.MIXED)
    W = H.weights(cfg, seed=8)
    lm = _load(tmp_path, cfg, W, "bfloat16", tokens=1024, seqs=4).language_model
    ids = _ids(140, cfg["vocab"], 12)
    want = O.Oracle(cfg, W, F64).forward(ids)
    for sizes in ([140], [2, 30, 64, 5], [100] + [1] * 40):
        assert H.rel_rms(_portions(lm, ids, sizes), want, Q["bfloat16"]) < TOL["bfloat16"], sizes


def test_unequal_batch_equals_each_alone_and_slots_are_reused(mixed32):
    cfg, W, lm = mixed32
    V = cfg["vocab"]
    reqs = [_ids(n, V, 20 + n) for n in (130, 1, 23, 70, 66, 5, 90)]
    alone = [_whole(lm, r) for r in reqs]
    free0, slots0 = lm.pool.free_pages, len(lm.pool._free_seqs)
    # four live requests at a time (the pool has four slots); the others queue and take over freed pages / slots
    live, done, queue, got = {}, {}, list(range(len(reqs))), {i: [] for i in range(len(reqs))}
    rng = np.random.default_rng(0)
    seen_slots = []
    while queue or live:
        while queue and len(live) < 4:
            i = queue.pop(0)
            live[i] = [lm.make_cache(), 0]
            seen_slots.append(live[i][0][0]._seq.seq)
        entries, who = [], []
        for i, (c, o) in live.items():
            if rng.random() < 0.25 and len(live) > 1:
                continue                                   # left out of this step
            n = int(min(len(reqs[i]) - o, rng.choice([1, 1, 2, 3, 17, 64])))
            entries.append((c[0]._seq, reqs[i][o:o + n]))
            who.append((i, n))
        if not entries:
            continue
        lg = lm.step(entries, want="all").cpu()
        r = 0
        for i, n in who:
            got[i].append(lg[r:r + n])
            r += n
            live[i][1] += n
            if live[i][1] == len(reqs[i]):
                live.pop(i)[0][0]._seq.release()
    assert len(set(seen_slots)) <= 4 and len(seen_slots) == len(reqs)          # slots were used again
    assert lm.pool.free_pages == free0 and len(lm.pool._free_seqs) == slots0   # everything was given back
    for i in range(len(reqs)):
        assert torch.equal(torch.cat(got[i]), alone[i]), i     # ... and whatever else is in the batch, whichever slot and pages


def test_pool_exhaustion_is_an_error_not_a_fault(tmp_path):
    cfg = H.config([H.layer("latent_attention")])
    lm = _load(tmp_path, cfg, H.weights(cfg), "float32", tokens=128, seqs=2).language_model
    a, b = lm.make_cache(), lm.make_cache()
    lm.step([(a[0]._seq, _ids(100, 97, 0))])
    with pytest.raises(RuntimeError):
        lm.step([(b[0]._seq, _ids(10, 97, 1))])               # both pages are taken
    with pytest.raises(RuntimeError):
        lm.make_cache()                                          # both slots are taken
    a[0]._seq.release()
    lm.step([(b[0]._seq, _ids(100, 97, 1))])
    b[0]._seq.release()


# ------------------------------------------------------------------------------------------------ far keys, borders
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_latent_attention_finds_one_key_anywhere(dtype):
    """operator level: one cached row is made to score far above the rest; the output must be that row's latent, wherever
    it sits (first token, page borders 63 / 64, tile borders 255 / 256, far back, the query's own position)"""
    from mlx_vlm_amd import ops
    from mlx_vlm_amd.models.cache import PAGE

    R, Dr, Hh, n = 24, 8, 3, 700
    g = torch.Generator().manual_seed(4)
    rows = torch.randn(n, R + Dr, generator=g) * 0.1
    pages = torch.randperm(16, generator=g)[: (n + PAGE - 1) // PAGE].to(torch.int32)         # scattered pages
    pool = torch.zeros(16, PAGE, R + Dr)
    for j in range(n):
        pool[pages[j // PAGE], j % PAGE] = rows[j]
    pool_d = pool.to(dtype).cuda()
    bt = torch.zeros(2, 16, dtype=torch.int32)
    bt[1, : len(pages)] = pages
    qdir = torch.randn(R + Dr, generator=g)
    qdir /= qdir.norm()
    for key in (0, 1, 63, 64, 65, 255, 256, 257, 511, 512, 640, 699):
        for qpos in (key, key + 1, 699):
            if qpos >= n:
                continue
            p2 = pool_d.clone()
            p2[pages[key // PAGE], key % PAGE] = (rows[key] + 6.0 * qdir).to(dtype)
            q = (qdir * 8.0).repeat(Hh, 1).reshape(1, Hh, R + Dr).cuda()
            out = ops.latent_attn(q, p2, torch.tensor([1], dtype=torch.int32).cuda(), torch.tensor([qpos], dtype=torch.int32).cuda(),
                                  bt.cuda(), Hh, R, Dr, 1.0).cpu()
            want = p2[pages[key // PAGE], key % PAGE, :R].float().cpu()
            assert (out[0] - want).abs().max() < 1e-3, (key, qpos)
        if key + 1 < n:                                        # ... and one position BEFORE the key it must not be seen
            out = ops.latent_attn(q, p2, torch.tensor([1], dtype=torch.int32).cuda(), torch.tensor([key - 1 if key else 0], dtype=torch.int32).cuda(),
                                  bt.cuda(), Hh, R, Dr, 1.0).cpu()
            if key:
                assert (out[0] - want).abs().max() > 0.05, key


def test_far_key_through_the_model_in_prompt_and_decoding(tmp_path):
    """model level: a latent-attention layer whose query and key projections are scaled up, so that softmax weight sits on
    few keys; a token 600 back is then visible in the logits - compared in a prompt, in portions and decoded one by one"""
    cfg = H.config([H.layer("latent_attention", heads=2, kv_rank=16, dim=16), H.layer("retention")], side=0)
    W = H.weights(cfg, seed=21)
    W["l0.mix.q"] = (W["l0.mix.q"].float() * 4).to(torch.bfloat16)
    W["l0.mix.uk"] = (W["l0.mix.uk"].float() * 4).to(torch.bfloat16)
    lm = _load(tmp_path, cfg, W, "float32", tokens=2048, seqs=2).language_model
    ids = _ids(700, cfg["vocab"], 3)
    ids[650:] = ids[40:90]                       # the tail repeats tokens seen 610 back
    want = O.Oracle(cfg, W, F64).forward(ids)
    whole = _whole(lm, ids)
    assert H.rel_rms(whole[600:], want[600:]) < TOL["float32"]
    assert H.rel_rms(_portions(lm, ids, [640] + [1] * 60)[600:], want[600:]) < TOL["float32"]
    assert H.rel_rms(_portions(lm, ids, [255, 2, 63])[600:], want[600:]) < TOL["float32"]


def test_first_tokens_and_a_one_token_request(mixed32):
    cfg, W, lm = mixed32
    for n in (1, 2, 3):
        ids = _ids(n, cfg["vocab"], 40 + n)
        assert H.rel_rms(_whole(lm, ids), O.Oracle(cfg, W, F64).forward(ids)) < TOL["float32"], n


def test_long_decoding_keeps_the_recurrent_state(tmp_path):
    cfg = H.config([H.layer("mlstm"), H.layer("retention", decay=[0.999, 0.9, 0.5])], side=4)
    W = H.weights(cfg, seed=31)
    lm = _load(tmp_path, cfg, W, "float32", tokens=1024, seqs=2).language_model
    ids = _ids(400, cfg["vocab"], 9)
    want = O.Oracle(cfg, W, F64).forward(ids)
    got = _portions(lm, ids, [20] + [1] * 380)
    assert H.rel_rms(got[-50:], want[-50:]) < TOL["float32"]


def test_other_sizes_wide_heads_and_many_experts(tmp_path):
    layers = [H.layer("mlstm", heads=1, dim=72, vdim=130, experts=20, top=4, ff=8), H.layer("latent_attention", heads=1, kv_rank=264, dim=8, rot_dim=2, vdim=40),
              H.layer("retention", heads=7, dim=8, vdim=8, rot_dims=2, decay=[0.9] * 7), H.layer("latent_attention", heads=2, kv_rank=264, rot_dim=2, kv_from=1)]
    cfg = H.config(layers, vocab=301, width=100, side=3, scale=0.7, eps=1e-3)
    W = H.weights(cfg, seed=41)
    ids = _ids(90, 301, 2)
    want = O.Oracle(cfg, W, F64).forward(ids)
    for dtype in ("float32", "bfloat16"):
        lm = _load(tmp_path, cfg, W, dtype, name=dtype).language_model
        assert H.rel_rms(_portions(lm, ids, [70, 2, 1]), want, Q[dtype]) < TOL[dtype], dtype


# ------------------------------------------------------------------------------------------------ generation paths
def _greedy_oracle(cfg, W, prompt, n):
    """teacher: float64 greedy continuation, and the margin of every choice"""
    orc = O.Oracle(cfg, W, F64)
    lg = orc.forward(prompt)[-1]
    out, margins = [], []
    for _ in range(n):
        top2 = torch.topk(lg, 2).values
        margins.append(float(top2[0] - top2[1]))
        out.append(int(lg.argmax()))
        lg = orc.forward([out[-1]])[-1]
    return out, margins


def test_greedy_generation_through_generate_step_and_the_batch_generator(tmp_path):
    from mlx_vlm_amd.batch import BatchGenerator
    from mlx_vlm_amd.generate import generate_step

    cfg = H.config(H.MIXED[:4])
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

    cfg = H.config(H.MIXED[:3])
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

    cfg = H.config(H.MIXED)
    W = H.weights(cfg, seed=71)
    lm = _load(tmp_path, cfg, W, "bfloat16", tokens=2048, seqs=6).language_model
    sargs = make_sampler().engine_args()
    prompts = [_ids(n, cfg["vocab"], 80 + n) for n in (40, 7, 66)]

    def run(use_graph):
        caches = lm.make_cache_batch(3)
        lg = lm.prefill(torch.cat([torch.as_tensor(p) for p in prompts]).cuda().reshape(-1, 1), None, caches, [len(p) for p in prompts])
        st = lm.decode_begin(caches, lg.argmax(-1), np.zeros((3, 1)), max_new_tokens=80)
        out = []
        for i in range(70):                                          # crosses a page border in every row
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


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_latent_attention_prompt_form_equals_row_form(dtype):
    """the two attention kernels (query blocks through LDS / one row per workgroup) against a dense softmax, ragged batch:
    two sequences at different offsets on scattered pages, blocks that end inside a tile"""
    from mlx_vlm_amd import ops
    from mlx_vlm_amd.models.cache import PAGE

    R, Dr, Hh = 40, 8, 3
    g = torch.Generator().manual_seed(9)
    lens, offs = [37, 5], [150, 0]                   # sequence 0: 37 new tokens after 150 cached ones; sequence 1: 5 from the start
    bt = torch.zeros(3, 8, dtype=torch.int32)
    bt[1, :3] = torch.tensor([5, 2, 7])
    bt[2, :1] = torch.tensor([4])
    pool = (torch.randn(8, PAGE, R + Dr, generator=g) * 0.5).to(dtype)
    tok_seq = torch.tensor([1] * 37 + [2] * 5, dtype=torch.int32)
    tok_pos = torch.tensor(list(range(150, 187)) + list(range(5)), dtype=torch.int32)
    q = torch.randn(42, Hh, R + Dr, generator=g)
    gate = torch.randn(42, Hh, generator=g).to(dtype)
    qb_start = torch.tensor([0, 16, 32, 37], dtype=torch.int32)
    qb_count = torch.tensor([16, 16, 5, 5], dtype=torch.int32)
    a = ops.latent_attn(q.cuda(), pool.cuda(), tok_seq.cuda(), tok_pos.cuda(), bt.cuda(), Hh, R, Dr, 0.3, gate=gate.cuda()).cpu()
    b = ops.latent_attn_blocks(q.cuda(), pool.cuda(), qb_start.cuda(), qb_count.cuda(), tok_seq.cuda(), tok_pos.cuda(), bt.cuda(), Hh, R, Dr,
                               0.3, gate=gate.cuda()).cpu()
    want = torch.zeros(42, Hh, R, dtype=torch.float64)
    for t in range(42):
        sq, pos = int(tok_seq[t]), int(tok_pos[t])
        rows = torch.stack([pool[bt[sq, j // PAGE], j % PAGE] for j in range(pos + 1)]).double()
        w = torch.softmax(torch.einsum("hd,jd->hj", q[t].double(), rows) * 0.3, -1)
        want[t] = torch.einsum("hj,jr->hr", w, rows[:, :R]) * torch.sigmoid(gate[t].double())[:, None]
    assert (a.double() - want).abs().max() < 2e-5 and (b.double() - want).abs().max() < 2e-5


def test_sampled_generation_uses_the_device_sampler_and_refuses_what_is_not_built(tmp_path):
    from mlx_vlm_amd.generate import generate_step

    cfg = H.config(H.MIXED[:3])
    model = _load(tmp_path, cfg, H.weights(cfg, seed=91), "bfloat16", tokens=1024, seqs=4)
    p = _ids(20, cfg["vocab"], 5)
    runs = [[t for t, _ in generate_step(p[None], model, None, None, max_tokens=16, temperature=0.8, top_p=0.9, seed=7)] for _ in range(2)]
    assert runs[0] == runs[1] and len(runs[0]) == 16 and all(0 <= t < cfg["vocab"] for t in runs[0])
    other = [t for t, _ in generate_step(p[None], model, None, None, max_tokens=16, temperature=0.8, top_p=0.9, seed=8)]
    greedy = [t for t, _ in generate_step(p[None], model, None, None, max_tokens=16, temperature=0.0)]
    assert other != runs[0] or greedy != runs[0]                    # the draw depends on the seed / temperature
    with pytest.raises(NotImplementedError):
        list(generate_step(p[None], model, None, None, max_tokens=4, repetition_penalty=1.3))
    assert len(model.language_model.pool._free_seqs) == 4           # every generation gave its slot back
