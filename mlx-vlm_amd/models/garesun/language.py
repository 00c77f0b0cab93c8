"""Garesun language model on the HIP operator library.

One `step()` runs a RAGGED batch: any number of segments, each a run of consecutive tokens of one sequence - a whole
prompt, a portion of one, or a single decoded token - side by side.  Every kernel takes per-token (sequence, position)
or per-segment (slot, first position) tables, so a prompt portion next to decode rows is one launch sequence, and the
result of a token does not depend on how its prompt was cut or on its neighbours in the batch.  `prefill`,
`decode_begin` / `decode_run` and `decode_step_rows` are the entry points the generation paths (generate.py, batch.py)
call on every language model; here they are thin wrappers over `step()`.

Numerics: the residual stream is fp32 in both serving modes.  dtype bfloat16: weights, projections and cached latents
are bf16 (fp32 accumulation); float32: everything is fp32.  Norm statistics, rotary angles, attention scores and
softmax, router logits, recurrent state and gates are fp32 in both.

Per layer (x: stream, h = LayerNorm(x)):
    proj  = h @ [mixer projections | expert up-projections | shared up]^T      one GEMM (rows packed at load)
    mixer : recurrence kernels (rotation, scan, head norm and output gate fused) or latent attention (absorbed form)
    ff    : router (fp32) -> top-k gate table -> relu^2 * gate into the columns behind the mixer's output
    x    += [mixer out | expert activations] @ [W_o | W_down of every expert | shared W_down]^T     one GEMM
    x    += unit_rms(proj_side(gelu_tanh(gate_side x) * side_embed[token, layer slice])) * w        per-layer token input
"""
from __future__ import annotations

import ctypes as C
import os
from types import SimpleNamespace
from typing import Dict, List, Optional, Sequence

import numpy as np
import torch

from ... import _lib, ops
from ..base import LanguageModelOutput
from ..cache import PAGE, HybridPool, PagedSequence, RecurrentCache, RowCache
from .config import ModelConfig


def _al8(n: int) -> int:
    return (n + 7) & ~7


def _pack_rows(parts, dtype, device):
    """[(name, tensor [n_i, K])] -> (one matrix with every part starting at a multiple of 8 rows, {name: first row})"""
    K = parts[0][1].shape[1]
    offs, n = {}, 0
    for name, t in parts:
        offs[name] = n
        n = _al8(n + t.shape[0])
    out = torch.zeros(n, K, dtype=dtype, device=device)
    for name, t in parts:
        out[offs[name]: offs[name] + t.shape[0]] = t
    return out, offs


def _pack_cols(parts, dtype, device):
    """[(name, tensor [N, k_i])] -> (one matrix [N, sum of 8-aligned k_i], {name: first column})"""
    N = parts[0][1].shape[0]
    offs, n = {}, 0
    for name, t in parts:
        offs[name] = n
        n = _al8(n + t.shape[1])
    out = torch.zeros(N, n, dtype=dtype, device=device)
    for name, t in parts:
        out[:, offs[name]: offs[name] + t.shape[1]] = t
    return out, offs


def _inv_freq(dims: int, base: float, device):
    i = np.arange(dims // 2, dtype=np.float64)
    return torch.from_numpy((float(base) ** (-2.0 * i / dims)).astype(np.float32)).to(device)


class DecodeRows:
    """Device-resident state of B decoding rows: the fields the generation loops read and write (token, position, context
    length, sampling step counter, logits / log-probs of the last step)."""

    def __init__(self, lm: "LanguageModel", B: int, ring_len: int = 64):
        dev, V = lm.device, lm.config.vocab
        i32 = torch.int32
        self.B, self.ring_len, self.nsplit = B, ring_len, 1
        self.tok = torch.zeros(B, dtype=i32, device=dev)
        self.pos = torch.zeros(B, dtype=i32, device=dev)
        self.ctx = torch.zeros(B, dtype=i32, device=dev)
        self.step = torch.zeros(1, dtype=i32, device=dev)
        self.out_ring = torch.zeros(ring_len, B, dtype=i32, device=dev)
        VL = _al8(V)           # row pitch: 16-byte aligned rows for any vocabulary
        self.logits = torch.zeros(B, VL, dtype=torch.bfloat16, device=dev)[:, :V]
        self.logprobs = torch.zeros(B, VL, dtype=torch.bfloat16, device=dev)[:, :V]
        self.seqs: List[PagedSequence] = []
        self.row_seqs: List[PagedSequence] = []
        self.graph_key = None

    def row_penalty_tables(self):
        raise NotImplementedError("per-request logits processors are not built for this model")


class LanguageModel:
    MAX_DECODE_ROWS = 64
    # steps of up to this many rows run their big projections on the weight-streaming kernels (with the expert skip); wider
    # steps take the MFMA GEMM (measured: 1 / 2 / 4 / 8 rows 0.86 / 1.05 / 1.25 / 1.34 ms per step at width 1536 with 2, against
    # 1.39 / 2.11 ms at 4 / 8 rows with 8).  Environment override for measurements.
    STREAM_ROWS = int(os.environ.get("VLM_GARESUN_STREAM_ROWS", "2"))
    STATEFUL = True                # recurrent layers: a step that ran cannot be taken back by moving the cache offset
    supports_logits_to_keep = True

    def __init__(self, config: ModelConfig, device="cuda", dtype="bfloat16", kv_pool_tokens: int = 32768, max_seqs: int = 16,
                 **_ignored):
        self.config = self.args = config
        self.model_type = config.model_type
        self.device = device
        if isinstance(dtype, str):
            dtype = {"bfloat16": torch.bfloat16, "bf16": torch.bfloat16, "float32": torch.float32, "fp32": torch.float32}[dtype]
        if dtype not in (torch.bfloat16, torch.float32):
            raise ValueError("Garesun serves in bfloat16 or float32")
        self.dtype = dtype
        self._kv_pool_tokens, self._max_seqs = int(kv_pool_tokens), int(max_seqs)
        self.pool: Optional[HybridPool] = None
        self._L: List[SimpleNamespace] = []
        self._w: Dict[str, torch.Tensor] = {}
        self._graphs: Dict[tuple, object] = {}       # captured decode steps, see _decode_rows

    @property
    def layers(self):
        return list(range(len(self.config.layers)))

    # ------------------------------------------------------------------ weights
    def load_weights(self, W: Dict[str, torch.Tensor]):
        cfg, dev, T = self.config, self.device, self.dtype

        def g(name):
            if name not in W:
                raise KeyError(f"Garesun checkpoint: tensor {name!r} missing")
            return W[name].to(device=dev, dtype=T).contiguous()

        self._w = dict(embed=g("embed"), final_norm=g("final.norm"), head=g("head"))
        if cfg.side_dim:
            self._w["side_embed"] = g("side.embed")
            if self._w["side_embed"].shape[1] < cfg.side_dim * len(cfg.layers):
                raise ValueError("side.embed is narrower than layers x token_side.dim")
        if self._w["embed"].shape != (cfg.vocab, cfg.width) or self._w["head"].shape != (cfg.vocab, cfg.width):
            raise ValueError("embed / head shapes do not match config vocab / width")
        row_layers, state_layers = {}, {}
        self._L = []
        for i, L in enumerate(cfg.layers):
            p, m = f"l{i}.", L.mixer
            ns = SimpleNamespace(type=L.type, cfg=L, norm1=g(p + "norm1"))
            parts = []
            if L.type in ("retention", "mlstm"):
                H, D, Dv = int(m["heads"]), int(m["dim"]), int(m["vdim"])
                ns.H, ns.D, ns.Dv, ns.kmix = H, D, Dv, H * Dv
                names = ("q", "k", "v", "g") + (("i", "f") if L.type == "mlstm" else ())
                parts = [(n, g(p + "mix." + n)) for n in names]
                gated = L.type == "mlstm"
                state_layers[i] = (H, D, Dv + (1 if gated else 0), gated)
                if gated:
                    ns.ib, ns.fb, ns.normw, ns.cap = g(p + "mix.i.b"), g(p + "mix.f.b"), g(p + "mix.norm"), float(m["gate_cap"])
                    ns.inv_freq, ns.rot_dims = None, 0
                else:
                    ns.decay = torch.tensor([float(x) for x in m["decay"]], dtype=torch.float32, device=dev)
                    ns.rot_dims = int(m["rot"]["dims"])
                    if ns.rot_dims > D or ns.rot_dims % 2:
                        raise ValueError(f"layer {i}: rot.dims {ns.rot_dims} for head dim {D}")
                    ns.inv_freq = _inv_freq(ns.rot_dims, m["rot"]["base"], dev) if ns.rot_dims else None
            else:
                H, D, Dr, Dv, R = int(m["heads"]), int(m["dim"]), int(m["rot_dim"]), int(m["vdim"]), int(m["kv_rank"])
                if int(m["rot"]["dims"]) != Dr or Dr % 2:
                    raise ValueError(f"layer {i}: the rotated part is rot_dim wide (rot.dims {m['rot']['dims']} != {Dr})")
                ns.H, ns.D, ns.Dr, ns.Dv, ns.R, ns.kmix, ns.scale = H, D, Dr, Dv, R, H * Dv, float(m["scale"])
                ns.src = i if m.get("kv_from") is None else int(m["kv_from"])
                ns.inv_freq = _inv_freq(Dr, m["rot"]["base"], dev) if Dr else None
                parts = [("q", g(p + "mix.q")), ("g", g(p + "mix.g"))]
                if ns.src == i:
                    parts.append(("dkv", g(p + "mix.dkv")))
                    ns.dkv_norm = g(p + "mix.dkv.norm")
                    row_layers[i] = R + Dr
                # per-head maps of the latent, moved to the query side (transposed) and the output side
                ns.uk_t = g(p + "mix.uk").view(H, D, R).transpose(1, 2).contiguous()          # [H, R, D]
                ns.uv = g(p + "mix.uv").view(H, Dv, R).contiguous()                           # [H, Dv, R]
            outs = [("mix", g(p + "mix.o"))]
            ns.E, ns.top, ns.ff, ns.sff = L.experts, L.top, L.expert_ff, L.shared_ff
            if L.mlp is not None:
                ups = [g(p + f"mlp.e{e}.up") for e in range(ns.E)] + ([g(p + "mlp.shared.up")] if ns.sff else [])
                downs = [g(p + f"mlp.e{e}.down") for e in range(ns.E)] + ([g(p + "mlp.shared.down")] if ns.sff else [])
                parts.append(("up", torch.cat(ups, dim=0)))
                outs.append(("ff", torch.cat(downs, dim=1)))
                ns.router = g(p + "mlp.router")
            ns.wproj, ns.off = _pack_rows(parts, T, dev)
            ns.wout, ns.koff = _pack_cols(outs, T, dev)
            if cfg.side_dim:
                ns.side_gate, ns.side_proj, ns.side_norm = g(p + "side.gate"), g(p + "side.proj"), g(p + "side.norm")
            self._L.append(ns)
        # +1 page / slot: the idle rows of a continuous batch write into a scratch sequence (batch.py)
        self.pool = HybridPool(len(cfg.layers), row_layers, state_layers, self._kv_pool_tokens, self._max_seqs, device=dev, dtype=T)
        return self

    # ------------------------------------------------------------------ cache
    def make_cache(self):
        seq = PagedSequence(self.pool)
        return [RowCache(seq, i) if L.type == "latent_attention" else RecurrentCache(seq, i) for i, L in enumerate(self.config.layers)]

    def make_cache_batch(self, n: int):
        return [self.make_cache() for _ in range(n)]

    # ------------------------------------------------------------------ GEMM routing
    def _linear(self, a, w, out=None, out_dtype=None, skip=None, accumulate=False):
        """a [M, K] @ w[N, K]^T: the MFMA GEMM for bf16 operands of a prompt-sized batch with 8-aligned shapes, the generic
        kernel for everything else (fp32 mode, odd shapes, fp32 outputs), and for the up-to-8 rows of a decode step over bf16
        weights the weight-streaming form (`skip`: the expert-column skip of ops.linear_rows_bf16w)"""
        M, K = a.shape
        N = w.shape[0]
        want = out.dtype if out is not None else (out_dtype or a.dtype)
        if (not accumulate and a.dtype == torch.bfloat16 and w.dtype == torch.bfloat16 and want == torch.bfloat16 and M > self.STREAM_ROWS and K % 8 == 0 and N % 8 == 0
                and a.stride(0) % 8 == 0 and w.stride(0) % 8 == 0 and (out is None or out.stride(0) % 8 == 0)
                and a.data_ptr() % 16 == 0 and (out is None or out.data_ptr() % 16 == 0)):
            return ops.gemm(a, w, out=out)
        if M <= 8 and w.dtype == torch.bfloat16 and K % 8 == 0 and w.stride(0) % 8 == 0 and w.data_ptr() % 16 == 0:
            return ops.linear_rows_bf16w(a, w, out=out, out_dtype=out_dtype, accumulate=accumulate, **(skip or {}))
        return ops.linear_any(a, w, out=out, out_dtype=out_dtype, accumulate=accumulate)

    # ------------------------------------------------------------------ the step
    def step(self, entries, want="last", advance: bool = True, reserve_extra: int = 0, logits_dtype=torch.float32):
        """entries: [(PagedSequence, ids)] - ids a host int array or a device int32 tensor, the NEXT tokens of that sequence.
        want: "last" (one row per entry), "all", or one list of indices (into the entry's ids) per entry.
        -> logits [wanted rows in entry order, vocab] of logits_dtype (None when nothing is wanted)."""
        plan = self._plan(entries, want, reserve_extra)
        out = self._run(plan, logits_dtype)
        if advance:
            for s, n in zip(plan.seqs, plan.lens):
                s.offset += n
        return out

    def _plan(self, entries, want="last", reserve_extra: int = 0, static=None):
        """Host side of a step: pages reserved, the per-token / per-segment tables built and uploaded in ONE copy.
        static: (int32 device buffer, ids tensor) of a captured step to refill instead of allocating."""
        dev = self.device
        lens = [int(ids.numel() if isinstance(ids, torch.Tensor) else np.asarray(ids).size) for _, ids in entries]
        if not entries or min(lens) <= 0:
            raise ValueError("step: every entry brings at least one token")
        if len({id(s) for s, _ in entries}) != len(entries):
            raise ValueError("step: one entry per sequence")
        nseg, Tn = len(entries), int(sum(lens))
        seqs = [s for s, _ in entries]
        for s, n in zip(seqs, lens):
            s.reserve(s.offset + n + reserve_extra)
        cu = np.concatenate([[0], np.cumsum(lens)]).astype(np.int32)
        if isinstance(want, str) and want == "last":
            rows = cu[1:] - 1
        elif isinstance(want, str) and want == "all":
            rows = np.arange(Tn, dtype=np.int32)
        else:
            rows = np.concatenate([cu[j] + np.asarray(w, dtype=np.int32).reshape(-1) for j, w in enumerate(want)] or [np.zeros(0, np.int32)])
        rows = np.asarray(rows, dtype=np.int32)
        tok_seq = np.concatenate([np.full(n, s.seq, np.int32) for s, n in zip(seqs, lens)])
        tok_pos = np.concatenate([np.arange(s.offset, s.offset + n, dtype=np.int32) for s, n in zip(seqs, lens)])
        seg_slot = np.asarray([s.seq for s in seqs], dtype=np.int32)
        seg_pos0 = np.asarray([s.offset for s in seqs], dtype=np.int32)
        host_ids = static is None and all(not isinstance(ids, torch.Tensor) for _, ids in entries)
        # query blocks of the prompt-form attention: up to 16 consecutive tokens of one segment
        qb = [(cu[j] + o, min(16, n - o)) for j, n in enumerate(lens) for o in range(0, n, 16)]
        qb_start, qb_count = np.asarray([b[0] for b in qb], dtype=np.int32), np.asarray([b[1] for b in qb], dtype=np.int32)
        meta = [tok_seq, tok_pos, cu, seg_slot, seg_pos0, rows, qb_start, qb_count]
        if host_ids:
            meta.append(np.concatenate([np.asarray(ids, dtype=np.int32).reshape(-1) for _, ids in entries]))
        host = np.concatenate(meta)
        if static is not None:
            md = static[0]
            md[: host.size].copy_(_lib.h2d(host, dev))
        else:
            md = _lib.h2d(host, dev)
        o, parts = 0, []
        for a in meta:
            parts.append(md[o:o + a.size])
            o += a.size
        if static is not None:
            ids_d = static[1]
        elif host_ids:
            ids_d = parts[8]
        else:
            ids_d = torch.cat([(ids if isinstance(ids, torch.Tensor) else _lib.h2d(np.asarray(ids, dtype=np.int32), dev))
                               .reshape(-1).to(torch.int32) for _, ids in entries])
        return SimpleNamespace(seqs=seqs, lens=lens, nseg=nseg, Tn=Tn, rows=rows, all_rows=bool(rows.size == Tn and np.array_equal(rows, np.arange(Tn))),
                               tok_seq=parts[0], tok_pos=parts[1], cu=parts[2], slot=parts[3], pos0=parts[4], rows_d=parts[5], qb_start=parts[6],
                               qb_count=parts[7], ids=ids_d, md=md)

    def _run(self, pl, logits_dtype=torch.float32):
        """Device side of a step: nothing here looks at host data that changes between two steps of the same shape, so a
        decode step can be captured once and replayed."""
        cfg, dev, T = self.config, self.device, self.dtype
        f32 = torch.float32
        nseg, Tn = pl.nseg, pl.Tn
        tok_seq_d, tok_pos_d, cu_d, slot_d, pos0_d, ids_d = pl.tok_seq, pl.tok_pos, pl.cu, pl.slot, pl.pos0, pl.ids
        pool, bt = self.pool, self.pool.block_table
        is32 = T == f32
        few = Tn <= self.STREAM_ROWS and not is32           # decode rows over bf16 weights: weight-streaming projections with the expert skip
        x = ops.embed_scale_f32(ids_d, self._w["embed"], cfg.embedding_scale)
        keep = [pl.md, ids_d]
        for i, ns in enumerate(self._L):
            h = ops.layernorm_nobias(x, ns.norm1, cfg.norm_eps)
            gate = None
            if ns.cfg.mlp is not None:
                z = self._linear(h, ns.router, out_dtype=f32)
                gate, _, _ = ops.moe_route(z, ns.top)
                keep += [z, gate]
            skip = dict(skip_gate=gate, skip_col0=ns.off["up"], E=ns.E, ff=ns.ff) if (few and gate is not None) else None
            proj = self._linear(h, ns.wproj, skip=skip)
            cat = torch.zeros(Tn, ns.wout.shape[1], dtype=T, device=dev)
            col = lambda name: proj[:, ns.off[name]:]          # noqa: E731   (2-D view: data_ptr at the column, stride(0) = pitch)
            if ns.type in ("retention", "mlstm"):
                gated = ns.type == "mlstm"
                Cc = ns.Dv + (1 if gated else 0)
                raw = torch.empty(Tn, ns.H, Cc, dtype=f32, device=dev)
                a = _lib.RecurrenceArgs()
                a.q, a.k, a.v, a.g = (col(n).data_ptr() for n in ("q", "k", "v", "g"))
                a.ldq = a.ldk = a.ldv = a.ldg = proj.stride(0)
                if gated:
                    mtok = torch.empty(Tn, ns.H, dtype=f32, device=dev)
                    mprev = torch.empty(nseg, ns.H, dtype=f32, device=dev)
                    a.ipre, a.fpre, a.ldi, a.ldf = col("i").data_ptr(), col("f").data_ptr(), proj.stride(0), proj.stride(0)
                    a.ib, a.fb, a.cap = ns.ib.data_ptr(), ns.fb.data_ptr(), ns.cap
                    a.mstate, a.mtok, a.mprev = pool.scalar[i].data_ptr(), mtok.data_ptr(), mprev.data_ptr()
                    a.normw, a.gate_act = ns.normw.data_ptr(), 1
                    a.qscale, a.kscale = float(ns.D) ** -0.5, 1.0
                    keep += [mtok, mprev]
                else:
                    a.decay = ns.decay.data_ptr()
                    a.inv_freq = ns.inv_freq.data_ptr() if ns.inv_freq is not None else None
                    a.rot_dims, a.gate_act = ns.rot_dims, 0
                    a.qscale, a.kscale = 1.0, float(ns.D) ** -0.5
                a.eps = cfg.norm_eps
                a.seg_start, a.seg_slot, a.seg_pos0 = cu_d.data_ptr(), slot_d.data_ptr(), pos0_d.data_ptr()
                a.state, a.raw, a.out, a.ldo = pool.state[i].data_ptr(), raw.data_ptr(), cat.data_ptr(), cat.stride(0)
                a.H, a.D, a.Dv, a.gated = ns.H, ns.D, ns.Dv, int(gated)
                ops.linear_recurrence(a, nseg, Tn, is32)
                keep.append(raw)
            else:
                H, D, Dr, Dv, R = ns.H, ns.D, ns.Dr, ns.Dv, ns.R
                if ns.src == i:
                    ops.latent_kv_write(col("dkv"), ns.dkv_norm, R, Dr, ns.inv_freq, tok_seq_d, tok_pos_d, bt, pool.rows[i], cfg.norm_eps)
                qabs = torch.empty(Tn, H * (R + Dr), dtype=f32, device=dev)
                # absorbed keys: q'_h = U_k,h^T q_h for every head (batch = heads, strides inside the packed rows)
                ops.linear_any(col("q"), ns.uk_t.view(H * R, D), out=qabs, M=Tn, N=R, K=D, batch=H, stride_a=D + Dr, stride_w=R * D,
                               stride_c=R + Dr)
                if Dr:
                    ops.rope_pairs_rows(proj[:, ns.off["q"] + D:], D + Dr, H, Dr, ns.inv_freq, tok_pos_d, qabs[:, R:], R + Dr)
                # prompt form (key tiles shared by a block of queries) wherever a step brings more than decode rows, and always
                # in float32 serving - one kernel there, so that a token's bits do not depend on the schedule
                if (is32 or Tn > 8) and R <= 512 and (32 * _al8(R + Dr) + 512) * 4 <= 150 * 1024:
                    ol = ops.latent_attn_blocks(qabs.view(Tn, H, R + Dr), pool.rows[ns.src], pl.qb_start, pl.qb_count, tok_seq_d, tok_pos_d,
                                                bt, H, R, Dr, ns.scale, gate=col("g"))
                else:
                    ol = ops.latent_attn(qabs.view(Tn, H, R + Dr), pool.rows[ns.src], tok_seq_d, tok_pos_d, bt, H, R, Dr, ns.scale,
                                         gate=col("g"))
                ops.linear_any(ol.view(Tn, H * R), ns.uv.view(H * Dv, R), out=cat, M=Tn, N=Dv, K=R, batch=H, stride_a=R, stride_w=Dv * R,
                               stride_c=Dv)
                keep += [qabs, ol]
            if gate is not None:
                ops.moe_relu2_gate(col("up"), gate, ns.E, ns.ff, ns.sff, cat[:, ns.koff["ff"]:])
            if T == torch.bfloat16 and Tn > self.STREAM_ROWS:
                y = self._linear(cat, ns.wout)
                ops.stream_add_(x, y)
                keep.append(y)
            elif few:
                self._linear(cat, ns.wout, out=x, accumulate=True)      # (unchosen experts: zero activations, weights not read)
            else:
                ops.linear_any(cat, ns.wout, out=x, accumulate=True)
            if cfg.side_dim:
                sg = self._linear(x, ns.side_gate, out_dtype=T)
                gg = ops.gelu_tanh_gate_rows(sg, self._w["side_embed"], ids_d, i * cfg.side_dim)
                y2 = self._linear(gg, ns.side_proj)
                ops.unit_rms_add_(x, y2, ns.side_norm, cfg.norm_eps)
                keep += [sg, gg, y2]
            keep += [h, proj, cat]
            if self._trace is not None:
                self._trace.append(x.clone())
        self._keep = keep
        if pl.rows.size == 0:
            return None
        xl = x if pl.all_rows else x.index_select(0, pl.rows_d.long())
        hn = ops.layernorm_nobias(xl, self._w["final_norm"], cfg.norm_eps)
        # rows at a pitch of vocab rounded up to 8: 16-byte aligned bf16 rows for the samplers, whatever the vocabulary
        out = torch.empty(hn.shape[0], _al8(cfg.vocab), dtype=logits_dtype, device=dev)[:, : cfg.vocab]
        return self._linear(hn, self._w["head"], out=out)

    _trace = None      # a list: step() appends the stream after every layer (debugging / tests)

    # ------------------------------------------------------------------ entry points of generate.py / batch.py
    def prefill(self, inputs, position_ids, caches, lengths: Sequence[int], logits_rows: str = "last", reserve_extra: int = 0):
        """inputs: the token ids of the concatenated sequences (int32 [T, 1] as Model.get_input_embeddings hands them on);
        position_ids are implied by the cache offsets.  -> logits bf16 [n_seq or T, V] for the samplers"""
        ids = inputs.reshape(-1)
        if ids.dtype not in (torch.int32, torch.int64):
            raise TypeError("Garesun.prefill takes token ids (the per-layer token input needs them), not embeddings")
        entries, o = [], 0
        for c, n in zip(caches, lengths):
            entries.append((c[0]._seq, ids[o:o + n]))
            o += n
        lg = self.step(entries, want=logits_rows, reserve_extra=reserve_extra, logits_dtype=torch.bfloat16)
        return lg

    def decode_state(self, B: int):
        raise NotImplementedError("logits processors (penalties / logit_bias) are not built for this model")

    def new_decode_state(self, cap: int) -> DecodeRows:
        return DecodeRows(self, cap)

    def decode_begin(self, caches, first_tokens, rope_deltas, max_new_tokens: int, rope_pos=None) -> DecodeRows:
        seqs = [c[0]._seq for c in caches]
        st = DecodeRows(self, len(seqs))
        for s in seqs:
            s.reserve(s.offset + max_new_tokens)
        if isinstance(first_tokens, torch.Tensor):
            st.tok.copy_(first_tokens.reshape(-1).to(torch.int32))
        else:
            st.tok.copy_(_lib.h2d(np.asarray(first_tokens, dtype=np.int32).reshape(-1), self.device))
        st.seqs = st.row_seqs = seqs
        return st

    def _rows_step(self, st: DecodeRows, seqs, advance: bool):
        lg = self.step([(s, st.tok[r:r + 1]) for r, s in enumerate(seqs)], want="last", advance=advance, logits_dtype=torch.bfloat16)
        st.logits[:len(seqs)].copy_(lg)

    def _sample_rows(self, st: DecodeRows, n: int, sampler_args: dict, with_logprobs: bool = True):
        tok, lp = ops.sample(st.logits[:n], step=st.step, want_logprobs=with_logprobs, **sampler_args)
        st.tok[:n].copy_(tok)
        if lp is not None:
            st.logprobs[:n].copy_(lp)

    def _decode_rows(self, st: DecodeRows, seqs, sampler_args: dict, with_logprobs: bool, use_graph: bool, advance: bool):
        """One decode step of rows 0..n-1 of st (one token each, fed from st.tok): forward, sampling on the device, the sampled
        token written back as the next input.  With use_graph the launch sequence of a (state, row count, sampler) is captured
        into a HIP graph the second time it runs and replayed from then on: the host then only reserves pages and refills the
        small table of (sequence slot, position) per row - a step is ~100 launches, which the host cannot issue as fast as the
        GPU runs them."""
        n = len(seqs)
        entries = [(s, st.tok[r:r + 1]) for r, s in enumerate(seqs)]
        key = (id(st), n, bool(with_logprobs), tuple(sorted(sampler_args.items())))
        ent = self._graphs.get(key) if use_graph else None
        if ent is None:
            self._rows_step(st, seqs, advance=False)
            self._sample_rows(st, n, sampler_args, with_logprobs)
            self.decode_advance_rows(st, n)
            if use_graph:
                self._graphs[key] = "seen"           # the first run loads the kernels; the second one is captured
        else:
            if ent == "seen":
                meta = torch.zeros(8 * n + 1, dtype=torch.int32, device=self.device)
                pl = self._plan(entries, "last", static=(meta, st.tok[:n]))
                g = torch.cuda.CUDAGraph()
                with torch.cuda.graph(g):
                    lg = self._run(pl, torch.bfloat16)
                    st.logits[:n].copy_(lg)
                    self._sample_rows(st, n, sampler_args, with_logprobs)
                    self.decode_advance_rows(st, n)
                ent = self._graphs[key] = (g, meta, st, self._keep, lg)
            else:
                self._plan(entries, "last", static=(ent[1], st.tok[:n]))
            ent[0].replay()
        if advance:
            for s in seqs:
                s.offset += 1

    def decode_run(self, st: DecodeRows, n_steps: int, sampler_args: dict, use_graph: bool = True, penalties=None):
        """n_steps decode steps of st's rows: step, sample on the device, feed the sampled token back"""
        if penalties:
            raise NotImplementedError("logits processors are not built for this model")
        for _ in range(n_steps):
            self._decode_rows(st, st.seqs, sampler_args, True, use_graph, advance=True)

    def decode_step_rows(self, st: DecodeRows, B: int, block_table, sampler_args: dict, use_graph: bool = True,
                         with_logprobs: bool = True, row_penalties: bool = False, q8: bool = False):
        """One decode step of a continuous batch: the live rows are st.row_seqs (the scheduler's rows, in row order); rows
        past them are idle and are not run.  The scheduler advances the sequences' offsets itself."""
        if row_penalties or q8:
            raise NotImplementedError("per-request logits processors / quantized caches are not built for this model")
        self._decode_rows(st, st.row_seqs, sampler_args, with_logprobs, use_graph, advance=False)

    def decode_forward_rows(self, st: DecodeRows, B: int, block_table, q8: bool = False):
        self._rows_step(st, st.row_seqs, advance=False)

    def decode_advance_rows(self, st: DecodeRows, B: int):
        _lib.check(_lib.lib().vlm_decode_advance(st.ctx.data_ptr(), st.pos.data_ptr(), st.tok.data_ptr(), st.out_ring.data_ptr(),
                                                 st.ring_len, st.step.data_ptr(), int(B),
                                                 C.c_void_p(torch.cuda.current_stream().cuda_stream)), "decode_advance")

    def quantize_kv(self, seqs, bits: int = 8, group_size: int = 64):
        raise NotImplementedError("quantized caches are not built for this model")

    def __call__(self, inputs, inputs_embeds=None, mask=None, cache=None, **kwargs):
        """module contract: ids [1, L] (or [L]) appended to `cache` (a new one when None) -> logits [1, L or 1, V]"""
        ids = inputs.detach().cpu().numpy() if isinstance(inputs, torch.Tensor) else np.asarray(inputs)
        ids = ids.reshape(1, -1) if ids.ndim == 1 else ids
        if ids.shape[0] != 1:
            raise NotImplementedError("one sequence per call; batches go through step()")
        if cache is None:
            cache = self.make_cache()
        keep1 = kwargs.get("logits_to_keep") == 1
        lg = self.step([(cache[0]._seq, ids.reshape(-1))], want="last" if keep1 else "all")
        return LanguageModelOutput(logits=lg.view(1, -1, lg.shape[-1]))
