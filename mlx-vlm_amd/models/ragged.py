"""Language models that run a RAGGED step on the HIP operator library: the shared part.

One `step()` runs any number of segments, each a run of consecutive tokens of one sequence - a whole prompt, a portion of
one, or a single decoded token - side by side.  The host builds ONE int32 table per step (token -> sequence slot / position,
segment -> slot / first position, query blocks, wanted rows) and every kernel indexes through it, so a prompt portion next
to decode rows is one launch sequence and the result of a token does not depend on how its prompt was cut or on its
neighbours in the batch.  `prefill`, `decode_begin` / `decode_run` and `decode_step_rows` are the entry points the
generation paths (generate.py, batch.py) call on every language model; here they are thin wrappers over `step()`.

A model derives from RaggedLanguageModel and brings `load_weights` (which also builds `self.pool`, a HybridPool),
`make_cache` and `_run(plan, logits_dtype)` - the device side of a step.  Numerics: the residual stream is fp32 in both
serving modes; dtype bfloat16: weights and projections bf16 (fp32 accumulation); float32: everything fp32.
"""
from __future__ import annotations

import ctypes as C
import os
from types import SimpleNamespace
from typing import Dict, List, Optional, Sequence

import numpy as np
import torch

from .. import _lib, ops
from .base import LanguageModelOutput
from .cache import HybridPool, PagedSequence


def _al8(n: int) -> int:
    return (n + 7) & ~7


def pack_rows(parts, dtype, device):
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


def pack_cols(parts, dtype, device):
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


def inv_freq(dims: int, base: float, device):
    i = np.arange(dims // 2, dtype=np.float64)
    return torch.from_numpy((float(base) ** (-2.0 * i / dims)).astype(np.float32)).to(device)


class DecodeRows:
    """Device-resident state of B decoding rows: the fields the generation loops read and write (token, position, context
    length, sampling step counter, logits / log-probs of the last step)."""

    def __init__(self, lm: "RaggedLanguageModel", B: int, ring_len: int = 64):
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


class RaggedLanguageModel:
    NAME = "model"
    MAX_DECODE_ROWS = 64
    # steps of up to this many rows run their big projections on the weight-streaming kernels (with the expert skip); wider
    # steps take the MFMA GEMM (measured: 1 / 2 / 4 / 8 rows 0.86 / 1.05 / 1.25 / 1.34 ms per step at width 1536 with 2, against
    # 1.39 / 2.11 ms at 4 / 8 rows with 8).  Environment override for measurements.
    STREAM_ROWS = int(os.environ.get("VLM_STREAM_ROWS") or os.environ.get("VLM_GARESUN_STREAM_ROWS") or "2")
    STATEFUL = True                # recurrent layers: a step that ran cannot be taken back by moving the cache offset
    supports_logits_to_keep = True

    def __init__(self, config, device="cuda", dtype="bfloat16", kv_pool_tokens: int = 32768, max_seqs: int = 16,
                 **_ignored):
        self.config = self.args = config
        self.model_type = config.model_type
        self.device = device
        if isinstance(dtype, str):
            dtype = {"bfloat16": torch.bfloat16, "bf16": torch.bfloat16, "float32": torch.float32, "fp32": torch.float32}[dtype]
        if dtype not in (torch.bfloat16, torch.float32):
            raise ValueError(f"{self.NAME} serves in bfloat16 or float32")
        self.dtype = dtype
        self._kv_pool_tokens, self._max_seqs = int(kv_pool_tokens), int(max_seqs)
        self.pool: Optional[HybridPool] = None
        self._L: List[SimpleNamespace] = []
        self._w: Dict[str, torch.Tensor] = {}
        self._graphs: Dict[tuple, object] = {}       # captured decode steps, see _decode_rows

    @property
    def layers(self):
        return list(range(len(self.config.layers)))

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

    _trace = None      # a list: step() appends the stream after every layer (debugging / tests)

    # ------------------------------------------------------------------ entry points of generate.py / batch.py
    def prefill(self, inputs, position_ids, caches, lengths: Sequence[int], logits_rows: str = "last", reserve_extra: int = 0):
        """inputs: the token ids of the concatenated sequences (int32 [T, 1] as Model.get_input_embeddings hands them on);
        position_ids are implied by the cache offsets.  -> logits bf16 [n_seq or T, V] for the samplers"""
        ids = inputs.reshape(-1)
        if ids.dtype not in (torch.int32, torch.int64):
            raise TypeError(f"{self.NAME}.prefill takes token ids, not embeddings")
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


class TokenIdModel:
    """Module contract the generation paths expect from `models.<type>.Model` (`language_model`, `get_input_embeddings`,
    `sanitize`, `load_weights`) for a text-only model whose language model looks its embeddings up inside the step:
    `get_input_embeddings` hands the token ids through as the "embeddings" (int32 [B, L, 1])."""
    NAME = "model"
    LanguageModel = None

    def __init__(self, config, device="cuda", **kwargs):
        self.config = config
        self.model_type = config.model_type
        self.vision_tower = None
        self.language_model = self.LanguageModel(config, device=device, **kwargs)

    @property
    def layers(self):
        return self.language_model.layers

    def get_input_embeddings(self, input_ids=None, pixel_values=None, **kwargs):
        from .base import InputEmbeddingsFeatures

        if pixel_values is not None:
            raise ValueError(f"{self.NAME} is a text-only model")
        ids = np.asarray(input_ids.detach().cpu().numpy() if isinstance(input_ids, torch.Tensor) else input_ids, dtype=np.int32)
        if ids.ndim == 1:
            ids = ids[None]
        B, L = ids.shape
        pos = np.broadcast_to(np.arange(L, dtype=np.int64)[None], (B, L)).copy()
        return InputEmbeddingsFeatures(inputs_embeds=_lib.h2d(ids.reshape(B, L, 1), self.language_model.device), position_ids=pos,
                                       rope_deltas=np.zeros((B, 1), dtype=np.int64))

    def sanitize(self, weights):
        return weights

    def load_weights(self, weights):
        self.language_model.load_weights(weights)
        return self

    def __call__(self, input_ids, pixel_values=None, mask=None, cache=None, **kwargs):
        return self.language_model(input_ids, cache=cache, **kwargs)
