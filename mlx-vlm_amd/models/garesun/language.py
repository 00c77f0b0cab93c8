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

from types import SimpleNamespace
from typing import Dict

import torch

from ... import _lib, ops
from ..cache import HybridPool, PagedSequence, RecurrentCache, RowCache
from ..ragged import DecodeRows, RaggedLanguageModel, _al8  # noqa: F401  (DecodeRows: the row state callers import from here)
from ..ragged import inv_freq as _inv_freq
from ..ragged import pack_cols as _pack_cols
from ..ragged import pack_rows as _pack_rows
from .config import ModelConfig


class LanguageModel(RaggedLanguageModel):
    NAME = "Garesun"

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
