// Delta-rule recurrences: matrix states S [D, Dv] per head (fp32, one per sequence slot) whose update READS the old state
// before it writes - the new association k -> v replaces what the state returned for that key instead of adding to it.
//
//   * gated (mode 0): one decay g_t and one write strength beta_t per head and token
//         S' = g_t S_(t-1)        u_t = beta_t (v_t - S'^T k_t)        S_t = S' + k_t u_t^T        o_t = S_t^T q_t
//     q and k are unit vectors per head (x / sqrt(sum x^2 + 1e-6), q times D^-1/2) of short causal convolutions (silu) of
//     the projections; q / k heads may be shared by groups of value heads.
//   * general (mode 1): a decay w_t and a removal rate a_t per key channel, unit key u_t = k_t / sqrt(sum k_t^2 + 1e-6)
//         S_t = diag(w_t) S_(t-1) - (a_t * u_t) (u_t^T S_(t-1)) + k_t v_t^T                        o_t = S_t^T r_t
//     both correction terms read S_(t-1).
//
// The work is split into a PREPARE pass (everything per token that does not depend on the state: convolutions, unit norms,
// gates, decays - evaluated in fp32, written as fp32 rows), the SCAN (sequential in the tokens of a segment, same arithmetic
// wherever a prompt was cut) and the finish pass shared with linear_recurrence.hip (per-head unit RMS, weight, output gate).
// A segment is a run of consecutive tokens of one sequence: the state (and the convolution's last taps - 1 inputs) comes from
// the sequence's slot - or is zero when the segment starts at position 0, so a slot that is used again needs no clearing -
// and goes back there.
//
// Scan work split: workgroup = (segment, head, tile of 32 state columns) = four waves of 8 columns; eight neighbouring lanes
// hold the eight parts of one state column's rows in registers (heads up to 1024 wide).
#include "common.hpp"
#include "../../include/vlm_hip.h"
#include "recurrence_finish.hpp"

namespace {

constexpr int CT = 32;       // state columns per workgroup (four waves of eight)

__device__ __forceinline__ float sigmoid_f(float x) { return 1.f / (1.f + expf(-x)); }
__device__ __forceinline__ float softplus_f(float x) { return fmaxf(x, 0.f) + log1pf(expf(-fabsf(x))); }
__device__ __forceinline__ float silu_f(float x) { return x * sigmoid_f(x); }

__device__ __forceinline__ int segment_of(const int* __restrict__ seg_start, int nseg, int t) {
  int lo = 0, hi = nseg;                 // largest s with seg_start[s] <= t
  while (hi - lo > 1) {
    const int mid = (lo + hi) >> 1;
    if (seg_start[mid] <= t) lo = mid; else hi = mid;
  }
  return lo;
}

// ---------------------------------------------------------------------------------------------------------------- prepare
// general form: grid (tokens, heads), one wave.  lw = W2 tanh(low) + w0 is the small second map of the decay (rank R).
template <typename T>
__global__ __launch_bounds__(64) void delta_prep_general_kernel(vlm_delta_prep_general_args p) {
  extern __shared__ float smem[];        // [R] tanh of the low-rank decay input
  const long t = blockIdx.x;
  const int h = blockIdx.y, lane = threadIdx.x, D = p.D, HD = p.H * p.D;
  const T* low = (const T*)p.low + t * p.ld_low;
  for (int j = lane; j < p.R; j += 64) smem[j] = tanhf(ld_f(low + j));
  __syncthreads();
  const T* kr = (const T*)p.k + t * p.ld + (long)h * D;
  float ss = 0.f;
  for (int i = lane; i < D; i += 64) {
    const float kv = ld_f(kr + i);
    ss += kv * kv;
  }
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) ss += __shfl_xor(ss, o);
  const float rn = 1.0f / sqrtf(ss + 1e-6f);
  const long o0 = t * HD + (long)h * D;
  for (int i = lane; i < D; i += 64) {
    const int c = h * D + i;
    const float kv = ld_f(kr + i), u = kv * rn;
    float lw = ld_f((const T*)p.w0 + c);
    const T* w2 = (const T*)p.w2 + (long)c * p.R;
    for (int j = 0; j < p.R; ++j) lw = fmaf(ld_f(w2 + j), smem[j], lw);
    const float a = sigmoid_f(ld_f((const T*)p.a + t * p.ld + c) + ld_f((const T*)p.a_bias + c));
    p.q[o0 + i] = ld_f((const T*)p.r + t * p.ld + c);
    p.kw[o0 + i] = kv;
    p.kr[o0 + i] = u;
    p.v[o0 + i] = ld_f((const T*)p.v_in + t * p.ld + c);
    p.w[o0 + i] = expf(-0.6065306597126334f * sigmoid_f(lw));      // exp(-1/2) = 0.60653...
    p.b[o0 + i] = a * u;
  }
}

// gated form: grid (tokens), 256 lanes.  Channels: q [KH * D] | k [KH * D] | v [H * Dv]; conv weights [channels][taps] with
// the current token's tap last; conv state fp32 [slot][taps - 1][channels] = the inputs at the taps - 1 positions before the
// segment (positions below 0 count as zeros whatever the slot holds).
template <typename T>
__global__ __launch_bounds__(256) void delta_prep_gated_kernel(vlm_delta_prep_gated_args p, int nseg) {
  extern __shared__ float y[];           // [channels] conv + silu
  const int t = blockIdx.x, tid = threadIdx.x;
  const int KD = p.KH * p.D, HV = p.H * p.Dv, Cn = 2 * KD + HV, taps = p.taps;
  const int seg = segment_of(p.seg_start, nseg, t);
  const int t0 = p.seg_start[seg], pos0 = p.seg_pos0[seg], pos = pos0 + (t - t0);
  const float* cs = p.conv_state + (long)p.seg_slot[seg] * (taps - 1) * Cn;
  for (int c = tid; c < Cn; c += 256) {
    const T* src;
    const T* cw;
    int cc;
    if (c < KD) { src = (const T*)p.q_in; cw = (const T*)p.q_conv; cc = c; }
    else if (c < 2 * KD) { src = (const T*)p.k_in; cw = (const T*)p.k_conv; cc = c - KD; }
    else { src = (const T*)p.v_in; cw = (const T*)p.v_conv; cc = c - 2 * KD; }
    float acc = 0.f;
    for (int j = 0; j < taps; ++j) {     // tap j sits taps - 1 - j tokens back
      const int pp = pos - (taps - 1) + j;
      float x = 0.f;
      if (pp >= pos0) x = ld_f(src + (long)(t0 + (pp - pos0)) * p.ld + cc);
      else if (pp >= 0) x = cs[(long)(taps - 1 - (pos0 - pp)) * Cn + c];
      acc = fmaf(ld_f(cw + (long)cc * taps + j), x, acc);
    }
    y[c] = silu_f(acc);
  }
  __syncthreads();
  const int wave = tid >> 6, lane = tid & 63;
  for (int hh = wave; hh < 2 * p.KH; hh += 4) {          // unit vectors: q heads then k heads
    const float* src = y + (long)hh * p.D;
    float ss = 0.f;
    for (int i = lane; i < p.D; i += 64) ss += src[i] * src[i];
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) ss += __shfl_xor(ss, o);
    const float rn = 1.0f / sqrtf(ss + 1e-6f);
    const bool isq = hh < p.KH;
    float* dst = (isq ? p.q : p.k) + (long)t * KD + (long)(isq ? hh : hh - p.KH) * p.D;
    const float sc = isq ? p.qscale : 1.f;
    for (int i = lane; i < p.D; i += 64) dst[i] = src[i] * rn * sc;
  }
  for (int c = tid; c < HV; c += 256) p.v[(long)t * HV + c] = y[2 * KD + c];
  for (int h = tid; h < p.H; h += 256) {
    p.beta[(long)t * p.H + h] = sigmoid_f(ld_f((const T*)p.b_in + (long)t * p.ld + h));
    const float dt = softplus_f(ld_f((const T*)p.a_in + (long)t * p.ld + h) + ld_f((const T*)p.dt_bias + h));
    p.g[(long)t * p.H + h] = expf(-expf(ld_f((const T*)p.A_log + h)) * dt);
  }
}

// the slot's last taps - 1 inputs after the segment: grid (segments), lanes over channels.  Entry j holds the input at
// position end - (taps - 1) + j; for a segment shorter than taps - 1 the older entries move down (entry j reads old entry
// j + n, ascending j: read before overwritten).
template <typename T>
__global__ __launch_bounds__(256) void delta_conv_state_kernel(vlm_delta_prep_gated_args p) {
  const int seg = blockIdx.x;
  const int KD = p.KH * p.D, HV = p.H * p.Dv, Cn = 2 * KD + HV, taps = p.taps;
  const int t0 = p.seg_start[seg], n = p.seg_start[seg + 1] - t0, pos0 = p.seg_pos0[seg];
  float* cs = p.conv_state + (long)p.seg_slot[seg] * (taps - 1) * Cn;
  for (int c = blockIdx.y * 256 + threadIdx.x; c < Cn; c += gridDim.y * 256) {
    const T* src;
    int cc;
    if (c < KD) { src = (const T*)p.q_in; cc = c; }
    else if (c < 2 * KD) { src = (const T*)p.k_in; cc = c - KD; }
    else { src = (const T*)p.v_in; cc = c - 2 * KD; }
    for (int j = 0; j < taps - 1; ++j) {
      const int pp = pos0 + n - (taps - 1) + j;
      float x = 0.f;
      if (pp >= pos0) x = ld_f(src + (long)(t0 + (pp - pos0)) * p.ld + cc);
      else if (pp >= 0) x = cs[(long)(j + n) * Cn + c];
      cs[(long)j * Cn + c] = x;
    }
  }
}

// ------------------------------------------------------------------------------------------------------------------- scan
// lane = (column c = lane >> 3 of the wave's 8, row group rg = lane & 7): rows [DR rg, DR rg + DR) of one state column in
// registers; the eight lanes of a column are half a DPP row, so S^T k and S^T q are DR fused multiply-adds per lane and three
// DPP exchanges - no barrier and no LDS traffic inside the token loop besides the broadcast reads of the token's vectors.
constexpr int RG = 8;        // lanes (row groups) per state column
constexpr int CW = 64 / RG;  // columns per wave
__device__ __forceinline__ float group_sum(float v) {
  v += vlm_dpp<0xB1, 0xf>(0.f, v);     // quad_perm [1,0,3,2]
  v += vlm_dpp<0x4E, 0xf>(0.f, v);     // quad_perm [2,3,0,1]
  v += vlm_dpp<0x141, 0xf>(0.f, v);    // row_half_mirror: the other quad of the eight lanes
  return v;
}

template <int DR, bool GENERAL>
__global__ __launch_bounds__(256) void delta_scan_kernel(vlm_delta_rule_args p, int TB) {
  extern __shared__ __align__(16) float smem[];
  constexpr int GP = DR + 4;              // a row group's pitch in LDS (the four groups' reads of one instruction spread over the banks)
  constexpr int DP = RG * GP, NV = GENERAL ? 5 : 2;
  const int seg = blockIdx.x, h = blockIdx.y, c0 = blockIdx.z * CT;
  const int D = p.D, Dv = p.Dv;
  const int tid = threadIdx.x, wave = tid >> 6, lane = tid & 63;
  const int rg = lane & (RG - 1), cl = wave * CW + lane / RG, col = c0 + cl, row0 = rg * DR;
  const int kh = h / (p.H / p.KH);
  float* ks = smem;                       // [TB][DP] write key
  float* qs = ks + TB * DP;               // [TB][DP] read-out key
  float* us = qs + TB * DP;               // [TB][DP] read key   (GENERAL; the gated form reads with the write key)
  float* ws = us + (GENERAL ? TB * DP : 0);      // [TB][DP] decay per key channel (GENERAL)
  float* bs = ws + (GENERAL ? TB * DP : 0);      // [TB][DP] removal row (GENERAL)
  float* vs = smem + NV * TB * DP;        // [TB][CT]
  float* sc = vs + TB * CT;               // [TB][2]: g, beta (gated)
  const int t_begin = p.seg_start[seg], t_end = p.seg_start[seg + 1];
  const int slot = p.seg_slot[seg], pos0 = p.seg_pos0[seg];
  float* S = p.state + ((long)slot * p.H + h) * (long)D * Dv;
  float s[DR];
#pragma unroll
  for (int r = 0; r < DR; ++r) {
    const int row = row0 + r;
    s[r] = (pos0 > 0 && row < D && col < Dv) ? S[(long)row * Dv + col] : 0.f;
  }
  for (int t0 = t_begin; t0 < t_end; t0 += TB) {
    const int nb = min(TB, t_end - t0);
    __syncthreads();                      // (the previous block's vectors are no longer read)
    for (int idx = tid; idx < nb * RG * DR; idx += 256) {
      const int t = idx / (RG * DR), i = idx % (RG * DR);
      const long off = (long)(t0 + t) * p.ldk + (long)kh * D + i;
      const int dst = t * DP + (i / DR) * GP + i % DR;
      const bool in = i < D;
      ks[dst] = in ? p.kw[off] : 0.f;
      qs[dst] = in ? p.q[off] : 0.f;
      if (GENERAL) {
        us[dst] = in ? p.kr[off] : 0.f;
        ws[dst] = in ? p.w[off] : 0.f;
        bs[dst] = in ? p.b[off] : 0.f;
      }
    }
    for (int idx = tid; idx < nb * CT; idx += 256) {
      const int t = idx / CT, c = c0 + idx % CT;
      vs[idx] = c < Dv ? p.v[(long)(t0 + t) * p.ldv + (long)h * Dv + c] : 0.f;
    }
    if (!GENERAL && tid < nb) {
      sc[tid * 2 + 0] = p.g[(long)(t0 + tid) * p.H + h];
      sc[tid * 2 + 1] = p.beta[(long)(t0 + tid) * p.H + h];
    }
    __syncthreads();
    for (int t = 0; t < nb; ++t) {
      const float4* kr = reinterpret_cast<const float4*>((GENERAL ? us : ks) + t * DP + rg * GP);
      float d0 = 0.f, d1 = 0.f, d2 = 0.f, d3 = 0.f;        // four chains, fixed order
      if (GENERAL) {
#pragma unroll
        for (int r = 0; r < DR / 4; ++r) {
          const float4 kk = kr[r];
          d0 = fmaf(s[4 * r + 0], kk.x, d0);
          d1 = fmaf(s[4 * r + 1], kk.y, d1);
          d2 = fmaf(s[4 * r + 2], kk.z, d2);
          d3 = fmaf(s[4 * r + 3], kk.w, d3);
        }
      } else {
        const float g = sc[t * 2];
#pragma unroll
        for (int r = 0; r < DR / 4; ++r) {
          const float4 kk = kr[r];
          s[4 * r + 0] *= g;
          s[4 * r + 1] *= g;
          s[4 * r + 2] *= g;
          s[4 * r + 3] *= g;
          d0 = fmaf(s[4 * r + 0], kk.x, d0);
          d1 = fmaf(s[4 * r + 1], kk.y, d1);
          d2 = fmaf(s[4 * r + 2], kk.z, d2);
          d3 = fmaf(s[4 * r + 3], kk.w, d3);
        }
      }
      const float d = group_sum((d0 + d1) + (d2 + d3));
      const float4* kwr = reinterpret_cast<const float4*>(ks + t * DP + rg * GP);
      const float4* qr = reinterpret_cast<const float4*>(qs + t * DP + rg * GP);
      const float vv = vs[t * CT + cl];
      float a0 = 0.f, a1 = 0.f, a2 = 0.f, a3 = 0.f;
      if (GENERAL) {
        const float4* wr = reinterpret_cast<const float4*>(ws + t * DP + rg * GP);
        const float4* br = reinterpret_cast<const float4*>(bs + t * DP + rg * GP);
#pragma unroll
        for (int r = 0; r < DR / 4; ++r) {
          const float4 kk = kwr[r], qq = qr[r], ww = wr[r], bb = br[r];
          s[4 * r + 0] = fmaf(kk.x, vv, fmaf(-bb.x, d, ww.x * s[4 * r + 0]));
          s[4 * r + 1] = fmaf(kk.y, vv, fmaf(-bb.y, d, ww.y * s[4 * r + 1]));
          s[4 * r + 2] = fmaf(kk.z, vv, fmaf(-bb.z, d, ww.z * s[4 * r + 2]));
          s[4 * r + 3] = fmaf(kk.w, vv, fmaf(-bb.w, d, ww.w * s[4 * r + 3]));
          a0 = fmaf(s[4 * r + 0], qq.x, a0);
          a1 = fmaf(s[4 * r + 1], qq.y, a1);
          a2 = fmaf(s[4 * r + 2], qq.z, a2);
          a3 = fmaf(s[4 * r + 3], qq.w, a3);
        }
      } else {
        const float u = sc[t * 2 + 1] * (vv - d);
#pragma unroll
        for (int r = 0; r < DR / 4; ++r) {
          const float4 kk = kwr[r], qq = qr[r];
          s[4 * r + 0] = fmaf(kk.x, u, s[4 * r + 0]);
          s[4 * r + 1] = fmaf(kk.y, u, s[4 * r + 1]);
          s[4 * r + 2] = fmaf(kk.z, u, s[4 * r + 2]);
          s[4 * r + 3] = fmaf(kk.w, u, s[4 * r + 3]);
          a0 = fmaf(s[4 * r + 0], qq.x, a0);
          a1 = fmaf(s[4 * r + 1], qq.y, a1);
          a2 = fmaf(s[4 * r + 2], qq.z, a2);
          a3 = fmaf(s[4 * r + 3], qq.w, a3);
        }
      }
      const float o = group_sum((a0 + a1) + (a2 + a3));
      if (rg == 0 && col < Dv) p.raw[((long)(t0 + t) * p.H + h) * Dv + col] = o;
    }
  }
#pragma unroll
  for (int r = 0; r < DR; ++r) {
    const int row = row0 + r;
    if (row < D && col < Dv) S[(long)row * Dv + col] = s[r];
  }
}

template <int DR, bool GENERAL>
int launch_scan(const vlm_delta_rule_args& a, int nseg, hipStream_t st) {
  constexpr int DP = RG * (DR + 4), NV = GENERAL ? 5 : 2;
  auto lds = [&](int tb) { return (size_t)tb * (NV * DP + CT + 2) * sizeof(float); };
  int TB = 16;
  while (TB > 1 && lds(TB) > 48 * 1024) TB >>= 1;
  if (lds(TB) > 48 * 1024) return VLM_ERR_SHAPE;
  dim3 grid(nseg, a.H, (a.Dv + CT - 1) / CT), block(256);
  hipLaunchKernelGGL((delta_scan_kernel<DR, GENERAL>), grid, block, lds(TB), st, a, TB);
  VLM_CHECK_LAUNCH();
  return VLM_OK;
}

template <bool GENERAL>
int run_scan(const vlm_delta_rule_args& a, int nseg, hipStream_t st) {
  if (a.D <= 32) return launch_scan<4, GENERAL>(a, nseg, st);
  if (a.D <= 64) return launch_scan<8, GENERAL>(a, nseg, st);
  if (a.D <= 128) return launch_scan<16, GENERAL>(a, nseg, st);
  if (a.D <= 256) return launch_scan<32, GENERAL>(a, nseg, st);
  if (a.D <= 512) return launch_scan<64, GENERAL>(a, nseg, st);
  if (a.D <= 1024) return launch_scan<128, GENERAL>(a, nseg, st);
  return VLM_ERR_SHAPE;
}

}  // namespace

extern "C" int vlm_delta_prep_general(const vlm_delta_prep_general_args* a, int ntok, int dtype, void* stream) {
  if (!a || ntok < 0) return VLM_ERR_ARG;
  if (!a->r || !a->k || !a->v_in || !a->a || !a->a_bias || !a->low || !a->w2 || !a->w0 || !a->q || !a->kw || !a->kr || !a->v || !a->w ||
      !a->b || a->H <= 0 || a->D <= 0 || a->R <= 0 || a->ld < (long)a->H * a->D || a->ld_low < a->R)
    return VLM_ERR_ARG;
  if (ntok == 0) return VLM_OK;
  if (a->H > 65535 || a->R > 8192) return VLM_ERR_SHAPE;
  hipStream_t st = (hipStream_t)stream;
  const size_t lds = (size_t)a->R * sizeof(float);
  if (dtype) hipLaunchKernelGGL(delta_prep_general_kernel<float>, dim3(ntok, a->H), dim3(64), lds, st, *a);
  else hipLaunchKernelGGL(delta_prep_general_kernel<bf16_t>, dim3(ntok, a->H), dim3(64), lds, st, *a);
  VLM_CHECK_LAUNCH();
  return VLM_OK;
}

extern "C" int vlm_delta_prep_gated(const vlm_delta_prep_gated_args* a, int nseg, int ntok, int dtype, void* stream) {
  if (!a || nseg < 0 || ntok < 0) return VLM_ERR_ARG;
  if (!a->q_in || !a->k_in || !a->v_in || !a->q_conv || !a->k_conv || !a->v_conv || !a->b_in || !a->a_in || !a->A_log || !a->dt_bias ||
      !a->q || !a->k || !a->v || !a->beta || !a->g || !a->seg_start || !a->seg_slot || !a->seg_pos0 || a->H <= 0 || a->KH <= 0 ||
      a->H % a->KH || a->D <= 0 || a->Dv <= 0 || a->taps < 1 || (a->taps > 1 && !a->conv_state))
    return VLM_ERR_ARG;
  if (nseg == 0 || ntok == 0) return VLM_OK;
  const long Cn = 2L * a->KH * a->D + (long)a->H * a->Dv;
  if (Cn * sizeof(float) > 48 * 1024) return VLM_ERR_SHAPE;
  hipStream_t st = (hipStream_t)stream;
  const size_t lds = (size_t)Cn * sizeof(float);
  const unsigned cy = (unsigned)((Cn + 255) / 256 < 64 ? (Cn + 255) / 256 : 64);
  if (dtype) {
    hipLaunchKernelGGL(delta_prep_gated_kernel<float>, dim3(ntok), dim3(256), lds, st, *a, nseg);
    VLM_CHECK_LAUNCH();
    if (a->taps > 1) hipLaunchKernelGGL(delta_conv_state_kernel<float>, dim3(nseg, cy), dim3(256), 0, st, *a);
  } else {
    hipLaunchKernelGGL(delta_prep_gated_kernel<bf16_t>, dim3(ntok), dim3(256), lds, st, *a, nseg);
    VLM_CHECK_LAUNCH();
    if (a->taps > 1) hipLaunchKernelGGL(delta_conv_state_kernel<bf16_t>, dim3(nseg, cy), dim3(256), 0, st, *a);
  }
  VLM_CHECK_LAUNCH();
  return VLM_OK;
}

extern "C" int vlm_delta_rule(const vlm_delta_rule_args* a, int nseg, int ntok, int dtype, void* stream) {
  if (!a || nseg < 0 || ntok < 0) return VLM_ERR_ARG;
  if (!a->q || !a->kw || !a->v || !a->state || !a->raw || !a->gate || !a->out || !a->seg_start || !a->seg_slot || !a->seg_pos0)
    return VLM_ERR_ARG;
  if (a->H <= 0 || a->KH <= 0 || a->H % a->KH || a->D <= 0 || a->Dv <= 0) return VLM_ERR_ARG;
  if (a->mode == 1 ? (!a->kr || !a->w || !a->b) : (a->mode != 0 || !a->beta || !a->g)) return VLM_ERR_ARG;
  if (a->ldk < (long)a->KH * a->D || a->ldv < (long)a->H * a->Dv || a->ldg < (long)a->H * a->Dv || a->ldo < (long)a->H * a->Dv)
    return VLM_ERR_ARG;
  if (nseg == 0 || ntok == 0) return VLM_OK;
  if (nseg > 65535 * 16 || a->H > 65535) return VLM_ERR_SHAPE;
  hipStream_t st = (hipStream_t)stream;
  const int rc = a->mode == 1 ? run_scan<true>(*a, nseg, st) : run_scan<false>(*a, nseg, st);
  if (rc != VLM_OK) return rc;
  if (dtype)
    hipLaunchKernelGGL((recurrence_finish_kernel<float, false>), dim3(ntok, a->H), dim3(64), 0, st, a->raw, a->H, a->Dv,
                       (const float*)nullptr, a->eps, (const float*)a->gate, a->ldg, (const float*)a->normw, a->gate_act,
                       (float*)a->out, a->ldo);
  else
    hipLaunchKernelGGL((recurrence_finish_kernel<bf16_t, false>), dim3(ntok, a->H), dim3(64), 0, st, a->raw, a->H, a->Dv,
                       (const float*)nullptr, a->eps, (const bf16_t*)a->gate, a->ldg, (const bf16_t*)a->normw, a->gate_act,
                       (bf16_t*)a->out, a->ldo);
  VLM_CHECK_LAUNCH();
  return VLM_OK;
}
