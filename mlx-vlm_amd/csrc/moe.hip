// Mixture-of-experts routing and the expert activation, for experts whose up / down projections are stacked into ONE matrix
// each (rows of W_up: expert 0's ff rows, expert 1's, ..., then the shared expert's; columns of W_down in the same order).
// A token's routed output is then   down( gate_e(t) * act(up_e h) for every expert e )   with gate_e(t) = 0 for the experts
// the token did not choose: one up GEMM, this activation pass, one down GEMM - the sum over experts is the k loop of the down
// projection, and the experts a token skipped contribute exact zeros.
//
//   vlm_moe_route        logits fp32 [T][E] -> the `top` largest per token (lowest index wins a tie), softmax over the chosen
//                        logits only; dense gate table fp32 [T][E] (0 where not chosen) + the chosen (index, weight) lists
//   vlm_moe_relu2_gate   out[t][c] = relu(up[t][c])^2 * gate[t][c / ff]   for c < E * ff,   relu(up[t][c])^2 for the
//                        `shared` columns behind them (an expert every token uses); T-typed in and out, fp32 inside
#include "common.hpp"
#include "../../include/vlm_hip.h"

namespace {

template <typename T> __device__ __forceinline__ float ld_f(const T* p);
template <> __device__ __forceinline__ float ld_f<float>(const float* p) { return *p; }
template <> __device__ __forceinline__ float ld_f<bf16_t>(const bf16_t* p) { return bf2f(*p); }
template <typename T> __device__ __forceinline__ void st_f(T* p, float v);
template <> __device__ __forceinline__ void st_f<float>(float* p, float v) { *p = v; }
template <> __device__ __forceinline__ void st_f<bf16_t>(bf16_t* p, float v) { *p = f2bf(v); }

// one wave per token; lane l owns experts l, l + 64, ... (a bit per owned expert records what earlier rounds took)
__global__ __launch_bounds__(256) void moe_route_kernel(const float* __restrict__ z, int T, int E, int top, float* __restrict__ gate,
                                                        int* __restrict__ idx, float* __restrict__ wgt) {
  const int t = blockIdx.x * 4 + (threadIdx.x >> 6), lane = threadIdx.x & 63;
  if (t >= T) return;
  const float* zr = z + (long)t * E;
  for (int e = lane; e < E; e += 64) gate[(long)t * E + e] = 0.f;
  unsigned taken = 0u;
  float zmax = 0.f, denom = 0.f;
  float my_val = 0.f;                    // lane j < top keeps the j-th chosen logit
  int my_idx = -1;
  for (int j = 0; j < top; ++j) {
    float best = -INFINITY;
    int bi = 0x7fffffff;
    for (int e = lane, i = 0; e < E; e += 64, ++i) {
      const float v = zr[e];
      if (!((taken >> i) & 1u) && (v > best || (v == best && e < bi))) {
        best = v;
        bi = e;
      }
    }
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) {
      const float ob = __shfl_xor(best, o);
      const int oi = __shfl_xor(bi, o);
      if (ob > best || (ob == best && oi < bi)) {
        best = ob;
        bi = oi;
      }
    }
    if (bi == 0x7fffffff) break;         // fewer comparable candidates than `top` (NaN logits): what was found is kept
    if (lane == (bi & 63)) taken |= 1u << (bi >> 6);
    if (j == 0) zmax = best;
    if (lane == j) {
      my_val = best;
      my_idx = bi;
    }
    denom += expf(best - zmax);
  }
  const float w = my_idx >= 0 ? expf(my_val - zmax) / denom : 0.f;
  if (lane < top) {
    idx[(long)t * top + lane] = my_idx < 0 ? 0 : my_idx;
    wgt[(long)t * top + lane] = w;
  }
  for (int j = 0; j < top; ++j) {        // the owner of an expert writes its gate (it also wrote the zero)
    const int ej = __shfl(my_idx, j);
    const float wj = __shfl(w, j);
    if (ej >= 0 && lane == (ej & 63)) gate[(long)t * E + ej] = wj;
  }
}

template <typename T>
__global__ __launch_bounds__(256) void moe_relu2_gate_kernel(const T* __restrict__ up, long ldu, const float* __restrict__ gate, int E,
                                                             int ff, int shared, T* __restrict__ out, long ldo, int rows) {
  const int cols = E * ff + shared;
  const long i = (long)blockIdx.x * 256 + threadIdx.x;
  if (i >= (long)rows * cols) return;
  const long t = i / cols;
  const int c = (int)(i % cols);
  const float u = fmaxf(ld_f(up + t * ldu + c), 0.f);
  const float g = c < E * ff ? gate[t * E + c / ff] : 1.f;
  st_f(out + t * ldo + c, u * u * g);
}

}  // namespace

extern "C" int vlm_moe_route(const void* logits, int T, int E, int top, void* gate, void* idx, void* wgt, void* stream) {
  if (!logits || !gate || !idx || !wgt || T < 0 || E <= 0 || top <= 0 || top > E) return VLM_ERR_ARG;
  if (top > 64 || E > 2048) return VLM_ERR_SHAPE;
  if (T == 0) return VLM_OK;
  hipLaunchKernelGGL(moe_route_kernel, dim3((T + 3) / 4), dim3(256), 0, (hipStream_t)stream, (const float*)logits, T, E, top,
                     (float*)gate, (int*)idx, (float*)wgt);
  VLM_CHECK_LAUNCH();
  return VLM_OK;
}

extern "C" int vlm_moe_relu2_gate(const void* up, long ldu, const void* gate, int E, int ff, int shared, void* out, long ldo, int rows,
                                  int dtype, void* stream) {
  if (!up || !out || rows < 0 || E < 0 || ff < 0 || shared < 0 || (E > 0 && !gate)) return VLM_ERR_ARG;
  const long cols = (long)E * ff + shared;
  if (cols <= 0 || ldu < cols || ldo < cols) return VLM_ERR_ARG;
  if (rows == 0) return VLM_OK;
  const unsigned nb = (unsigned)((rows * cols + 255) / 256);
  hipStream_t st = (hipStream_t)stream;
  if (dtype)
    hipLaunchKernelGGL(moe_relu2_gate_kernel<float>, dim3(nb), dim3(256), 0, st, (const float*)up, ldu, (const float*)gate, E, ff,
                       shared, (float*)out, ldo, rows);
  else
    hipLaunchKernelGGL(moe_relu2_gate_kernel<bf16_t>, dim3(nb), dim3(256), 0, st, (const bf16_t*)up, ldu, (const float*)gate, E, ff,
                       shared, (bf16_t*)out, ldo, rows);
  VLM_CHECK_LAUNCH();
  return VLM_OK;
}
