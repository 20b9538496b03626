// Routed feed-forward (mixture of experts) around the grouped GEMM of gemm_rows.hip:
//   ssd_moe_route    z = W_r h in fp32; the `top` largest logits per token (lowest index wins a tie) and the softmax over them
//   ssd_moe_plan     counting sort of the T * top (token, slot) pairs by expert: offsets[E+1], perm (sorted row -> pair), inv (pair -> sorted row)
//   ssd_moe_combine  out[t] = sum_j weight[t][j] * y[inv[t * top + j]] (+ shared[t]) in slot order, fp32
// Between plan and combine the caller runs the experts as two grouped GEMMs over the sorted rows (up with the activation as epilogue,
// then down).  A pair's row is computed by itself, so a token's result does not depend on the other tokens of the batch or on the order
// the sort happened to give its expert's rows.
#include "common.h"

namespace {

template <typename T> __device__ __forceinline__ float ldf(const T* p);
template <> __device__ __forceinline__ float ldf<float>(const float* p) { return *p; }
template <> __device__ __forceinline__ float ldf<bf16_t>(const bf16_t* p) { return bf2f(*p); }

constexpr int MOE_MAX_E = 4096, MOE_MAX_TOP = 32;

template <typename T>
__global__ void __launch_bounds__(256)
moe_route_kernel(const T* __restrict__ h, const T* __restrict__ wr, int32_t* __restrict__ idx, float* __restrict__ wt, int W, int E,
                 int top) {
  extern __shared__ float z[];      // [E]
  const int t = blockIdx.x, wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
  const T* hr = h + (size_t)t * W;
  for (int e = wave; e < E; e += 4) {
    const T* wrow = wr + (size_t)e * W;
    float s = 0.f;
    for (int k = lane; k < W; k += 64) s = fmaf(ldf<T>(hr + k), ldf<T>(wrow + k), s);
    s = wave_sum(s);
    if (lane == 0) z[e] = s;
  }
  __syncthreads();
  if (threadIdx.x == 0) {
    float val[MOE_MAX_TOP];
    for (int j = 0; j < top; ++j) {
      float best = -INFINITY; int bi = 0;
      for (int e = 0; e < E; ++e) {
        const float v = z[e];
        if (v > best) { best = v; bi = e; }
      }
      val[j] = best;
      idx[(size_t)t * top + j] = bi;
      z[bi] = -INFINITY;
    }
    float den = 0.f;
    const float vmax = val[0];
    for (int j = 0; j < top; ++j) { val[j] = expf(val[j] - vmax); den += val[j]; }
    for (int j = 0; j < top; ++j) wt[(size_t)t * top + j] = val[j] / den;
  }
}

__global__ void __launch_bounds__(1024)
moe_plan_kernel(const int32_t* __restrict__ idx, int n, int E, int32_t* __restrict__ offsets, int32_t* __restrict__ perm,
                int32_t* __restrict__ inv) {
  extern __shared__ int cnt[];      // [E] counts, then cursors
  for (int e = threadIdx.x; e < E; e += blockDim.x) cnt[e] = 0;
  __syncthreads();
  for (int i = threadIdx.x; i < n; i += blockDim.x) atomicAdd(&cnt[idx[i]], 1);
  __syncthreads();
  if (threadIdx.x == 0) {
    int run = 0;
    for (int e = 0; e < E; ++e) { const int c = cnt[e]; offsets[e] = run; cnt[e] = run; run += c; }
    offsets[E] = run;
  }
  __syncthreads();
  for (int i = threadIdx.x; i < n; i += blockDim.x) {
    const int pos = atomicAdd(&cnt[idx[i]], 1);
    perm[pos] = i;
    inv[i] = pos;
  }
}

__global__ void __launch_bounds__(256)
moe_combine_kernel(const float* __restrict__ y, const int32_t* __restrict__ inv, const float* __restrict__ wt,
                   const float* __restrict__ shared, float* __restrict__ out, int top, int W) {
  const int t = blockIdx.x;
  for (int c = threadIdx.x; c < W; c += 256) {
    float s = 0.f;
    for (int j = 0; j < top; ++j) s = fmaf(wt[(size_t)t * top + j], y[(size_t)inv[(size_t)t * top + j] * W + c], s);
    if (shared) s += shared[(size_t)t * W + c];
    out[(size_t)t * W + c] = s;
  }
}

}  // namespace

#define LAUNCH_OK() (hipGetLastError() == hipSuccess ? SSD_OK : SSD_ERR_LAUNCH)

extern "C" int ssd_moe_route(const void* h_rows, const void* w_router, int32_t* idx, float* weights, int T, int W, int E, int top,
                             int f32, void* stream) {
  if (!h_rows || !w_router || !idx || !weights) return SSD_ERR_ARG;
  if (T <= 0 || W <= 0 || E <= 0 || E > MOE_MAX_E || top <= 0 || top > E || top > MOE_MAX_TOP) return SSD_ERR_SHAPE;
  if (f32)
    hipLaunchKernelGGL(moe_route_kernel<float>, dim3(T), dim3(256), E * sizeof(float), (hipStream_t)stream, (const float*)h_rows,
                       (const float*)w_router, idx, weights, W, E, top);
  else
    hipLaunchKernelGGL(moe_route_kernel<bf16_t>, dim3(T), dim3(256), E * sizeof(float), (hipStream_t)stream, (const bf16_t*)h_rows,
                       (const bf16_t*)w_router, idx, weights, W, E, top);
  return LAUNCH_OK();
}

extern "C" int ssd_moe_plan(const int32_t* idx, int T, int top, int E, int32_t* offsets, int32_t* perm, int32_t* inv, void* stream) {
  if (!idx || !offsets || !perm || !inv) return SSD_ERR_ARG;
  if (T <= 0 || top <= 0 || E <= 0 || E > MOE_MAX_E) return SSD_ERR_SHAPE;
  hipLaunchKernelGGL(moe_plan_kernel, dim3(1), dim3(1024), E * sizeof(int), (hipStream_t)stream, idx, T * top, E, offsets, perm, inv);
  return LAUNCH_OK();
}

extern "C" int ssd_moe_combine(const void* y_rows, const int32_t* inv, const float* weights, const void* shared_rows, void* out_rows,
                               int T, int top, int W, void* stream) {
  if (!y_rows || !inv || !weights || !out_rows) return SSD_ERR_ARG;
  if (T <= 0 || top <= 0 || W <= 0) return SSD_ERR_SHAPE;
  hipLaunchKernelGGL(moe_combine_kernel, dim3(T), dim3(256), 0, (hipStream_t)stream, (const float*)y_rows, inv, weights,
                     (const float*)shared_rows, (float*)out_rows, top, W);
  return LAUNCH_OK();
}
