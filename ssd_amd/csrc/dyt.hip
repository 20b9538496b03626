// Kernels of decoders whose layers are PARALLEL (mixer and feed-forward read the same normalised row and their outputs are summed
// into an fp32 residual) and whose norm is Dynamic Tanh, y = tanh(alpha * x) * w + b, which needs no statistic of the row:
//  * ssd_dyt_embed       x = dyt(table[id]) as fp32 residual rows (+ a second fp32 copy, + an element-type copy with a row stride of its
//                        own: the right half of the [x | x0] rows that a loop's input projection reads)
//  * ssd_dyt_rows        out = dyt(x (+ a vector added to every row first, written back)) as GEMM-input rows, optional row gather
//  * ssd_parallel_tail   x += y_mix + ff, ff = a dense fp32 row, or the routed mix  sum_j weights[j] * ydn[inv[t*top+j]]
//                        (+ sigmoid(gate logit) * shared row), or nothing; then the next layer's dyt(x) as GEMM-input rows, or the
//                        element-type copy of x into the left half of the [x | x0] rows
//  * ssd_glu_rows        out = act(a) * b for fp32 rows [a | b] (gate and up projections stacked), act = silu or tanh-form gelu
// Everything is elementwise in fp32 (grid = rows x column blocks); a row's result depends on that row alone.  `f32` selects the element type of weights and of
// GEMM-input rows: 0 = bf16, 1 = fp32.  alpha is read from device memory (a one-element tensor of the checkpoint, kept as fp32).
#include "common.h"

namespace {

template <typename T> __device__ __forceinline__ float ldf(const T* p);
template <> __device__ __forceinline__ float ldf<float>(const float* p) { return *p; }
template <> __device__ __forceinline__ float ldf<bf16_t>(const bf16_t* p) { return bf2f(*p); }
template <typename T> __device__ __forceinline__ void stf(T* p, float v);
template <> __device__ __forceinline__ void stf<float>(float* p, float v) { *p = v; }
template <> __device__ __forceinline__ void stf<bf16_t>(bf16_t* p, float v) { *p = (bf16_t)f2bf(v); }

__device__ __forceinline__ float sigmoidf_(float z) { return 1.0f / (1.0f + expf(-z)); }

template <typename T>
__global__ void __launch_bounds__(256)
dyt_embed_kernel(const int64_t* __restrict__ ids, const T* __restrict__ table, const float* __restrict__ alpha, const T* __restrict__ w,
                 const T* __restrict__ b, float* __restrict__ x, float* __restrict__ x0, T* __restrict__ cat, long ld_cat, int W,
                 long vocab) {
  const int t = blockIdx.x;
  const long id = ids[t];
  const bool ok = id >= 0 && id < vocab;
  const T* src = table + (size_t)(ok ? id : 0) * W;
  const float a = *alpha;
  for (int c = blockIdx.y * 256 + threadIdx.x; c < W; c += 256 * gridDim.y) {
    const float e = ok ? ldf<T>(src + c) : 0.f;
    const float v = tanhf(a * e) * ldf<T>(w + c) + ldf<T>(b + c);
    x[(size_t)t * W + c] = v;
    if (x0) x0[(size_t)t * W + c] = v;
    if (cat) stf<T>(cat + (size_t)t * ld_cat + c, v);
  }
}

template <typename T>
__global__ void __launch_bounds__(256)
dyt_rows_kernel(float* __restrict__ x, const T* __restrict__ add_vec, const float* __restrict__ alpha, const T* __restrict__ w,
                const T* __restrict__ b, T* __restrict__ out, const int32_t* __restrict__ gather, int W) {
  const int ro = blockIdx.x;
  const int ri = gather ? gather[ro] : ro;
  float* xr = x + (size_t)ri * W;
  const float a = *alpha;
  for (int c = blockIdx.y * 256 + threadIdx.x; c < W; c += 256 * gridDim.y) {
    float v = xr[c];
    if (add_vec) { v += ldf<T>(add_vec + c); xr[c] = v; }
    stf<T>(out + (size_t)ro * W + c, tanhf(a * v) * ldf<T>(w + c) + ldf<T>(b + c));
  }
}

template <typename T>
__global__ void __launch_bounds__(256)
parallel_tail_kernel(float* __restrict__ x, const float* __restrict__ y_mix, const float* __restrict__ y_ff,
                     const float* __restrict__ ydn, const int32_t* __restrict__ inv, const float* __restrict__ wt, int top,
                     const float* __restrict__ shared, const float* __restrict__ sgate, long ld_sgate,
                     const float* __restrict__ alpha, const T* __restrict__ w, const T* __restrict__ b, T* __restrict__ next_out,
                     T* __restrict__ cat, long ld_cat, int W) {
  const int t = blockIdx.x;
  float* xr = x + (size_t)t * W;
  const float sg = (shared && sgate) ? sigmoidf_(sgate[(size_t)t * ld_sgate]) : 1.0f;
  const float a = next_out ? *alpha : 0.f;
  for (int c = blockIdx.y * 256 + threadIdx.x; c < W; c += 256 * gridDim.y) {
    float ff = 0.f;
    if (y_ff) {
      ff = y_ff[(size_t)t * W + c];
    } else if (ydn) {
      for (int j = 0; j < top; ++j) ff = fmaf(wt[(size_t)t * top + j], ydn[(size_t)inv[(size_t)t * top + j] * W + c], ff);
      if (shared) ff += sg * shared[(size_t)t * W + c];
    }
    const float v = xr[c] + (y_mix[(size_t)t * W + c] + ff);
    xr[c] = v;
    if (next_out) stf<T>(next_out + (size_t)t * W + c, tanhf(a * v) * ldf<T>(w + c) + ldf<T>(b + c));
    if (cat) stf<T>(cat + (size_t)t * ld_cat + c, v);
  }
}

template <typename T>
__global__ void __launch_bounds__(256)
glu_rows_kernel(const float* __restrict__ ab, T* __restrict__ out, int F, int act) {
  const size_t r = blockIdx.x;
  const float* a = ab + r * 2 * F;
  for (int c = blockIdx.y * 256 + threadIdx.x; c < F; c += 256 * gridDim.y) {
    const float z = a[c], u = a[F + c];
    float g;
    if (act == 0) g = z * sigmoidf_(z);
    else g = 0.5f * z * (1.0f + tanhf(0.7978845608028654f * (z + 0.044715f * z * z * z)));
    stf<T>(out + r * F + c, g * u);
  }
}

}  // namespace

#define LAUNCH_OK() (hipGetLastError() == hipSuccess ? SSD_OK : SSD_ERR_LAUNCH)

// rows x column blocks: everything here is elementwise, so a few rows (decoding) still spread over the chip
static inline dim3 row_grid(int rows, int cols) {
  int cb = (cols + 255) / 256;
  if (rows >= 1024) cb = 1;
  else if (cb > 64) cb = 64;
  return dim3(rows, cb);
}

extern "C" int ssd_dyt_embed(const int64_t* ids, const void* table, const float* alpha, const void* weight, const void* bias, void* x,
                             void* x0, void* cat, long ld_cat, int T, int W, long vocab, int f32, void* stream) {
  if (!ids || !table || !alpha || !weight || !bias || !x) return SSD_ERR_ARG;
  if (T <= 0 || W <= 0 || vocab <= 0 || (cat && ld_cat < W)) return SSD_ERR_SHAPE;
  if (f32)
    hipLaunchKernelGGL(dyt_embed_kernel<float>, row_grid(T, W), dim3(256), 0, (hipStream_t)stream, ids, (const float*)table, alpha,
                       (const float*)weight, (const float*)bias, (float*)x, (float*)x0, (float*)cat, ld_cat, W, vocab);
  else
    hipLaunchKernelGGL(dyt_embed_kernel<bf16_t>, row_grid(T, W), dim3(256), 0, (hipStream_t)stream, ids, (const bf16_t*)table, alpha,
                       (const bf16_t*)weight, (const bf16_t*)bias, (float*)x, (float*)x0, (bf16_t*)cat, ld_cat, W, vocab);
  return LAUNCH_OK();
}

extern "C" int ssd_dyt_rows(void* x, const void* add_vec, const float* alpha, const void* weight, const void* bias, void* out_rows,
                            const int32_t* gather, int T, int W, int f32, void* stream) {
  if (!x || !alpha || !weight || !bias || !out_rows) return SSD_ERR_ARG;
  if (T <= 0 || W <= 0 || (gather && add_vec)) return SSD_ERR_SHAPE;
  if (f32)
    hipLaunchKernelGGL(dyt_rows_kernel<float>, row_grid(T, W), dim3(256), 0, (hipStream_t)stream, (float*)x, (const float*)add_vec, alpha,
                       (const float*)weight, (const float*)bias, (float*)out_rows, gather, W);
  else
    hipLaunchKernelGGL(dyt_rows_kernel<bf16_t>, row_grid(T, W), dim3(256), 0, (hipStream_t)stream, (float*)x, (const bf16_t*)add_vec, alpha,
                       (const bf16_t*)weight, (const bf16_t*)bias, (bf16_t*)out_rows, gather, W);
  return LAUNCH_OK();
}

extern "C" int ssd_parallel_tail(void* x, const void* y_mix, const void* y_ff, const void* ydn_rows, const int32_t* inv,
                                 const float* weights, int top, const void* shared_rows, const float* shared_gate, long ld_shared_gate,
                                 const float* next_alpha, const void* next_weight, const void* next_bias, void* next_out, void* cat,
                                 long ld_cat, int T, int W, int f32, void* stream) {
  if (!x || !y_mix) return SSD_ERR_ARG;
  if (ydn_rows && !y_ff && (!inv || !weights)) return SSD_ERR_ARG;
  if (next_out && (!next_alpha || !next_weight || !next_bias)) return SSD_ERR_ARG;
  if (T <= 0 || W <= 0 || (ydn_rows && !y_ff && top <= 0) || (cat && ld_cat < W)) return SSD_ERR_SHAPE;
  if (f32)
    hipLaunchKernelGGL(parallel_tail_kernel<float>, row_grid(T, W), dim3(256), 0, (hipStream_t)stream, (float*)x, (const float*)y_mix,
                       (const float*)y_ff, (const float*)ydn_rows, inv, weights, top, (const float*)shared_rows, shared_gate,
                       ld_shared_gate, next_alpha, (const float*)next_weight, (const float*)next_bias, (float*)next_out, (float*)cat,
                       ld_cat, W);
  else
    hipLaunchKernelGGL(parallel_tail_kernel<bf16_t>, row_grid(T, W), dim3(256), 0, (hipStream_t)stream, (float*)x, (const float*)y_mix,
                       (const float*)y_ff, (const float*)ydn_rows, inv, weights, top, (const float*)shared_rows, shared_gate,
                       ld_shared_gate, next_alpha, (const bf16_t*)next_weight, (const bf16_t*)next_bias, (bf16_t*)next_out,
                       (bf16_t*)cat, ld_cat, W);
  return LAUNCH_OK();
}

extern "C" int ssd_glu_rows(const void* ab_rows, void* out_rows, int rows, int F, int act, int f32, void* stream) {
  if (!ab_rows || !out_rows) return SSD_ERR_ARG;
  if (rows <= 0 || F <= 0 || act < 0 || act > 1) return SSD_ERR_SHAPE;
  if (f32)
    hipLaunchKernelGGL(glu_rows_kernel<float>, row_grid(rows, F), dim3(256), 0, (hipStream_t)stream, (const float*)ab_rows, (float*)out_rows,
                       F, act);
  else
    hipLaunchKernelGGL(glu_rows_kernel<bf16_t>, row_grid(rows, F), dim3(256), 0, (hipStream_t)stream, (const float*)ab_rows,
                       (bf16_t*)out_rows, F, act);
  return LAUNCH_OK();
}
