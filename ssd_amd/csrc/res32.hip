// Kernels of decoders that keep the residual stream in fp32 and normalise on BOTH sides of a sublayer ("sandwich" layers):
//     x <- x + w_post * rms(f(w_pre * rms(x)))
//  * ssd_embed_res32        token rows of the embedding table as fp32 residual rows (+ a second copy for designs that re-inject it)
//  * ssd_rmsnorm_res32      y = w * x / sqrt(mean(x^2) + eps) from the fp32 residual to GEMM-input rows; optionally x += add first
//                           (the re-injected embedding before a repeated pass) and a row gather (logit rows)
//  * ssd_rmsnorm_add_res32  x += w * rms(y) for the fp32 sublayer output y
//  * ssd_sandwich_tail      (routed mix ->) post-norm + residual sum -> (re-injection ->) the next sublayer's pre-norm, one launch
//  * ssd_rows_f32_to_bf16   fp32 rows -> bf16 rows with their own row stride, padding columns = -inf (fp32 logits for the bf16 sampling kernels)
// All reductions are fp32, one workgroup of 256 threads per row, a fixed summation order per row (independent of the batch).
// `f32` selects the element type of weights and of GEMM-input rows: 0 = bf16, 1 = fp32.
#include "common.h"

namespace {

template <typename T> __device__ __forceinline__ float ldf(const T* p);
template <> __device__ __forceinline__ float ldf<float>(const float* p) { return *p; }
template <> __device__ __forceinline__ float ldf<bf16_t>(const bf16_t* p) { return bf2f(*p); }
template <typename T> __device__ __forceinline__ void stf(T* p, float v);
template <> __device__ __forceinline__ void stf<float>(float* p, float v) { *p = v; }
template <> __device__ __forceinline__ void stf<bf16_t>(bf16_t* p, float v) { *p = (bf16_t)f2bf(v); }

__device__ __forceinline__ float block_sum_256(float v, float* red) {
  v = wave_sum(v);
  const int wave = threadIdx.x >> 6;
  __syncthreads();
  if ((threadIdx.x & 63) == 0) red[wave] = v;
  __syncthreads();
  return (red[0] + red[1]) + (red[2] + red[3]);
}
// the same for NT threads (a multiple of 256): waves summed in groups of four, the groups in order
template <int NT>
__device__ __forceinline__ float block_sum(float v, float* red) {
  v = wave_sum(v);
  const int wave = threadIdx.x >> 6;
  __syncthreads();
  if ((threadIdx.x & 63) == 0) red[wave] = v;
  __syncthreads();
  float s = 0.f;
#pragma unroll
  for (int q = 0; q < NT / 256; ++q) s += (red[4 * q] + red[4 * q + 1]) + (red[4 * q + 2] + red[4 * q + 3]);
  return s;
}

template <typename T>
__global__ void __launch_bounds__(256)
embed_res32_kernel(const int64_t* __restrict__ ids, const T* __restrict__ table, float* __restrict__ x, float* __restrict__ x0, int W,
                   long vocab) {
  const int t = blockIdx.x;
  long id = ids[t];
  const bool ok = id >= 0 && id < vocab;
  const T* src = table + (size_t)(ok ? id : 0) * W;
  for (int c = threadIdx.x; c < W; c += 256) {
    const float v = ok ? ldf<T>(src + c) : 0.f;
    x[(size_t)t * W + c] = v;
    if (x0) x0[(size_t)t * W + c] = v;
  }
}

template <typename T>
__global__ void __launch_bounds__(256)
rmsnorm_res32_kernel(float* __restrict__ x, const float* __restrict__ add, const T* __restrict__ w, float eps, T* __restrict__ out,
                     const int32_t* __restrict__ gather, int W) {
  __shared__ float red[4];
  const int ro = blockIdx.x;
  const int ri = gather ? gather[ro] : ro;
  float* xr = x + (size_t)ri * W;
  float ss = 0.f;
  for (int c = threadIdx.x; c < W; c += 256) {
    float v = xr[c];
    if (add) { v += add[(size_t)ri * W + c]; xr[c] = v; }
    ss += v * v;
  }
  ss = block_sum_256(ss, red);
  const float r = 1.0f / sqrtf(ss / (float)W + eps);
  for (int c = threadIdx.x; c < W; c += 256) stf<T>(out + (size_t)ro * W + c, xr[c] * r * ldf<T>(w + c));
}

template <typename T>
__global__ void __launch_bounds__(256)
rmsnorm_add_res32_kernel(const float* __restrict__ y, const T* __restrict__ w, float eps, float* __restrict__ x, int W) {
  __shared__ float red[4];
  const float* yr = y + (size_t)blockIdx.x * W;
  float* xr = x + (size_t)blockIdx.x * W;
  float ss = 0.f;
  for (int c = threadIdx.x; c < W; c += 256) { const float v = yr[c]; ss += v * v; }
  ss = block_sum_256(ss, red);
  const float r = 1.0f / sqrtf(ss / (float)W + eps);
  for (int c = threadIdx.x; c < W; c += 256) xr[c] += yr[c] * r * ldf<T>(w + c);
}

// The whole tail of a sandwich sublayer for one token row per workgroup:
//   y = the sublayer's fp32 output row, or the routed feed-forward's mix  sum_j weights[j] * ydn[inv[t * top + j]] (+ shared[t])
//   x += w_post * rms(y);   then, if a next sublayer follows:  x += next_add (the re-injected embedding before a repeated pass),
//   next_out = w_next * rms(x)  -- the input rows of the next sublayer's first GEMM.
// Three launches (mix, post-norm + residual sum, next pre-norm) in one; the same arithmetic in the same order as the separate kernels.
template <typename T, int NT>
__global__ void __launch_bounds__(NT)
sandwich_tail_kernel(const float* __restrict__ y, const float* __restrict__ ydn, const int32_t* __restrict__ inv,
                     const float* __restrict__ wt, const float* __restrict__ shared, int top, float* __restrict__ ytmp,
                     const T* __restrict__ w_post, float eps, float* __restrict__ x, const float* __restrict__ next_add,
                     const T* __restrict__ w_next, T* __restrict__ next_out, int W) {
  __shared__ float red[NT / 64];
  const int t = blockIdx.x;
  float* xr = x + (size_t)t * W;
  const float* yr = y ? y + (size_t)t * W : ytmp + (size_t)t * W;
  float ss = 0.f;
  if (y) {
    for (int c = threadIdx.x; c < W; c += NT) { const float v = yr[c]; ss += v * v; }
  } else {
    float* yw = ytmp + (size_t)t * W;
    for (int c = threadIdx.x; c < W; c += NT) {
      float v = 0.f;
      for (int j = 0; j < top; ++j) v = fmaf(wt[(size_t)t * top + j], ydn[(size_t)inv[(size_t)t * top + j] * W + c], v);
      if (shared) v += shared[(size_t)t * W + c];
      yw[c] = v;                    // read back below by the thread that wrote it
      ss += v * v;
    }
  }
  ss = block_sum<NT>(ss, red);
  const float r = 1.0f / sqrtf(ss / (float)W + eps);
  float s2 = 0.f;
  for (int c = threadIdx.x; c < W; c += NT) {
    float v = xr[c] + yr[c] * r * ldf<T>(w_post + c);
    if (next_add) v += next_add[(size_t)t * W + c];
    xr[c] = v;
    s2 += v * v;
  }
  if (!w_next) return;
  s2 = block_sum<NT>(s2, red);
  const float r2 = 1.0f / sqrtf(s2 / (float)W + eps);
  for (int c = threadIdx.x; c < W; c += NT) stf<T>(next_out + (size_t)t * W + c, xr[c] * r2 * ldf<T>(w_next + c));
}

__global__ void rows_f32_to_bf16_kernel(const float* __restrict__ src, bf16_t* __restrict__ dst, int cols, long ld_src, long ld_dst) {
  const long r = blockIdx.x;
  for (int c = blockIdx.y * blockDim.x + threadIdx.x; c < ld_dst; c += gridDim.y * blockDim.x) dst[r * ld_dst + c] = c < cols ? (bf16_t)f2bf(src[r * ld_src + c]) : (bf16_t)0xff80u;
}

}  // namespace

#define LAUNCH_OK() (hipGetLastError() == hipSuccess ? SSD_OK : SSD_ERR_LAUNCH)

extern "C" int ssd_embed_res32(const int64_t* ids, const void* table, void* x_out, void* x0_out, int T, int W, long vocab, int f32,
                               void* stream) {
  if (!ids || !table || !x_out) return SSD_ERR_ARG;
  if (T <= 0 || W <= 0 || vocab <= 0) return SSD_ERR_SHAPE;
  if (f32)
    hipLaunchKernelGGL(embed_res32_kernel<float>, dim3(T), dim3(256), 0, (hipStream_t)stream, ids, (const float*)table, (float*)x_out,
                       (float*)x0_out, W, vocab);
  else
    hipLaunchKernelGGL(embed_res32_kernel<bf16_t>, dim3(T), dim3(256), 0, (hipStream_t)stream, ids, (const bf16_t*)table, (float*)x_out,
                       (float*)x0_out, W, vocab);
  return LAUNCH_OK();
}

extern "C" int ssd_rmsnorm_res32(void* x, const void* add, const void* weight, float eps, void* out_rows, const int32_t* gather,
                                 int T, int W, int f32, void* stream) {
  if (!x || !weight || !out_rows) return SSD_ERR_ARG;
  if (T <= 0 || W <= 0) return SSD_ERR_SHAPE;
  if (add && gather) return SSD_ERR_ARG;          // the in-place add is a whole-batch step
  if (f32)
    hipLaunchKernelGGL(rmsnorm_res32_kernel<float>, dim3(T), dim3(256), 0, (hipStream_t)stream, (float*)x, (const float*)add,
                       (const float*)weight, eps, (float*)out_rows, gather, W);
  else
    hipLaunchKernelGGL(rmsnorm_res32_kernel<bf16_t>, dim3(T), dim3(256), 0, (hipStream_t)stream, (float*)x, (const float*)add,
                       (const bf16_t*)weight, eps, (bf16_t*)out_rows, gather, W);
  return LAUNCH_OK();
}

extern "C" int ssd_rmsnorm_add_res32(const void* y, const void* weight, float eps, void* x, int T, int W, int f32, void* stream) {
  if (!y || !weight || !x) return SSD_ERR_ARG;
  if (T <= 0 || W <= 0) return SSD_ERR_SHAPE;
  if (f32)
    hipLaunchKernelGGL(rmsnorm_add_res32_kernel<float>, dim3(T), dim3(256), 0, (hipStream_t)stream, (const float*)y,
                       (const float*)weight, eps, (float*)x, W);
  else
    hipLaunchKernelGGL(rmsnorm_add_res32_kernel<bf16_t>, dim3(T), dim3(256), 0, (hipStream_t)stream, (const float*)y,
                       (const bf16_t*)weight, eps, (float*)x, W);
  return LAUNCH_OK();
}

extern "C" int ssd_rows_f32_to_bf16(const void* src, void* dst, int rows, int cols, long ld_src, long ld_dst, void* stream) {
  if (!src || !dst) return SSD_ERR_ARG;
  if (rows <= 0 || cols <= 0 || ld_src < cols || ld_dst < cols) return SSD_ERR_SHAPE;
  const int chunks = (int)((ld_dst + 2047) / 2048);
  hipLaunchKernelGGL(rows_f32_to_bf16_kernel, dim3(rows, chunks), dim3(256), 0, (hipStream_t)stream, (const float*)src, (bf16_t*)dst, cols,
                     ld_src, ld_dst);
  return LAUNCH_OK();
}

extern "C" int ssd_sandwich_tail(const void* y_rows, const void* ydn_rows, const int32_t* inv, const float* weights,
                                 const void* shared_rows, int top, void* y_scratch, const void* post_weight, float eps, void* x,
                                 const void* next_add, const void* next_weight, void* next_out, int T, int W, int f32, void* stream) {
  if (!post_weight || !x) return SSD_ERR_ARG;
  if (!y_rows && (!ydn_rows || !inv || !weights || !y_scratch || top <= 0)) return SSD_ERR_ARG;
  if ((next_weight == nullptr) != (next_out == nullptr) || (next_add && !next_weight)) return SSD_ERR_ARG;
  if (T <= 0 || W <= 0) return SSD_ERR_SHAPE;
  if (T <= 64 && W >= 2048) {          // few rows: a row is a latency chain, so give it 1024 threads
    if (f32)
      hipLaunchKernelGGL((sandwich_tail_kernel<float, 1024>), dim3(T), dim3(1024), 0, (hipStream_t)stream, (const float*)y_rows,
                         (const float*)ydn_rows, inv, weights, (const float*)shared_rows, top, (float*)y_scratch,
                         (const float*)post_weight, eps, (float*)x, (const float*)next_add, (const float*)next_weight, (float*)next_out, W);
    else
      hipLaunchKernelGGL((sandwich_tail_kernel<bf16_t, 1024>), dim3(T), dim3(1024), 0, (hipStream_t)stream, (const float*)y_rows,
                         (const float*)ydn_rows, inv, weights, (const float*)shared_rows, top, (float*)y_scratch,
                         (const bf16_t*)post_weight, eps, (float*)x, (const float*)next_add, (const bf16_t*)next_weight,
                         (bf16_t*)next_out, W);
    return LAUNCH_OK();
  }
  if (f32)
    hipLaunchKernelGGL((sandwich_tail_kernel<float, 256>), dim3(T), dim3(256), 0, (hipStream_t)stream, (const float*)y_rows,
                       (const float*)ydn_rows, inv, weights, (const float*)shared_rows, top, (float*)y_scratch,
                       (const float*)post_weight, eps, (float*)x, (const float*)next_add, (const float*)next_weight, (float*)next_out, W);
  else
    hipLaunchKernelGGL((sandwich_tail_kernel<bf16_t, 256>), dim3(T), dim3(256), 0, (hipStream_t)stream, (const float*)y_rows,
                       (const float*)ydn_rows, inv, weights, (const float*)shared_rows, top, (float*)y_scratch,
                       (const bf16_t*)post_weight, eps, (float*)x, (const float*)next_add, (const bf16_t*)next_weight,
                       (bf16_t*)next_out, W);
  return LAUNCH_OK();
}
