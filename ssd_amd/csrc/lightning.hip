// Linear attention with a per-head scalar decay over a recurrent fp32 state ("lightning" mixers):
//     S_t = decay_h * S_(t-1) + k_t v_t^T        (S: [D][Dv] per sequence and head, zero before position 0)
//     o_t = S_t^T q_t
// q, k, v = silu of the projection rows.  The state of a live sequence sits in a slot of a per-layer-run pool
// state[slots][H][D][Dv] (fp32); a forward reads the slot unless the rows it brings start at position 0, walks its rows in order and
// writes the slot back, so a prompt may arrive in portions of any size and decoding is the one-row case of the same kernel.
//  * ssd_lightning_scan       proj rows fp32 [T][ld] holding [q | k | v | ...] -> o fp32 [T][H*Dv], state updated in place
//  * ssd_lightning_gate_norm  out = w * o / sqrt(mean(o^2) + eps) * sigmoid(g) over the concatenated heads, as GEMM-input rows
// The arithmetic of a row is the same whatever the portion: per state element one multiply-add chain in token order, the output a sum
// over d in a fixed order -- whole prompt, portions and token-by-token decoding give bit-identical rows.
#include "common.h"

namespace {

template <typename T> __device__ __forceinline__ float ldf(const T* p);
template <> __device__ __forceinline__ float ldf<float>(const float* p) { return *p; }
template <> __device__ __forceinline__ float ldf<bf16_t>(const bf16_t* p) { return bf2f(*p); }
template <typename T> __device__ __forceinline__ void stf(T* p, float v);
template <> __device__ __forceinline__ void stf<float>(float* p, float v) { *p = v; }
template <> __device__ __forceinline__ void stf<bf16_t>(bf16_t* p, float v) { *p = (bf16_t)f2bf(v); }

__device__ __forceinline__ float sigmoidf_(float z) { return 1.0f / (1.0f + expf(-z)); }
__device__ __forceinline__ float siluf_(float z) { return z * sigmoidf_(z); }

// One workgroup per (sequence, head).  Threads form NG groups of EP lanes (EP = power of two >= min(Dv, 256)): lane e of group g owns
// the state elements (d, e) with d = g, g + NG, ...; the groups' partial outputs meet in LDS and are summed in group order.
__global__ void __launch_bounds__(256)
lightning_scan_kernel(const float* __restrict__ proj, long ld, int q_off, int k_off, int v_off, const float* __restrict__ decay,
                      const int64_t* __restrict__ positions, const int32_t* __restrict__ cu_q, int q_per_seq,
                      const int32_t* __restrict__ state_slots, float* __restrict__ state, float* __restrict__ out, int H, int D, int Dv,
                      int EP) {
  extern __shared__ float lds[];
  float* S = lds;                         // [D][Dv]
  float* sq = S + (size_t)D * Dv;         // [D]
  float* sk = sq + D;                     // [D]
  float* sv = sk + D;                     // [Dv]
  float* po = sv + Dv;                    // [NG][Dv]
  const int b = blockIdx.x, h = blockIdx.y, tid = threadIdx.x;
  const int row0 = cu_q ? cu_q[b] : b * q_per_seq;
  const int row1 = cu_q ? cu_q[b + 1] : (b + 1) * q_per_seq;
  if (row1 <= row0) return;
  const int slot = state_slots[b];
  float* sp = state + ((size_t)slot * H + h) * D * Dv;
  const bool fresh = positions[row0] == 0;
  for (int i = tid; i < D * Dv; i += 256) S[i] = fresh ? 0.f : sp[i];
  const float dc = decay[h];
  const int NG = 256 / EP, g = tid / EP, el = tid % EP;
  for (int r = row0; r < row1; ++r) {
    const float* pr = proj + (size_t)r * ld;
    __syncthreads();                      // the previous row's readers of sq / sk / sv / po are done; S is loaded
    for (int i = tid; i < D; i += 256) {
      sq[i] = siluf_(pr[q_off + h * D + i]);
      sk[i] = siluf_(pr[k_off + h * D + i]);
    }
    for (int i = tid; i < Dv; i += 256) sv[i] = siluf_(pr[v_off + h * Dv + i]);
    __syncthreads();
    for (int e = el; e < Dv; e += EP) {
      const float ve = sv[e];
      float o = 0.f;
      for (int d = g; d < D; d += NG) {
        const float s = fmaf(dc, S[d * Dv + e], sk[d] * ve);
        S[d * Dv + e] = s;
        o = fmaf(s, sq[d], o);
      }
      po[g * Dv + e] = o;
    }
    __syncthreads();
    for (int e = tid; e < Dv; e += 256) {
      float o = 0.f;
      for (int gg = 0; gg < NG; ++gg) o += po[gg * Dv + e];
      out[(size_t)r * H * Dv + h * Dv + e] = o;
    }
  }
  __syncthreads();
  for (int i = tid; i < D * Dv; i += 256) sp[i] = S[i];
}

template <typename T>
__global__ void __launch_bounds__(256)
lightning_gate_norm_kernel(const float* __restrict__ o, const float* __restrict__ proj, long ld, int g_off, const T* __restrict__ w,
                           float eps, T* __restrict__ out, int N) {
  __shared__ float red[4];
  const size_t t = blockIdx.x;
  const float* orow = o + t * N;
  float ss = 0.f;
  for (int c = threadIdx.x; c < N; c += 256) { const float v = orow[c]; ss += v * v; }
  ss = wave_sum(ss);
  if ((threadIdx.x & 63) == 0) red[threadIdx.x >> 6] = ss;
  __syncthreads();
  ss = (red[0] + red[1]) + (red[2] + red[3]);
  const float r = 1.0f / sqrtf(ss / (float)N + eps);
  const float* gr = proj + t * ld + g_off;
  for (int c = threadIdx.x; c < N; c += 256) stf<T>(out + t * N + c, orow[c] * r * ldf<T>(w + c) * sigmoidf_(gr[c]));
}

}  // namespace

#define LAUNCH_OK() (hipGetLastError() == hipSuccess ? SSD_OK : SSD_ERR_LAUNCH)

extern "C" int ssd_lightning_scan(const void* proj_rows, long ld, int q_off, int k_off, int v_off, const float* decay,
                                  const int64_t* positions, const int32_t* cu_q, int q_per_seq, const int32_t* state_slots,
                                  void* state, void* out_rows, int B, int H, int D, int Dv, void* stream) {
  if (!proj_rows || !decay || !positions || !state_slots || !state || !out_rows) return SSD_ERR_ARG;
  if (B <= 0 || H <= 0 || D <= 0 || Dv <= 0 || (!cu_q && q_per_seq <= 0)) return SSD_ERR_SHAPE;
  int EP = 1;
  while (EP < Dv && EP < 256) EP <<= 1;
  const size_t bytes = ((size_t)D * Dv + 2 * (size_t)D + Dv + (size_t)(256 / EP) * Dv) * sizeof(float);
  if (bytes > 160 * 1024) return SSD_ERR_SHAPE;
  if (bytes > 64 * 1024 &&
      hipFuncSetAttribute((const void*)lightning_scan_kernel, hipFuncAttributeMaxDynamicSharedMemorySize, (int)bytes) != hipSuccess)
    return SSD_ERR_LAUNCH;
  hipLaunchKernelGGL(lightning_scan_kernel, dim3(B, H), dim3(256), bytes, (hipStream_t)stream, (const float*)proj_rows, ld, q_off, k_off,
                     v_off, decay, positions, cu_q, q_per_seq, state_slots, (float*)state, (float*)out_rows, H, D, Dv, EP);
  return LAUNCH_OK();
}

extern "C" int ssd_lightning_gate_norm(const void* o_rows, const void* proj_rows, long ld, int g_off, const void* weight, float eps,
                                       void* out_rows, int T, int N, int f32, void* stream) {
  if (!o_rows || !proj_rows || !weight || !out_rows) return SSD_ERR_ARG;
  if (T <= 0 || N <= 0) return SSD_ERR_SHAPE;
  if (f32)
    hipLaunchKernelGGL(lightning_gate_norm_kernel<float>, dim3(T), dim3(256), 0, (hipStream_t)stream, (const float*)o_rows,
                       (const float*)proj_rows, ld, g_off, (const float*)weight, eps, (float*)out_rows, N);
  else
    hipLaunchKernelGGL(lightning_gate_norm_kernel<bf16_t>, dim3(T), dim3(256), 0, (hipStream_t)stream, (const float*)o_rows,
                       (const float*)proj_rows, ld, g_off, (const bf16_t*)weight, eps, (bf16_t*)out_rows, N);
  return LAUNCH_OK();
}
