// Latent attention over a paged cache, with a sliding window.  Queries and keys / values pass through low-rank latents:
//     c_q = rms(W_dq h) w_dq,  q = W_uq c_q   (per head [D unrotated | R rotated])
//     [c' | k_r] = W_dkv h,   c = rms(c') w_dkv (the latent, Cr wide),   k_r (R wide): ONE rotated key part for all heads
//     key_h = [W_uk,h c | rope(k_r)],  value_h = W_uv,h c
// Only [c | rope(k_r)] is cached per token (Cr + R numbers for every head together).  The attention runs in the latent space:
//     score(t, j, h) = scale * ( <W_uk,h^T q_unrot(t,h), c_j> + <rope(q_rot(t,h)), rope(k_r,j)> )
//     o_lat(t, h)    = gate(t,h) * sum_j softmax_j(score) c_j          over  0 <= p_t - p_j < window
// and the caller's per-head GEMMs map q_unrot -> W_uk^T q_unrot before and o_lat -> W_uv o_lat after: every head reads the same
// cached rows, which is what makes decoding cheap.
// Rotation: the first `rot_dims` of the R rotated entries turn, entry i pairing with i + rot_dims / 2, by angle p * f_i (fp32) with
// cos and sin scaled by `mag`; f and mag come from the host (they carry the YaRN frequency blend).
//  * ssd_latent_store  fp32 projection rows [dq | dkv | gate logits] -> c_q rows, the cache row of every token, sigmoid gates
//  * ssd_latent_attn   scalar fp32 form for any sizes and both element types: a wave owns a (token, head) row, a lane a key for the
//                      scores and latent columns for the weighted sum; keys in steps of 64 from the window's first key, so a row's
//                      arithmetic depends on its position alone (not on the portion or the batch it arrives in)
#include "common.h"

namespace {

template <typename T> __device__ __forceinline__ float ldf(const T* p);
template <> __device__ __forceinline__ float ldf<float>(const float* p) { return *p; }
template <> __device__ __forceinline__ float ldf<bf16_t>(const bf16_t* p) { return bf2f(*p); }
template <typename T> __device__ __forceinline__ void stf(T* p, float v);
template <> __device__ __forceinline__ void stf<float>(float* p, float v) { *p = v; }
template <> __device__ __forceinline__ void stf<bf16_t>(bf16_t* p, float v) { *p = (bf16_t)f2bf(v); }

__device__ __forceinline__ float sigmoidf_(float z) { return 1.0f / (1.0f + expf(-z)); }

// LDS written by some lanes of a wave and read by others: order the accesses (the hardware serves one wave's LDS operations in order)
__device__ __forceinline__ void wave_sync() {
  __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
  __builtin_amdgcn_wave_barrier();
  __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
}

__device__ __forceinline__ float block_sum_256(float v, float* red) {
  v = wave_sum(v);
  __syncthreads();
  if ((threadIdx.x & 63) == 0) red[threadIdx.x >> 6] = v;
  __syncthreads();
  return (red[0] + red[1]) + (red[2] + red[3]);
}

// entry i (< R) of a rotated part x at position pos
template <typename F>
__device__ __forceinline__ float rope_entry(F x, int i, int R, int rot_dims, float pos, const float* __restrict__ freqs, float mag) {
  const int half = rot_dims >> 1;
  if (i >= rot_dims) return x(i);
  const int f = i < half ? i : i - half;
  const float ang = pos * freqs[f];
  const float c = cosf(ang) * mag, s = sinf(ang) * mag;
  return i < half ? x(i) * c - x(i + half) * s : x(i) * c + x(i - half) * s;
}

template <typename T>
__global__ void __launch_bounds__(256)
latent_store_kernel(const float* __restrict__ proj, long ld, int Qr, int Cr, int R, int H, const T* __restrict__ wq,
                    const T* __restrict__ wkv, float eps, const int64_t* __restrict__ positions, const float* __restrict__ freqs,
                    float mag, int rot_dims, const int32_t* __restrict__ slots, T* __restrict__ cq_out, T* __restrict__ cache,
                    float* __restrict__ gate_out) {
  __shared__ float red[4];
  const size_t t = blockIdx.x;
  const float* pr = proj + t * ld;
  const float* dq = pr;
  const float* dkv = pr + Qr;
  float sq = 0.f, sc = 0.f;
  for (int i = threadIdx.x; i < Qr; i += 256) sq += dq[i] * dq[i];
  for (int i = threadIdx.x; i < Cr; i += 256) sc += dkv[i] * dkv[i];
  sq = block_sum_256(sq, red);
  sc = block_sum_256(sc, red);
  const float rq = 1.0f / sqrtf(sq / (float)Qr + eps), rc = 1.0f / sqrtf(sc / (float)Cr + eps);
  for (int i = threadIdx.x; i < Qr; i += 256) stf<T>(cq_out + t * Qr + i, dq[i] * rq * ldf<T>(wq + i));
  for (int i = threadIdx.x; i < H; i += 256) gate_out[t * H + i] = sigmoidf_(pr[Qr + Cr + R + i]);
  const int slot = slots[t];
  if (slot < 0) return;
  T* row = cache + (size_t)slot * (Cr + R);
  for (int i = threadIdx.x; i < Cr; i += 256) stf<T>(row + i, dkv[i] * rc * ldf<T>(wkv + i));
  const float pos = (float)positions[t];
  const float* kr = dkv + Cr;
  for (int i = threadIdx.x; i < R; i += 256)
    stf<T>(row + Cr + i, rope_entry([&](int j) { return kr[j]; }, i, R, rot_dims, pos, freqs, mag));
}

constexpr int LAT_MAXC = 16;       // latent columns per lane: Cr <= 64 * LAT_MAXC

template <typename T>
__global__ void __launch_bounds__(256)
latent_attn_kernel(const float* __restrict__ q_abs, const T* __restrict__ q_rows, const T* __restrict__ cache,
                   const float* __restrict__ gate, const int32_t* __restrict__ block_tables, int max_blocks,
                   const int64_t* __restrict__ positions, const int32_t* __restrict__ cu_q, int q_per_seq, int B, int H, int D, int R,
                   int Cr, int block_size, int window, float scale, const float* __restrict__ freqs, float mag, int rot_dims,
                   T* __restrict__ out) {
  extern __shared__ float lds[];
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
  const int t = blockIdx.x, h = blockIdx.y * 4 + wave;
  const int KW = Cr + R;
  float* sq = lds + (size_t)wave * (KW + 128);      // [KW] the row's query in the latent space | rotated part
  float* sp = sq + KW;                              // [64] softmax weights of the current key step
  int* sj = reinterpret_cast<int*>(sp + 64);        // [64] their cache rows
  if (h >= H) return;                               // (whole waves; no block-wide barrier below)
  int b;
  if (cu_q) {
    int lo = 0, hi = B;                             // cu_q[lo] <= t < cu_q[hi]
    while (hi - lo > 1) { const int mid = (lo + hi) >> 1; if (cu_q[mid] <= t) lo = mid; else hi = mid; }
    b = lo;
  } else {
    b = t / q_per_seq;
  }
  const long p = positions[t];
  const float pos = (float)p;
  const long first = (window > 0 && p - window + 1 > 0) ? p - window + 1 : 0;
  for (int i = lane; i < Cr; i += 64) sq[i] = q_abs[((size_t)t * H + h) * Cr + i];
  const T* qr = q_rows + ((size_t)t * H + h) * (D + R) + D;
  for (int i = lane; i < R; i += 64)
    sq[Cr + i] = rope_entry([&](int j) { return ldf<T>(qr + j); }, i, R, rot_dims, pos, freqs, mag);
  wave_sync();
  float m = -INFINITY, den = 0.f;
  float acc[LAT_MAXC];
#pragma unroll
  for (int c = 0; c < LAT_MAXC; ++c) acc[c] = 0.f;
  const int32_t* bt = block_tables + (size_t)b * max_blocks;
  for (long j0 = first; j0 <= p; j0 += 64) {
    const long j = j0 + lane;
    const bool valid = j <= p;
    int row = 0;
    float s = -INFINITY;
    if (valid) {
      row = bt[j / block_size] * block_size + (int)(j % block_size);
      const T* kp = cache + (size_t)row * KW;
      float d = 0.f;
      for (int i = 0; i < KW; ++i) d = fmaf(sq[i], ldf<T>(kp + i), d);
      s = d * scale;
    }
    const float mn = fmaxf(m, wave_max(s));
    const float pj = valid ? expf(s - mn) : 0.f;
    const float resc = m == -INFINITY ? 0.f : expf(m - mn);
    den = den * resc + wave_sum(pj);
    m = mn;
    wave_sync();
    sp[lane] = pj;
    sj[lane] = row;
    wave_sync();
    const int cnt = (int)((p - j0 + 1) < 64 ? (p - j0 + 1) : 64);
#pragma unroll
    for (int c = 0; c < LAT_MAXC; ++c) {
      const int col = lane + 64 * c;
      if (col < Cr) {
        float a = acc[c] * resc;
        for (int kk = 0; kk < cnt; ++kk) a = fmaf(sp[kk], ldf<T>(cache + (size_t)sj[kk] * KW + col), a);
        acc[c] = a;
      }
    }
  }
  const float g = gate[(size_t)t * H + h] / den;
#pragma unroll
  for (int c = 0; c < LAT_MAXC; ++c) {
    const int col = lane + 64 * c;
    if (col < Cr) stf<T>(out + ((size_t)t * H + h) * Cr + col, acc[c] * g);
  }
}

}  // namespace

#define LAUNCH_OK() (hipGetLastError() == hipSuccess ? SSD_OK : SSD_ERR_LAUNCH)

extern "C" int ssd_latent_store(const void* proj_rows, long ld, int q_rank, int kv_rank, int rot, int H, const void* q_norm_w,
                                const void* kv_norm_w, float eps, const int64_t* positions, const float* freqs, float mag,
                                int rot_dims, const int32_t* slots, void* cq_out, void* cache, void* gate_out, int T, int f32,
                                void* stream) {
  if (!proj_rows || !q_norm_w || !kv_norm_w || !positions || !freqs || !slots || !cq_out || !cache || !gate_out) return SSD_ERR_ARG;
  if (T <= 0 || q_rank <= 0 || kv_rank <= 0 || rot < 0 || H <= 0 || rot_dims < 0 || rot_dims > rot || (rot_dims & 1) ||
      ld < (long)q_rank + kv_rank + rot + H)
    return SSD_ERR_SHAPE;
  if (f32)
    hipLaunchKernelGGL(latent_store_kernel<float>, dim3(T), dim3(256), 0, (hipStream_t)stream, (const float*)proj_rows, ld, q_rank,
                       kv_rank, rot, H, (const float*)q_norm_w, (const float*)kv_norm_w, eps, positions, freqs, mag, rot_dims, slots,
                       (float*)cq_out, (float*)cache, (float*)gate_out);
  else
    hipLaunchKernelGGL(latent_store_kernel<bf16_t>, dim3(T), dim3(256), 0, (hipStream_t)stream, (const float*)proj_rows, ld, q_rank,
                       kv_rank, rot, H, (const bf16_t*)q_norm_w, (const bf16_t*)kv_norm_w, eps, positions, freqs, mag, rot_dims, slots,
                       (bf16_t*)cq_out, (bf16_t*)cache, (float*)gate_out);
  return LAUNCH_OK();
}

extern "C" int ssd_latent_attn(const void* q_abs, const void* q_rows, const void* cache, const void* gate, const int32_t* block_tables,
                               int max_blocks, const int64_t* positions, const int32_t* cu_q, int q_per_seq, int B, int T, int H, int D,
                               int rot, int kv_rank, int block_size, int window, float scale, const float* freqs, float mag,
                               int rot_dims, void* out_rows, int f32, void* stream) {
  if (!q_abs || !q_rows || !cache || !gate || !block_tables || !positions || !freqs || !out_rows) return SSD_ERR_ARG;
  if (B <= 0 || T <= 0 || H <= 0 || D <= 0 || rot < 0 || kv_rank <= 0 || kv_rank > 64 * LAT_MAXC || block_size <= 0 || max_blocks <= 0 ||
      rot_dims < 0 || rot_dims > rot || (rot_dims & 1) || (!cu_q && q_per_seq <= 0))
    return SSD_ERR_SHAPE;
  const size_t bytes = (size_t)4 * (kv_rank + rot + 128) * sizeof(float);
  const dim3 grid(T, (H + 3) / 4);
  if (f32)
    hipLaunchKernelGGL(latent_attn_kernel<float>, grid, dim3(256), bytes, (hipStream_t)stream, (const float*)q_abs, (const float*)q_rows,
                       (const float*)cache, (const float*)gate, block_tables, max_blocks, positions, cu_q, q_per_seq, B, H, D, rot,
                       kv_rank, block_size, window, scale, freqs, mag, rot_dims, (float*)out_rows);
  else
    hipLaunchKernelGGL(latent_attn_kernel<bf16_t>, grid, dim3(256), bytes, (hipStream_t)stream, (const float*)q_abs,
                       (const bf16_t*)q_rows, (const bf16_t*)cache, (const float*)gate, block_tables, max_blocks, positions, cu_q,
                       q_per_seq, B, H, D, rot, kv_rank, block_size, window, scale, freqs, mag, rot_dims, (bf16_t*)out_rows);
  return LAUNCH_OK();
}
