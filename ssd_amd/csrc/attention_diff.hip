// Differential attention over the paged KV cache: every query head owns TWO softmax maps over the same values,
//     o = rms_noweight(a_1 - lambda * a_2) * out_scale * gate,      a_m = softmax(scale * q_m . k_m) v,
// with per-(head, map) RMS norm of q and k (weight shared by all heads and maps), no rotation, and a per-head sigmoid gate.
// Query / key size D and value size Dv are independent and arbitrary (any D, Dv <= 512); element type bf16 or fp32 (`f32`).
//   cache layout per layer: K [blocks][G][block_size][2 * D] (map 1 | map 2, normalised), V [blocks][G][block_size][Dv].
//   * ssd_diffattn_store   from the fused projection's fp32 rows [q | k | v | gate logits]: norm q -> q_out, norm k -> K cache at
//                          slots[t], v -> V cache, sigmoid(gate logits) -> gate_out fp32 [T][H].  slot -1: nothing is stored.
//   * ssd_diffattn_paged   one workgroup per (token, head): its 4 waves take 64-key tiles round-robin; inside a tile a lane owns
//                          a KEY for the scores (fp32 dot products, online softmax per map in fp32) and a VALUE COLUMN for the
//                          weighted sums (weights broadcast through LDS, fp32 accumulation); the waves' partial (max, sum,
//                          accumulator) triples merge in LDS in wave order, then the combination, the head norm, the scale
//                          and the gate are applied and the row is written as GEMM input.
//                          Scores, weights, sums and norms are fp32 whatever the element type.
//   A token's position and sequence come from positions[] / cu_q[] (varlen batches: prompt portions beside single tokens) or from
//   q_per_seq (fixed rows per sequence); it sees keys 0 .. position of ITS sequence, through that sequence's block table.
#include "common.h"

namespace {

template <typename T> __device__ __forceinline__ float ldf(const T* p);
template <> __device__ __forceinline__ float ldf<float>(const float* p) { return *p; }
template <> __device__ __forceinline__ float ldf<bf16_t>(const bf16_t* p) { return bf2f(*p); }
template <typename T> __device__ __forceinline__ void stf(T* p, float v);
template <> __device__ __forceinline__ void stf<float>(float* p, float v) { *p = v; }
template <> __device__ __forceinline__ void stf<bf16_t>(bf16_t* p, float v) { *p = (bf16_t)f2bf(v); }

constexpr int DA_MAXV = 8;      // value columns per lane: Dv <= 512

template <typename T>
__global__ void __launch_bounds__(256)
diffattn_store_kernel(const float* __restrict__ qkvg, const T* __restrict__ qw, const T* __restrict__ kw, float eps,
                      const int32_t* __restrict__ slots, T* __restrict__ q_out, float* __restrict__ gate_out, T* __restrict__ kc,
                      T* __restrict__ vc, int H, int G, int D, int Dv, int bs) {
  const int t = blockIdx.x, wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
  const int Nq = H * 2 * D, Nk = G * 2 * D, Nv = G * Dv;
  const float* row = qkvg + (size_t)t * (Nq + Nk + Nv + H);
  const int slot = slots[t];
  const long blk = slot >= 0 ? slot / bs : 0;
  const int off = slot >= 0 ? slot % bs : 0;
  // q units 0 .. 2H-1, then k units 0 .. 2G-1: one wave per (head, map) vector of D values
  for (int u = wave; u < 2 * H + 2 * G; u += 4) {
    const bool isq = u < 2 * H;
    const float* src = isq ? row + (size_t)u * D : row + Nq + (size_t)(u - 2 * H) * D;
    float ss = 0.f;
    for (int d = lane; d < D; d += 64) { const float v = src[d]; ss += v * v; }
    ss = wave_sum(ss);
    const float r = 1.0f / sqrtf(ss / (float)D + eps);
    if (isq) {
      T* dst = q_out + (size_t)t * Nq + (size_t)u * D;
      for (int d = lane; d < D; d += 64) stf<T>(dst + d, src[d] * r * ldf<T>(qw + d));
    } else if (slot >= 0) {
      const int ku = u - 2 * H, g = ku >> 1, mp = ku & 1;
      T* dst = kc + (((size_t)blk * G + g) * bs + off) * (2 * D) + (size_t)mp * D;
      for (int d = lane; d < D; d += 64) stf<T>(dst + d, src[d] * r * ldf<T>(kw + d));
    }
  }
  if (slot >= 0) {
    for (int c = threadIdx.x; c < Nv; c += 256) {
      const int g = c / Dv, d = c % Dv;
      stf<T>(vc + (((size_t)blk * G + g) * bs + off) * Dv + d, row[Nq + Nk + c]);
    }
  }
  for (int h = threadIdx.x; h < H; h += 256) gate_out[(size_t)t * H + h] = 1.0f / (1.0f + expf(-row[Nq + Nk + Nv + h]));
}

template <typename T>
__global__ void __launch_bounds__(256)
diffattn_paged_kernel(const T* __restrict__ q, const T* __restrict__ kc, const T* __restrict__ vc, const float* __restrict__ gate,
                      const int32_t* __restrict__ bt, int max_blocks, const int64_t* __restrict__ positions,
                      const int32_t* __restrict__ cu_q, int q_per_seq, int B, int H, int G, int D, int Dv, int bs, float scale,
                      float lambda, float out_scale, float eps, T* __restrict__ out) {
  extern __shared__ float smem[];
  const int t = blockIdx.x, h = blockIdx.y, wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
  const int g = h / (H / G);
  // ---- LDS carve-up ----
  float* sq = smem;                          // [2 * D] the two query vectors
  float* sp = sq + 2 * D;                    // [4 waves][2 maps][64] weights of the current tile
  long* srow = reinterpret_cast<long*>(sp + 4 * 2 * 64);   // [4 waves][64] cache row of every key of the tile (8-byte aligned: 2D + 512 floats)
  float* sacc = reinterpret_cast<float*>(srow + 4 * 64);    // [4 waves][2 maps][Dv] partial sums
  float* sml = sacc + 4 * 2 * Dv;            // [4 waves][4] m1, l1, m2, l2
  float* sred = sml + 16;                    // [4]

  int b;
  if (cu_q) {
    int lo = 0, hi = B;                      // the sequence whose row range holds t
    while (hi - lo > 1) { const int mid = (lo + hi) >> 1; if (cu_q[mid] <= t) lo = mid; else hi = mid; }
    b = lo;
  } else {
    b = t / q_per_seq;
  }
  const int nkeys = (int)positions[t] + 1;
  const int32_t* table = bt + (size_t)b * max_blocks;

  const T* qrow = q + ((size_t)t * H + h) * 2 * D;
  for (int d = threadIdx.x; d < 2 * D; d += 256) sq[d] = ldf<T>(qrow + d);
  __syncthreads();

  float m1 = -INFINITY, m2 = -INFINITY, l1 = 0.f, l2 = 0.f;
  float a1[DA_MAXV], a2[DA_MAXV];
#pragma unroll
  for (int i = 0; i < DA_MAXV; ++i) { a1[i] = 0.f; a2[i] = 0.f; }
  float* p1 = sp + (wave * 2 + 0) * 64;
  float* p2 = sp + (wave * 2 + 1) * 64;
  long* rowp = srow + wave * 64;

  const int ntiles = (nkeys + 63) >> 6;
  for (int kt = wave; kt < ntiles; kt += 4) {
    const int j = kt * 64 + lane;
    float s1 = -INFINITY, s2 = -INFINITY;
    long crow = 0;
    if (j < nkeys) {
      crow = ((long)table[j / bs] * G + g) * bs + (j % bs);
      const T* kr = kc + (size_t)crow * 2 * D;
      float d1 = 0.f, d2 = 0.f;
      for (int d = 0; d < D; ++d) {
        d1 = fmaf(sq[d], ldf<T>(kr + d), d1);
        d2 = fmaf(sq[D + d], ldf<T>(kr + D + d), d2);
      }
      s1 = d1 * scale;
      s2 = d2 * scale;
    }
    const float n1 = fmaxf(m1, wave_max(s1)), n2 = fmaxf(m2, wave_max(s2));
    const float c1 = __expf(m1 - n1), c2 = __expf(m2 - n2);       // first tile: exp(-inf) = 0
    const float e1 = j < nkeys ? __expf(s1 - n1) : 0.f, e2 = j < nkeys ? __expf(s2 - n2) : 0.f;
    l1 = l1 * c1 + wave_sum(e1);
    l2 = l2 * c2 + wave_sum(e2);
    m1 = n1; m2 = n2;
    p1[lane] = e1; p2[lane] = e2; rowp[lane] = crow;
    __builtin_amdgcn_wave_barrier();
    __builtin_amdgcn_s_waitcnt(0xc07f);        // lgkmcnt(0): this wave's LDS writes have landed (a wave is its own producer and consumer)
    const int cnt = min(64, nkeys - kt * 64);
#pragma unroll
    for (int i = 0; i < DA_MAXV; ++i) { a1[i] *= c1; a2[i] *= c2; }
    for (int jj = 0; jj < cnt; ++jj) {
      const float w1 = p1[jj], w2 = p2[jj];
      const T* vr = vc + (size_t)rowp[jj] * Dv;
#pragma unroll
      for (int i = 0; i < DA_MAXV; ++i) {
        const int d = lane + i * 64;
        if (d < Dv) { const float v = ldf<T>(vr + d); a1[i] = fmaf(w1, v, a1[i]); a2[i] = fmaf(w2, v, a2[i]); }
      }
    }
    __builtin_amdgcn_wave_barrier();
  }
  // ---- merge the four waves in wave order ----
#pragma unroll
  for (int i = 0; i < DA_MAXV; ++i) {
    const int d = lane + i * 64;
    if (d < Dv) { sacc[(wave * 2 + 0) * Dv + d] = a1[i]; sacc[(wave * 2 + 1) * Dv + d] = a2[i]; }
  }
  if (lane == 0) { sml[wave * 4 + 0] = m1; sml[wave * 4 + 1] = l1; sml[wave * 4 + 2] = m2; sml[wave * 4 + 3] = l2; }
  __syncthreads();
  float M1 = -INFINITY, M2 = -INFINITY;
  for (int w = 0; w < 4; ++w) { M1 = fmaxf(M1, sml[w * 4 + 0]); M2 = fmaxf(M2, sml[w * 4 + 2]); }
  float L1 = 0.f, L2 = 0.f, f1[4], f2[4];
  for (int w = 0; w < 4; ++w) {
    f1[w] = sml[w * 4 + 1] > 0.f ? __expf(sml[w * 4 + 0] - M1) : 0.f;
    f2[w] = sml[w * 4 + 3] > 0.f ? __expf(sml[w * 4 + 2] - M2) : 0.f;
    L1 += sml[w * 4 + 1] * f1[w];
    L2 += sml[w * 4 + 3] * f2[w];
  }
  float ss = 0.f;
  float o[(DA_MAXV + 3) / 4];
#pragma unroll
  for (int i = 0; i < (DA_MAXV + 3) / 4; ++i) {
    const int d = threadIdx.x + i * 256;
    o[i] = 0.f;
    if (d < Dv) {
      float s1 = 0.f, s2 = 0.f;
      for (int w = 0; w < 4; ++w) { s1 += sacc[(w * 2 + 0) * Dv + d] * f1[w]; s2 += sacc[(w * 2 + 1) * Dv + d] * f2[w]; }
      o[i] = s1 / L1 - lambda * (s2 / L2);
      ss += o[i] * o[i];
    }
  }
  ss = wave_sum(ss);
  if (lane == 0) sred[wave] = ss;
  __syncthreads();
  ss = (sred[0] + sred[1]) + (sred[2] + sred[3]);
  const float r = out_scale * gate[(size_t)t * H + h] / sqrtf(ss / (float)Dv + eps);
#pragma unroll
  for (int i = 0; i < (DA_MAXV + 3) / 4; ++i) {
    const int d = threadIdx.x + i * 256;
    if (d < Dv) stf<T>(out + ((size_t)t * H + h) * Dv + d, o[i] * r);
  }
}

}  // namespace

#define LAUNCH_OK() (hipGetLastError() == hipSuccess ? SSD_OK : SSD_ERR_LAUNCH)

extern "C" int ssd_diffattn_store(const void* qkvg_rows, const void* q_norm_w, const void* k_norm_w, float eps, const int32_t* slots,
                                  void* q_out, void* gate_out, void* k_cache, void* v_cache, int T, int H, int G, int D, int Dv,
                                  int block_size, int f32, void* stream) {
  if (!qkvg_rows || !q_norm_w || !k_norm_w || !slots || !q_out || !gate_out || !k_cache || !v_cache) return SSD_ERR_ARG;
  if (T <= 0 || H <= 0 || G <= 0 || H % G || D <= 0 || Dv <= 0 || block_size <= 0) return SSD_ERR_SHAPE;
  if (f32)
    hipLaunchKernelGGL(diffattn_store_kernel<float>, dim3(T), dim3(256), 0, (hipStream_t)stream, (const float*)qkvg_rows,
                       (const float*)q_norm_w, (const float*)k_norm_w, eps, slots, (float*)q_out, (float*)gate_out, (float*)k_cache,
                       (float*)v_cache, H, G, D, Dv, block_size);
  else
    hipLaunchKernelGGL(diffattn_store_kernel<bf16_t>, dim3(T), dim3(256), 0, (hipStream_t)stream, (const float*)qkvg_rows,
                       (const bf16_t*)q_norm_w, (const bf16_t*)k_norm_w, eps, slots, (bf16_t*)q_out, (float*)gate_out,
                       (bf16_t*)k_cache, (bf16_t*)v_cache, H, G, D, Dv, block_size);
  return LAUNCH_OK();
}

extern "C" int ssd_diffattn_paged(const void* q_rows, const void* k_cache, const void* v_cache, const void* gate,
                                  const int32_t* block_tables, int max_blocks, const int64_t* positions, const int32_t* cu_q,
                                  int q_per_seq, int B, int T, int H, int G, int D, int Dv, int block_size, float scale, float lambda,
                                  float out_scale, float eps, void* out_rows, int f32, void* stream) {
  if (!q_rows || !k_cache || !v_cache || !gate || !block_tables || !positions || !out_rows) return SSD_ERR_ARG;
  if (T <= 0 || B <= 0 || H <= 0 || G <= 0 || H % G || D <= 0 || Dv <= 0 || Dv > 64 * DA_MAXV || block_size <= 0 || max_blocks <= 0)
    return SSD_ERR_SHAPE;
  if (!cu_q && q_per_seq <= 0) return SSD_ERR_ARG;
  const size_t lds = (size_t)(2 * D + 4 * 2 * 64) * 4 + 4 * 64 * 8 + (size_t)(4 * 2 * Dv + 16 + 4) * 4 + 8;
  if (lds > 64 * 1024) return SSD_ERR_SHAPE;
  if (f32)
    hipLaunchKernelGGL(diffattn_paged_kernel<float>, dim3(T, H), dim3(256), lds, (hipStream_t)stream, (const float*)q_rows,
                       (const float*)k_cache, (const float*)v_cache, (const float*)gate, block_tables, max_blocks, positions, cu_q,
                       q_per_seq, B, H, G, D, Dv, block_size, scale, lambda, out_scale, eps, (float*)out_rows);
  else
    hipLaunchKernelGGL(diffattn_paged_kernel<bf16_t>, dim3(T, H), dim3(256), lds, (hipStream_t)stream, (const bf16_t*)q_rows,
                       (const bf16_t*)k_cache, (const bf16_t*)v_cache, (const float*)gate, block_tables, max_blocks, positions, cu_q,
                       q_per_seq, B, H, G, D, Dv, block_size, scale, lambda, out_scale, eps, (bf16_t*)out_rows);
  return LAUNCH_OK();
}
