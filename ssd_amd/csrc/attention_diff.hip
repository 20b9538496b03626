// Differential attention over the paged KV cache: every query head owns TWO softmax maps over the same values,
//     o = rms_noweight(a_1 - lambda * a_2) * out_scale * gate,      a_m = softmax(scale * q_m . k_m) v,
// with per-(head, map) RMS norm of q and k (weight shared by all heads and maps), no rotation, and a per-head sigmoid gate.
// Query / key size D and value size Dv are independent and arbitrary (any D, Dv <= 512); element type bf16 or fp32 (`f32`).
//   cache layout per layer: K [blocks][G][block_size][2 * D] (map 1 | map 2, normalised), V TRANSPOSED per page [blocks][G][Dv][block_size]
//   (the keys of a page are contiguous per value column: the weighted sum's MFMA operand is a plain 8-byte load).
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
  // q units 0 .. 2H-1, then k units 0 .. 2G-1: one wave per (head, map) vector of D values; the grid's y cuts the units (and the value /
  // gate columns below) so that a single decoding token still spreads over many workgroups
  for (int u = blockIdx.y * 4 + wave; u < 2 * H + 2 * G; u += 4 * gridDim.y) {
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
    for (int c = blockIdx.y * 256 + threadIdx.x; c < Nv; c += 256 * gridDim.y) {
      const int g = c / Dv, d = c % Dv;
      stf<T>(vc + (((size_t)blk * G + g) * Dv + d) * bs + off, row[Nq + Nk + c]);
    }
  }
  if (blockIdx.y == 0)
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
  long* srow = reinterpret_cast<long*>(sp + 4 * 2 * 64);   // [4 waves][64] V^T address of every key of the tile (8-byte aligned: 2D + 512 floats)
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
      const long pg = (long)table[j / bs] * G + g;
      crow = pg * Dv * bs + (j % bs);                  // element (value 0, this key) of the page's transposed V
      const T* kr = kc + (size_t)(pg * bs + (j % bs)) * 2 * D;
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
      const T* vr = vc + (size_t)rowp[jj];
#pragma unroll
      for (int i = 0; i < DA_MAXV; ++i) {
        const int d = lane + i * 64;
        if (d < Dv) { const float v = ldf<T>(vr + (size_t)d * bs); a1[i] = fmaf(w1, v, a1[i]); a2[i] = fmaf(w2, v, a2[i]); }
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

// ---------------------------------------------------------------------------------------------------------------------
// MFMA form (bf16, D % 8 == 0, D <= 128, Dv % 16 == 0, Dv <= 128, block_size % 32 == 0).  For one kv head, the query ROWS of a
// sequence are its (token, head of the group) pairs; a wave owns 16 rows and walks the keys in steps of 32 (never across a page):
//   S_m[key][row]  = K_m tile (A operand, loaded from the cache rows as they lie) x Q_m (B operand, in registers)   -- 16x16x32, fp32
//   online softmax per row and map in fp32 on the accumulator fragments (a lane holds 8 keys of one row)
//   O_m[dv][row]  += V^T tile (A operand: 2 x 8-byte loads from the transposed page) x P_m (B operand: the lane's 8 weights, bf16)
// The k slots of the second product are the keys in the order the first product's fragments hold them, so no data moves between lanes.
// tile mode  (prompt portions): workgroup = 4 waves = 64 consecutive rows of one sequence, every wave scans keys 0 .. its last row's position.
// split mode (<= 16 rows per sequence: decoding): the 4 waves share the rows and split the keys; partial (max, sum, O) merge in LDS
//            in wave order.  With a workspace the keys are first cut into slices over blockIdx.z; a one-wave merge kernel per
//            (sequence, kv head) then sums the slices in order.
// Keys past a row's position are masked by select (whatever the cache holds there); V of keys past the sequence's length is zeroed.
// ---------------------------------------------------------------------------------------------------------------------
constexpr int DM_KS = 4, DM_DVT = 8;

__device__ __forceinline__ float quad_max(float v) { v = fmaxf(v, __shfl_xor(v, 16, 64)); return fmaxf(v, __shfl_xor(v, 32, 64)); }
__device__ __forceinline__ float quad_sum(float v) { v += __shfl_xor(v, 16, 64); return v + __shfl_xor(v, 32, 64); }

constexpr int DM_WS_SLOT = 64 + 2 * DM_DVT * 64 * 4;      // floats per (sequence, kv head, key slice): max / sum rows, then the O fragments

// Combine the maps, norm over the head's values, scale, gate; lane (row r, values i*16 + qd*4 ..+3) holds acc[m][i][0..3].
__device__ __forceinline__ void diff_finalize(f32x4_t (&acc)[2][DM_DVT], const float (&ls)[2], int DVT, int Dv, float lambda,
                                              float out_scale, float gate, float eps, bool valid, bf16_t* orow) {
  const float i1 = 1.0f / ls[0], i2 = lambda / ls[1];
  float ss = 0.f;
#pragma unroll
  for (int i = 0; i < DM_DVT; ++i)
    if (i < DVT) {
      acc[0][i] = acc[0][i] * i1 - acc[1][i] * i2;
#pragma unroll
      for (int e = 0; e < 4; ++e) ss += acc[0][i][e] * acc[0][i][e];
    }
  ss = quad_sum(ss);
  const float rn = out_scale * gate / sqrtf(ss / (float)Dv + eps);
  if (valid) {
#pragma unroll
    for (int i = 0; i < DM_DVT; ++i)
      if (i < DVT) {
        const u32x2_t o = {pack_bf2(acc[0][i][0] * rn, acc[0][i][1] * rn), pack_bf2(acc[0][i][2] * rn, acc[0][i][3] * rn)};
        *reinterpret_cast<u32x2_t*>(orow + i * 16) = o;
      }
  }
}

__global__ void __launch_bounds__(256)
diffattn_mfma_kernel(const bf16_t* __restrict__ q, const bf16_t* __restrict__ kc, const bf16_t* __restrict__ vt,
                     const float* __restrict__ gate, const int32_t* __restrict__ bt, int max_blocks,
                     const int64_t* __restrict__ positions, const int32_t* __restrict__ ctx_lens, const int32_t* __restrict__ cu_q,
                     int q_per_seq, int B, int H, int G, int D, int Dv, int bs, float scale, float lambda, float out_scale, float eps,
                     bf16_t* __restrict__ out, int split, int nsplit, float* __restrict__ ws) {
  extern __shared__ float smem[];
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63, r = lane & 15, qd = lane >> 4;
  const int g = blockIdx.y, R = H / G;
  const int KS = (D + 31) >> 5, DVT = Dv >> 4;
  // ---- which sequence, which rows ----
  int b = 0, tile = blockIdx.x, tok0 = 0, qb = 0;
  if (split) {
    b = blockIdx.x; tile = 0;
    tok0 = cu_q ? cu_q[b] : b * q_per_seq;
    qb = cu_q ? cu_q[b + 1] - cu_q[b] : q_per_seq;
  } else {
    for (; b < B; ++b) {
      tok0 = cu_q ? cu_q[b] : b * q_per_seq;
      qb = cu_q ? cu_q[b + 1] - cu_q[b] : q_per_seq;
      const int nt = (qb * R + 63) >> 6;
      if (tile < nt) break;
      tile -= nt;
    }
    if (b >= B) return;
  }
  const int nrows = qb * R;
  const int row0 = split ? 0 : tile * 64 + wave * 16;
  if (!split && row0 >= nrows) return;                 // (tile mode has no workgroup barriers)
  const int row = row0 + r;
  const bool valid = row < nrows;
  const int rr = valid ? row : row0;
  const int token = tok0 + rr / R, head = g * R + rr % R;
  const int pos = (int)positions[token];
  const int ctx = ctx_lens[b];
  int maxpos = pos;
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) maxpos = max(maxpos, __shfl_xor(maxpos, o, 64));
  const int32_t* table = bt + (size_t)b * max_blocks;

  // ---- Q in registers: B operand, lane (row r, dims ks*32 + qd*8 ..+7) ----
  u32x4_t qreg[2][DM_KS];
  const bf16_t* qrow = q + ((size_t)token * H + head) * 2 * D;
#pragma unroll
  for (int m = 0; m < 2; ++m)
#pragma unroll
    for (int ks = 0; ks < DM_KS; ++ks) {
      qreg[m][ks] = u32x4_t{0u, 0u, 0u, 0u};
      const int d0 = ks * 32 + qd * 8;
      if (ks < KS && d0 < D && valid) qreg[m][ks] = *reinterpret_cast<const u32x4_t*>(qrow + m * D + d0);
    }

  float mx[2] = {-INFINITY, -INFINITY}, ls[2] = {0.f, 0.f};
  f32x4_t acc[2][DM_DVT];
#pragma unroll
  for (int m = 0; m < 2; ++m)
#pragma unroll
    for (int i = 0; i < DM_DVT; ++i) acc[m][i] = f32x4_t{0.f, 0.f, 0.f, 0.f};

  const int nsteps = (maxpos >> 5) + 1;
  int s_begin = 0, s_end = nsteps;
  if (split) {        // this workgroup's slice of the steps (all of them without a grid split), cut over the four waves
    const int per_wg = (nsteps + nsplit - 1) / nsplit;
    const int g_begin = min(nsteps, (int)blockIdx.z * per_wg), g_end = min(nsteps, g_begin + per_wg);
    const int per = (g_end - g_begin + 3) >> 2;
    s_begin = min(g_end, g_begin + wave * per);
    s_end = min(g_end, s_begin + per);
  }

  for (int st = s_begin; st < s_end; ++st) {
    const int k0 = st << 5;
    const size_t pg = (size_t)table[k0 / bs] * G + g;
    const int koff = k0 % bs;
    // every load of the step is issued before the first product: one memory round trip per 32 keys (the value tiles do not wait for
    // the softmax)
    u32x4_t kreg[2][2][DM_KS];
    u32x2_t vlo[DM_DVT], vhi[DM_DVT];
#pragma unroll
    for (int m = 0; m < 2; ++m)
#pragma unroll
      for (int hg = 0; hg < 2; ++hg) {
        const bf16_t* kr = kc + (pg * bs + koff + hg * 16 + r) * 2 * D + m * D + qd * 8;
#pragma unroll
        for (int ks = 0; ks < DM_KS; ++ks) {
          kreg[m][hg][ks] = u32x4_t{0u, 0u, 0u, 0u};
          if (ks < KS && ks * 32 + qd * 8 < D) kreg[m][hg][ks] = *reinterpret_cast<const u32x4_t*>(kr + ks * 32);
        }
      }
#pragma unroll
    for (int i = 0; i < DM_DVT; ++i) {
      vlo[i] = u32x2_t{0u, 0u};
      vhi[i] = u32x2_t{0u, 0u};
      if (i < DVT) {
        const bf16_t* vp = vt + (pg * Dv + i * 16 + r) * bs + koff + qd * 4;
        vlo[i] = *reinterpret_cast<const u32x2_t*>(vp);
        vhi[i] = *reinterpret_cast<const u32x2_t*>(vp + 16);
      }
    }
    f32x4_t s[2][2];
#pragma unroll
    for (int m = 0; m < 2; ++m)
#pragma unroll
      for (int hg = 0; hg < 2; ++hg) {
        s[m][hg] = f32x4_t{0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int ks = 0; ks < DM_KS; ++ks)
          if (ks < KS) s[m][hg] = mfma16(kreg[m][hg][ks], qreg[m][ks], s[m][hg]);
      }
    u32x4_t pb[2];
#pragma unroll
    for (int m = 0; m < 2; ++m) {
      float v[8];
      float tmax = -INFINITY;
#pragma unroll
      for (int hg = 0; hg < 2; ++hg)
#pragma unroll
        for (int e = 0; e < 4; ++e) {
          const int key = k0 + hg * 16 + qd * 4 + e;
          const float x = key <= pos ? s[m][hg][e] * scale : -INFINITY;
          v[hg * 4 + e] = x;
          tmax = fmaxf(tmax, x);
        }
      tmax = quad_max(tmax);
      const float mnew = fmaxf(mx[m], tmax);
      const float msafe = mnew == -INFINITY ? 0.f : mnew;
      const float corr = __expf(mx[m] - msafe);
      float psum = 0.f;
#pragma unroll
      for (int e = 0; e < 8; ++e) { v[e] = __expf(v[e] - msafe); psum += v[e]; }
      psum = quad_sum(psum);
      ls[m] = ls[m] * corr + psum;
      mx[m] = mnew;
#pragma unroll
      for (int i = 0; i < DM_DVT; ++i) acc[m][i] *= corr;
      pb[m] = u32x4_t{pack_bf2(v[0], v[1]), pack_bf2(v[2], v[3]), pack_bf2(v[4], v[5]), pack_bf2(v[6], v[7])};
    }
    const bool tail = k0 + 32 > ctx;
#pragma unroll
    for (int i = 0; i < DM_DVT; ++i) {
      if (i < DVT) {
        u32x2_t lo = vlo[i], hi = vhi[i];
        if (tail) {         // keys past the sequence: whatever the page holds there must not meet a zero weight as NaN
          const int kb = k0 + qd * 4;
          if (kb + 0 >= ctx) lo.x &= 0xffff0000u;
          if (kb + 1 >= ctx) lo.x &= 0x0000ffffu;
          if (kb + 2 >= ctx) lo.y &= 0xffff0000u;
          if (kb + 3 >= ctx) lo.y &= 0x0000ffffu;
          if (kb + 16 >= ctx) hi.x &= 0xffff0000u;
          if (kb + 17 >= ctx) hi.x &= 0x0000ffffu;
          if (kb + 18 >= ctx) hi.y &= 0xffff0000u;
          if (kb + 19 >= ctx) hi.y &= 0x0000ffffu;
        }
        const u32x4_t a = {lo.x, lo.y, hi.x, hi.y};
        acc[0][i] = mfma16(a, pb[0], acc[0][i]);
        acc[1][i] = mfma16(a, pb[1], acc[1][i]);
      }
    }
  }

  if (split) {
    // ---- merge the four waves' partials in wave order ----
    float* sm = smem;                       // [4 waves][2 maps][2: max, sum][16 rows]
    float* sbuf = smem + 4 * 2 * 2 * 16;    // [3 waves][2 maps][DVT][64 lanes][4]
    if (qd == 0) {
#pragma unroll
      for (int m = 0; m < 2; ++m) { sm[((wave * 2 + m) * 2 + 0) * 16 + r] = mx[m]; sm[((wave * 2 + m) * 2 + 1) * 16 + r] = ls[m]; }
    }
    __syncthreads();
#pragma unroll
    for (int m = 0; m < 2; ++m) {
      float M = -INFINITY;
      for (int w = 0; w < 4; ++w) M = fmaxf(M, sm[((w * 2 + m) * 2 + 0) * 16 + r]);
      float L = 0.f;
      for (int w = 0; w < 4; ++w) {
        const float mw = sm[((w * 2 + m) * 2 + 0) * 16 + r];
        L += mw == -INFINITY ? 0.f : sm[((w * 2 + m) * 2 + 1) * 16 + r] * __expf(mw - M);
      }
      const float f = mx[m] == -INFINITY ? 0.f : __expf(mx[m] - M);
#pragma unroll
      for (int i = 0; i < DM_DVT; ++i) acc[m][i] *= f;
      ls[m] = L;
      mx[m] = M;
    }
    // waves 1..3 leave their (already rescaled) O fragments in areas of their own; wave 0 adds them in wave order: one barrier
    const size_t area = (size_t)2 * DVT * 64 * 4;
    if (wave > 0) {
#pragma unroll
      for (int m = 0; m < 2; ++m)
#pragma unroll
        for (int i = 0; i < DM_DVT; ++i)
          if (i < DVT) *reinterpret_cast<f32x4_t*>(sbuf + (wave - 1) * area + ((size_t)(m * DVT + i) * 64 + lane) * 4) = acc[m][i];
    }
    __syncthreads();
    if (wave == 0) {
      for (int w = 0; w < 3; ++w)
#pragma unroll
        for (int m = 0; m < 2; ++m)
#pragma unroll
          for (int i = 0; i < DM_DVT; ++i)
            if (i < DVT) acc[m][i] += *reinterpret_cast<const f32x4_t*>(sbuf + w * area + ((size_t)(m * DVT + i) * 64 + lane) * 4);
    }
    if (wave != 0) return;
  }

  if (nsplit > 1) {
    // ---- this workgroup scanned one slice of the keys: leave (max, sum, O) for the merge kernel, in register layout ----
    const size_t slot = ((size_t)b * G + g) * nsplit + blockIdx.z;
    float* wml = ws + slot * DM_WS_SLOT;
    if (qd == 0) {
#pragma unroll
      for (int m = 0; m < 2; ++m) { wml[(m * 2 + 0) * 16 + r] = mx[m]; wml[(m * 2 + 1) * 16 + r] = ls[m]; }
    }
    f32x4_t* wacc = reinterpret_cast<f32x4_t*>(wml + 64);
#pragma unroll
    for (int m = 0; m < 2; ++m)
#pragma unroll
      for (int i = 0; i < DM_DVT; ++i)
        if (i < DVT) wacc[(m * DM_DVT + i) * 64 + lane] = acc[m][i];
    return;
  }
  diff_finalize(acc, ls, DVT, Dv, lambda, out_scale, gate[(size_t)token * H + head], eps, valid,
                out + ((size_t)token * H + head) * Dv + qd * 4);
}

// The second pass of a key-split decode: one workgroup per (sequence, kv head); its 4 waves share the value tiles (wave w sums tiles
// w, w + 4 of both maps over the slices, in slice order), the rows' mean squares meet in LDS, then every wave finishes its tiles.
__global__ void __launch_bounds__(256)
diffattn_merge_kernel(const float* __restrict__ ws, int nsplit, const float* __restrict__ gate, const int32_t* __restrict__ cu_q,
                      int q_per_seq, int H, int G, int Dv, float lambda, float out_scale, float eps, bf16_t* __restrict__ out) {
  __shared__ float sss[4][16];
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63, r = lane & 15, qd = lane >> 4;
  const int b = blockIdx.x, g = blockIdx.y, R = H / G, DVT = Dv >> 4;
  const int tok0 = cu_q ? cu_q[b] : b * q_per_seq;
  const int qb = cu_q ? cu_q[b + 1] - cu_q[b] : q_per_seq;
  const bool valid = r < qb * R;
  const int rr = valid ? r : 0;
  const int token = tok0 + rr / R, head = g * R + rr % R;
  const float* base = ws + ((size_t)b * G + g) * nsplit * DM_WS_SLOT;
  float M[2] = {-INFINITY, -INFINITY}, ls[2] = {0.f, 0.f};
  for (int sidx = 0; sidx < nsplit; ++sidx)
#pragma unroll
    for (int m = 0; m < 2; ++m) M[m] = fmaxf(M[m], base[(size_t)sidx * DM_WS_SLOT + (m * 2 + 0) * 16 + r]);
  constexpr int PER = DM_DVT / 4;
  f32x4_t acc[2][PER];
#pragma unroll
  for (int m = 0; m < 2; ++m)
#pragma unroll
    for (int k = 0; k < PER; ++k) acc[m][k] = f32x4_t{0.f, 0.f, 0.f, 0.f};
  for (int sidx = 0; sidx < nsplit; ++sidx) {
    const float* wml = base + (size_t)sidx * DM_WS_SLOT;
    const f32x4_t* wacc = reinterpret_cast<const f32x4_t*>(wml + 64);
#pragma unroll
    for (int m = 0; m < 2; ++m) {
      const float ms = wml[(m * 2 + 0) * 16 + r];
      const float f = ms == -INFINITY ? 0.f : __expf(ms - M[m]);
      ls[m] += wml[(m * 2 + 1) * 16 + r] * f;
#pragma unroll
      for (int k = 0; k < PER; ++k) {
        const int i = wave + 4 * k;
        if (i < DVT) acc[m][k] += wacc[(m * DM_DVT + i) * 64 + lane] * f;
      }
    }
  }
  const float i1 = 1.0f / ls[0], i2 = lambda / ls[1];
  float ss = 0.f;
#pragma unroll
  for (int k = 0; k < PER; ++k)
    if (wave + 4 * k < DVT) {
      acc[0][k] = acc[0][k] * i1 - acc[1][k] * i2;
#pragma unroll
      for (int e = 0; e < 4; ++e) ss += acc[0][k][e] * acc[0][k][e];
    }
  ss = quad_sum(ss);
  if (qd == 0) sss[wave][r] = ss;
  __syncthreads();
  ss = (sss[0][r] + sss[1][r]) + (sss[2][r] + sss[3][r]);
  const float rn = out_scale * gate[(size_t)token * H + head] / sqrtf(ss / (float)Dv + eps);
  if (valid) {
    bf16_t* orow = out + ((size_t)token * H + head) * Dv + qd * 4;
#pragma unroll
    for (int k = 0; k < PER; ++k) {
      const int i = wave + 4 * k;
      if (i < DVT) {
        const u32x2_t o = {pack_bf2(acc[0][k][0] * rn, acc[0][k][1] * rn), pack_bf2(acc[0][k][2] * rn, acc[0][k][3] * rn)};
        *reinterpret_cast<u32x2_t*>(orow + i * 16) = o;
      }
    }
  }
}

}  // namespace

#define LAUNCH_OK() (hipGetLastError() == hipSuccess ? SSD_OK : SSD_ERR_LAUNCH)

extern "C" int ssd_diffattn_store(const void* qkvg_rows, const void* q_norm_w, const void* k_norm_w, float eps, const int32_t* slots,
                                  void* q_out, void* gate_out, void* k_cache, void* v_cache, int T, int H, int G, int D, int Dv,
                                  int block_size, int f32, void* stream) {
  if (!qkvg_rows || !q_norm_w || !k_norm_w || !slots || !q_out || !gate_out || !k_cache || !v_cache) return SSD_ERR_ARG;
  if (T <= 0 || H <= 0 || G <= 0 || H % G || D <= 0 || Dv <= 0 || block_size <= 0) return SSD_ERR_SHAPE;
  int gy = (2 * H + 2 * G + 3) / 4;                 // one unit per wave when few tokens; fewer, fatter workgroups for prompt portions
  if (T >= 64) gy = (gy + 7) / 8;
  if (gy < 1) gy = 1;
  if (f32)
    hipLaunchKernelGGL(diffattn_store_kernel<float>, dim3(T, gy), dim3(256), 0, (hipStream_t)stream, (const float*)qkvg_rows,
                       (const float*)q_norm_w, (const float*)k_norm_w, eps, slots, (float*)q_out, (float*)gate_out, (float*)k_cache,
                       (float*)v_cache, H, G, D, Dv, block_size);
  else
    hipLaunchKernelGGL(diffattn_store_kernel<bf16_t>, dim3(T, gy), dim3(256), 0, (hipStream_t)stream, (const float*)qkvg_rows,
                       (const bf16_t*)q_norm_w, (const bf16_t*)k_norm_w, eps, slots, (bf16_t*)q_out, (float*)gate_out,
                       (bf16_t*)k_cache, (bf16_t*)v_cache, H, G, D, Dv, block_size);
  return LAUNCH_OK();
}

extern "C" int ssd_diffattn_paged(const void* q_rows, const void* k_cache, const void* v_cache, const void* gate,
                                  const int32_t* block_tables, int max_blocks, const int64_t* positions, const int32_t* context_lens,
                                  const int32_t* cu_q, int q_per_seq, int max_q, int B, int T, int H, int G, int D, int Dv,
                                  int block_size, float scale, float lambda, float out_scale, float eps, void* out_rows, int f32,
                                  void* workspace, long workspace_bytes, int ctx_hint, void* stream) {
  if (!q_rows || !k_cache || !v_cache || !gate || !block_tables || !positions || !out_rows) return SSD_ERR_ARG;
  if (T <= 0 || B <= 0 || H <= 0 || G <= 0 || H % G || D <= 0 || Dv <= 0 || Dv > 64 * DA_MAXV || block_size <= 0 || max_blocks <= 0)
    return SSD_ERR_SHAPE;
  if (!cu_q && q_per_seq <= 0) return SSD_ERR_ARG;
  if (!f32 && context_lens && max_q > 0 && D % 8 == 0 && D <= 32 * DM_KS && Dv % 16 == 0 && Dv <= 16 * DM_DVT && block_size % 32 == 0 &&
      (2 * D * 2) % 16 == 0) {
    const int R = H / G;
    const int split = max_q * R <= 16 ? 1 : 0;
    const int gx = split ? B : ((long)T * R + 63) / 64 + B;
    const size_t lds_m = split ? (size_t)(4 * 2 * 2 * 16 + 3 * 2 * (Dv / 16) * 64 * 4) * 4 : 0;
    // decoding rows of few sequences: cut the keys over more workgroups (a launch of B * G workgroups leaves most of the chip idle)
    // when the caller gave a workspace and says the contexts are long; every wave keeps at least 4 steps of 32 keys
    int nsplit = 1;
    if (split && workspace && ctx_hint > 0) {
      nsplit = 256 / (B * G);
      const int by_len = ctx_hint / (32 * 4 * 4);
      if (nsplit > by_len) nsplit = by_len;
      if (nsplit > 16) nsplit = 16;
      while (nsplit > 1 && (long)B * G * nsplit * DM_WS_SLOT * 4 > workspace_bytes) --nsplit;
      if (nsplit < 1) nsplit = 1;
    }
    hipLaunchKernelGGL(diffattn_mfma_kernel, dim3(gx, G, nsplit), dim3(256), lds_m, (hipStream_t)stream, (const bf16_t*)q_rows,
                       (const bf16_t*)k_cache, (const bf16_t*)v_cache, (const float*)gate, block_tables, max_blocks, positions,
                       context_lens, cu_q, q_per_seq, B, H, G, D, Dv, block_size, scale, lambda, out_scale, eps, (bf16_t*)out_rows, split,
                       nsplit, (float*)workspace);
    if (nsplit > 1)
      hipLaunchKernelGGL(diffattn_merge_kernel, dim3(B, G), dim3(256), 0, (hipStream_t)stream, (const float*)workspace, nsplit,
                         (const float*)gate, cu_q, q_per_seq, H, G, Dv, lambda, out_scale, eps, (bf16_t*)out_rows);
    return LAUNCH_OK();
  }
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
