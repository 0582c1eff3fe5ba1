// Causal attention of a prefill chunk: the (scores, softmax . V) pairs of m consecutive tokens in one
// launch.
//
// Reference: the same two ops as in decode (map_matmul_t_dev for the scores,
// shaders/src/f32/map_matmul_t.comp, and map_attn_softmax_value_dev, map_attn_softmax_value.comp:39-89;
// arithmetic adam/models/engine.py:2428-2441), which a caller that processes a prompt in chunks issues
// once per token: token t of the chunk sees the first seq0 + t rows of the K and V cache.  When a batch
// holds such a run -- same heads, cache and score rows for every token, query and output rows at a
// fixed stride from token to token, one more visible row each -- the run is launched here instead
// of token by token.
//
// A workgroup owns one query head and a tile of 16 consecutive tokens; its NW waves take the
// 16-row tiles of the cache in turn.  Per tile: scores on v_mfma_f32_16x16x16_f16 with A = the 16
// queries (scaled per query by a power of two into fp16 range and split hi + lo, so the products are
// exact and the sum is fp32) and B = the K tile; rows past a query's own position are masked; online
// softmax per wave and query; values with every lane owning D/64 dims of all 16 outputs.  The waves
// merge through LDS.  The raw scores of the chunk's last token are stored to the score rows: that
// is what the rows hold after the run executed token by token, each token overwriting the one before.
#include "attn_common.h"
#include <algorithm>

namespace adamah {

typedef _Float16 h4p_t __attribute__((ext_vector_type(4)));
typedef float f4p_t __attribute__((ext_vector_type(4)));
typedef uint32_t u2p_t __attribute__((ext_vector_type(2)));

#define ATTP_NEG (-1.0e30f)
#define ATTP_MAX_HEADS 64u
struct AttpBases { uint32_t q[ATTP_MAX_HEADS], sc[ATTP_MAX_HEADS], o[ATTP_MAX_HEADS], kb[ATTP_MAX_HEADS], vb[ATTP_MAX_HEADS]; };

#define ATTP_DPP(v, ctrl) __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), ctrl, 0xF, 0xF, false))
__device__ __forceinline__ float prow16_max(float v) {
  v = fmaxf(v, ATTP_DPP(v, 0xB1)); v = fmaxf(v, ATTP_DPP(v, 0x4E));
  v = fmaxf(v, ATTP_DPP(v, 0x141)); v = fmaxf(v, ATTP_DPP(v, 0x140));
  return v;
}
__device__ __forceinline__ float prow16_sum(float v) {
  v += ATTP_DPP(v, 0xB1); v += ATTP_DPP(v, 0x4E); v += ATTP_DPP(v, 0x141); v += ATTP_DPP(v, 0x140);
  return v;
}

template <int D, int NW>
__global__ void __launch_bounds__(NW * 64)
k_attn_prefill(const float* data, float* out, const __half* kv, uint64_t kv_shift, const AttpBases bs, uint32_t m,
               uint32_t seq0, uint32_t q_stride, uint32_t o_stride, float scale, float cap) {
  constexpr int NI = D / 32;           // 16-byte K loads per lane and tile
  constexpr int DPL = D / 64;          // V dims per lane
  constexpr int DW = DPL > 2 ? DPL / 2 : 1;
  constexpr uint32_t NT = NW * 64;
  __shared__ __attribute__((aligned(16))) float pbuf[NW][16][16];   // softmax weights of the wave's tile, [cache row][query]
  __shared__ float abuf[NW][16];       // per query: rescale factor of the tile
  __shared__ float obuf[NW][16][D];    // wave results; first the 16 queries, [query][dim]
  __shared__ float mlbuf[NW][16][2];
  __shared__ h4p_t qop[2 * NI][2][64]; // query operands of the matrix product: [k-step][hi, lo][lane]
  __shared__ uint32_t hmax[16];        // per query: bits of max |q|
  __shared__ float qinv[16];           // per query: 1 / (power-of-two scale)

  const uint32_t tid = threadIdx.x, lane = tid & 63u;
  const uint32_t wave = (uint32_t)__builtin_amdgcn_readfirstlane((int)(tid >> 6));
  const uint32_t c = lane & 15u, kc = lane >> 4;
  const uint32_t head = blockIdx.y, t0 = blockIdx.x * 16u;
  const uint32_t rows = min(16u, m - t0);                 // queries of this tile
  const uint32_t nkeys = seq0 + t0 + rows - 1u;           // cache rows the last of them sees
  const char* kbase = (const char*)(kv + ((uint64_t)bs.kb[head] - kv_shift));
  const char* vbase = (const char*)(kv + ((uint64_t)bs.vb[head] - kv_shift));
  const uint32_t klane = 16u * kc, vlane = 2u * (uint32_t)DPL * lane;

  auto fetch = [&](uint4 (&kr)[NI], uint32_t (&vr)[16][DW], uint32_t rb) {
    const uint32_t koff = min(rb + c, nkeys - 1u) * (2u * D) + klane;
#pragma unroll
    for (int i = 0; i < NI; i++) kr[i] = *(const uint4*)(kbase + koff + 64u * i);
#pragma unroll
    for (int u = 0; u < 16; u++) {
      const char* src = vbase + (uint64_t)(min(rb + u, nkeys - 1u) * (2u * D)) + vlane;
      if (DPL == 1) vr[u][0] = *(const uint16_t*)src;
      else if (DPL == 2) vr[u][0] = *(const uint32_t*)src;
      else { const uint2 t = *(const uint2*)src; vr[u][0] = t.x; vr[u][DW - 1] = t.y; }
    }
  };

  // queries -> LDS (obuf[0] is free until the end) with the per-query maximum on the way; then the
  // matrix-A operands: lane (query c, kc) of operand 2i+j holds dims 32i + 8kc + 4j .. +3 of query c
  uint4 kA[NI];
  uint32_t vA[16][DW];
  uint32_t rbase = wave * 16u;
  {
    float* qs = &obuf[0][0][0];
    if (tid < 16u) hmax[tid] = 0u;
    __syncthreads();
    for (uint32_t i = tid; i < 16u * D; i += NT) {          // a wave's 64 elements belong to one query
      const uint32_t r = i / D;
      const float x = r < rows ? data[(uint64_t)bs.q[head] + (uint64_t)(t0 + r) * q_stride + i % D] : 0.f;
      qs[i] = x;
      float mx = fabsf(x);
#pragma unroll
      for (int o = 32; o > 0; o >>= 1) mx = fmaxf(mx, __shfl_xor(mx, o, 64));
      if (lane == 0u) atomicMax(&hmax[r], __float_as_uint(mx));
    }
    if (rbase < nkeys) fetch(kA, vA, rbase);
    __builtin_amdgcn_sched_barrier(0);
    __syncthreads();
    const uint32_t e = (hmax[c] >> 23) & 0xFFu;
    float s = 1.f, inv = 1.f;
    if (e >= 14u && e <= 254u) { s = __uint_as_float((267u - e) << 23); inv = __uint_as_float((e - 13u) << 23); }
    if (wave == 0u && kc == 0u) qinv[c] = inv;
    for (uint32_t idx = wave; idx < 2u * NI; idx += NW) {
      const float4 q4 = *(const float4*)(qs + c * D + 32u * (idx >> 1) + 8u * kc + 4u * (idx & 1u));
      const float x[4] = {q4.x * s, q4.y * s, q4.z * s, q4.w * s};
      h4p_t hi4, lo4;
#pragma unroll
      for (int t = 0; t < 4; t++) {
        const _Float16 hi = (_Float16)x[t];
        hi4[t] = hi;
        lo4[t] = (_Float16)(x[t] - (float)hi);
      }
      qop[idx][0][lane] = hi4;
      qop[idx][1][lane] = lo4;
    }
    __syncthreads();
  }
  // after the matrix product lane (c, kc) holds queries 4kc..4kc+3 against cache row c of the tile
  float inv_s[4], m_run[4], l_run[4];
  uint32_t lim[4];                     // cache rows the query sees (0: no such query)
  bool last[4];
#pragma unroll
  for (int r = 0; r < 4; r++) {
    const uint32_t qr = 4u * kc + r;
    inv_s[r] = qinv[qr];
    lim[r] = qr < rows ? seq0 + t0 + qr : 0u;
    last[r] = qr < rows && t0 + qr == m - 1u;
    m_run[r] = ATTP_NEG;
    l_run[r] = 0.f;
  }
  const uint32_t sc_row = bs.sc[head];

  float acc[16][DPL];
#pragma unroll
  for (int h = 0; h < 16; h++)
#pragma unroll
    for (int j = 0; j < DPL; j++) acc[h][j] = 0.f;

  for (; rbase < nkeys; rbase += NW * 16u) {
    f4p_t s0 = {0.f, 0.f, 0.f, 0.f}, s1 = s0, s2 = s0, s3 = s0;
#pragma unroll
    for (int i = 0; i < NI; i++) {
      const u2p_t b0 = {kA[i].x, kA[i].y}, b1 = {kA[i].z, kA[i].w};
      s0 = __builtin_amdgcn_mfma_f32_16x16x16f16(qop[2 * i][0][lane], __builtin_bit_cast(h4p_t, b0), s0, 0, 0, 0);
      s1 = __builtin_amdgcn_mfma_f32_16x16x16f16(qop[2 * i][1][lane], __builtin_bit_cast(h4p_t, b0), s1, 0, 0, 0);
      s2 = __builtin_amdgcn_mfma_f32_16x16x16f16(qop[2 * i + 1][0][lane], __builtin_bit_cast(h4p_t, b1), s2, 0, 0, 0);
      s3 = __builtin_amdgcn_mfma_f32_16x16x16f16(qop[2 * i + 1][1][lane], __builtin_bit_cast(h4p_t, b1), s3, 0, 0, 0);
    }
    const uint32_t key = rbase + c;
    float v[4], mt[4];
#pragma unroll
    for (int r = 0; r < 4; r++) {
      const float raw = ((s0[r] + s2[r]) + (s1[r] + s3[r])) * inv_s[r];
      const bool ok = key < lim[r];
      if (ok && last[r]) out[(uint64_t)sc_row + key] = raw;
      v[r] = ok ? prep(raw, scale, cap) : ATTP_NEG;
      mt[r] = prow16_max(v[r]);
    }
#pragma unroll
    for (int r = 0; r < 4; r++) {
      const float m_new = fmaxf(m_run[r], mt[r]);
      const float alpha = __expf(m_run[r] - m_new);
      const float p = key < lim[r] ? __expf(v[r] - m_new) : 0.f;
      l_run[r] = l_run[r] * alpha + p;
      m_run[r] = m_new;
      pbuf[wave][c][4u * kc + r] = p;
      if (c == 0u) abuf[wave][4u * kc + r] = alpha;
    }
    __builtin_amdgcn_wave_barrier();
#pragma unroll
    for (int h = 0; h < 16; h++) {
      const float al = abuf[wave][h];
#pragma unroll
      for (int j = 0; j < DPL; j++) acc[h][j] *= al;
    }
#pragma unroll
    for (int u = 0; u < 16; u++) {
      float f[DPL];
      if (DPL == 1) f[0] = __half2float(__ushort_as_half((unsigned short)vA[u][0]));
      else {
#pragma unroll
        for (int w = 0; w < DW; w++) {
          const float2 t = __half22float2(*(const __half2*)&vA[u][w]);
          f[2 * w] = t.x; f[(2 * w + 1) % DPL] = t.y;
        }
      }
#pragma unroll
      for (int h4 = 0; h4 < 4; h4++) {
        const float4 pw = *(const float4*)&pbuf[wave][u][4 * h4];
#pragma unroll
        for (int j = 0; j < DPL; j++) {
          acc[4 * h4 + 0][j] = fmaf(pw.x, f[j], acc[4 * h4 + 0][j]);
          acc[4 * h4 + 1][j] = fmaf(pw.y, f[j], acc[4 * h4 + 1][j]);
          acc[4 * h4 + 2][j] = fmaf(pw.z, f[j], acc[4 * h4 + 2][j]);
          acc[4 * h4 + 3][j] = fmaf(pw.w, f[j], acc[4 * h4 + 3][j]);
        }
      }
    }
    __builtin_amdgcn_wave_barrier();
    if (rbase + NW * 16u < nkeys) fetch(kA, vA, rbase + NW * 16u);
  }

  // wave results to LDS: l summed over the 16 cache rows of the tiles; each lane owns its dims
#pragma unroll
  for (int r = 0; r < 4; r++) l_run[r] = prow16_sum(l_run[r]);
  __syncthreads();                     // the queries in obuf[0] have been consumed by every wave
#pragma unroll
  for (int h = 0; h < 16; h++)
#pragma unroll
    for (int j = 0; j < DPL; j++) obuf[wave][h][(uint32_t)DPL * lane + j] = acc[h][j];
  if (c == 0u) {
#pragma unroll
    for (int r = 0; r < 4; r++) { mlbuf[wave][4u * kc + r][0] = m_run[r]; mlbuf[wave][4u * kc + r][1] = l_run[r]; }
  }
  __syncthreads();
  for (uint32_t idx = tid; idx < 16u * D; idx += NT) {
    const uint32_t h = idx / D, d = idx % D;
    if (h >= rows) continue;
    float M = mlbuf[0][h][0];
#pragma unroll
    for (int w = 1; w < NW; w++) M = fmaxf(M, mlbuf[w][h][0]);
    float o = 0.f, L = 0.f;
#pragma unroll
    for (int w = 0; w < NW; w++) {
      const float e = __expf(mlbuf[w][h][0] - M);
      o = fmaf(obuf[w][h][d], e, o);
      L = fmaf(mlbuf[w][h][1], e, L);
    }
    out[(uint64_t)bs.o[head] + (uint64_t)(t0 + h) * o_stride + d] = o * (1.0f / L);
  }
}

// ---- the same chunk with both products on the matrix cores ------------------------------------------------
// k_attn_prefill above accumulates softmax . V with vector multiply-adds (16 queries x D/64 dims per lane and cache
// row) and walks the cache once per query head.  The form below keeps everything in v_mfma_f32_16x16x32_f16:
//
//   * a wave owns one query head and a tile of 16 consecutive tokens and walks the cache in tiles of 32 rows; the
//     four waves of a workgroup are four heads of the same token tile -- with grouped queries, the heads of one KV
//     head, so their K / V tiles come out of the L1 after the first wave has asked for them;
//   * scores transposed, S^T = K . Q^T: A = K tile (row = cache row, 8 consecutive dims per lane: one 16-byte
//     piece), B = the queries as exact hi + lo fp16 pairs after a power-of-two scale (held in registers for the
//     whole walk).  Read from the row-major cache, the sixteen pieces of neighbouring lanes lie in sixteen
//     different rows, and the L1 takes a load instruction's lanes four at a time only where they are neighbours in
//     memory: 64 tag look-ups per instruction instead of 16, which made the K loads (eight of a tile's sixteen) four
//     fifths of the CU's L1 time and the L1 the bound of the launch.  k_kv_tile_arrange therefore also writes the
//     visible K rows once per launch in operand order, [KV head][tile][32-dim step][16-row half][lane], and a
//     K load is 1 KB of consecutive memory like a V load;  The result leaves lane (query l % 16, g = l / 16) with cache rows 4g..4g+3 of
//     both 16-row halves of the tile: all eight values of a lane belong to ONE query, so the softmax statistics
//     are one (max, sum) pair per lane and the row maximum needs two cross-lane steps;
//   * that is also the A-operand layout of P . V with the contraction index (g, j) standing for cache row
//     4g + j (j < 4) or 16 + 4g + j - 4: P goes into the second product as it is (hi + lo fp16, so its products
//     with the fp16 values are exact), no transposition;
//   * the B operand of P . V needs eight cache ROWS per lane at one dim.  k_kv_tile_arrange writes the visible
//     part of the fp16 V cache once per launch into a scratch laid out [KV head][tile][16-dim block][g][dim][8 rows]
//     so that this operand is one 16-byte load, too (rows past the end: zeros);
//   * no LDS and no barrier in the walk: the accumulators (queries 4g..4g+3 x dim l % 16 per 16-dim block) are
//     rescaled only in tiles where some query's maximum moved, the factors fetched across lanes.
// Workgroup b serves head quad b % (H / 4): with eight KV heads, XCD x (workgroups x, x + 8, ...) walks the cache of
// KV head x only, which fits its L2; the token tiles with the longest walks come first.
typedef _Float16 h8p_t __attribute__((ext_vector_type(8)));
typedef float f4pu_t __attribute__((ext_vector_type(4), aligned(4)));
struct AttpVt { uint32_t grp[ATTP_MAX_HEADS]; };   // head -> index of its KV head's part of the transposed scratch
struct AttpVtSrc { uint32_t vb[ATTP_MAX_HEADS], kb[ATTP_MAX_HEADS]; };  // group -> bases of its V and K cache (element offsets in the map)

template <int D>
__global__ void __launch_bounds__(256)
k_kv_tile_arrange(const __half* kv, uint64_t kv_shift, const AttpVtSrc src, uint32_t nkeys, uint32_t tiles, uint4* vt, uint4* kt) {
  constexpr uint32_t NB = D / 16, KS = D / 32;
  const uint32_t T = blockIdx.x, grp = blockIdx.y;
  const unsigned short* v = (const unsigned short*)(kv + ((uint64_t)src.vb[grp] - kv_shift));
  for (uint32_t idx = threadIdx.x; idx < NB * 64u; idx += 256u) {
    const uint32_t b = idx >> 6, g = (idx >> 4) & 3u, n = idx & 15u;
    uint32_t w[4];
#pragma unroll
    for (uint32_t j = 0; j < 8; j++) {
      const uint32_t key = 32u * T + (j < 4u ? 4u * g + j : 16u + 4u * g + (j - 4u));
      const uint32_t x = key < nkeys ? (uint32_t)v[(uint64_t)key * D + 16u * b + n] : 0u;
      if (j & 1u) w[j >> 1] |= x << 16; else w[j >> 1] = x;
    }
    vt[((((uint64_t)grp * tiles + T) * NB + b) * 4u + g) * 16u + n] = make_uint4(w[0], w[1], w[2], w[3]);
  }
  // K: piece (step st, half kb, lane (g, n)) = dims 32 st + 8 g .. + 7 of row 32 T + 16 kb + n (rows past the end: zeros)
  const uint4* k = (const uint4*)(kv + ((uint64_t)src.kb[grp] - kv_shift));
  for (uint32_t idx = threadIdx.x; idx < 2u * KS * 64u; idx += 256u) {
    const uint32_t st = idx >> 7, kb = (idx >> 6) & 1u, g = (idx >> 4) & 3u, n = idx & 15u;
    const uint32_t key = 32u * T + 16u * kb + n;
    kt[((uint64_t)grp * tiles + T) * (2u * KS * 64u) + idx] =
        key < nkeys ? k[(uint64_t)key * (D / 8) + 4u * st + g] : make_uint4(0u, 0u, 0u, 0u);
  }
}

#define ATTP_MFMA32(a, b, c) __builtin_amdgcn_mfma_f32_16x16x32_f16(a, b, c, 0, 0, 0)

template <int D, bool CAP, int WPH>
__global__ void __launch_bounds__(256 * WPH)
k_attn_prefill_mfma(const float* data, float* out, const uint4* __restrict__ kt, const uint4* __restrict__ vt,
                    const AttpBases bs, const AttpVt gv, uint32_t H, uint32_t n_quads, uint32_t n_ttiles, uint32_t m,
                    uint32_t seq0, uint32_t q_stride, uint32_t o_stride, float scale, float cap, uint32_t vt_tiles) {
  constexpr int KS = D / 32;           // 32-dim steps of the score product
  constexpr int NB = D / 16;           // 16-dim blocks of the output
  const uint32_t lane = threadIdx.x & 63u;
  const uint32_t wave = (uint32_t)__builtin_amdgcn_readfirstlane((int)(threadIdx.x >> 6));
  const uint32_t n = lane & 15u, g = lane >> 4;
  // WPH = 2 (a launch that gives every CU one workgroup at most): two waves per head, the second four waves of the
  // workgroup walk the second half of the key tiles and hand their running state over in LDS at the end -- two waves
  // per SIMD, so that one's loads are served while the other one multiplies.
  const uint32_t half = WPH == 2 ? wave >> 2 : 0u;
  const uint32_t head_raw = (blockIdx.x % n_quads) * 4u + (wave & 3u);
  const bool live = head_raw < H;
  if (WPH == 1 && !live) return;       // (no barrier in the one-wave form)
  const uint32_t head = min(head_raw, H - 1u);
  const uint32_t t0 = (n_ttiles - 1u - blockIdx.x / n_quads) * 16u;
  const uint32_t rows = min(16u, m - t0);
  const uint32_t nkeys = seq0 + t0 + rows - 1u;          // cache rows the tile's last query sees
  const uint32_t n_tiles = (nkeys + 31u) >> 5;
  const uint32_t t_split = WPH == 2 ? (n_tiles + 1u) >> 1 : n_tiles;
  const uint32_t T_lo = !live ? 0u : half ? t_split : 0u, T_hi = !live ? 0u : half ? n_tiles : t_split;
  const uint4* kbase = kt + (uint64_t)gv.grp[head] * vt_tiles * (2u * KS * 64u) + lane;
  const uint4* vbase = vt + (uint64_t)gv.grp[head] * vt_tiles * (NB * 64u) + g * 16u + n;

  // this lane's query (n): dims 32 step + 8g .. + 7, scaled by a power of two into fp16 range, hi + lo
  h8p_t qh[KS], ql[KS];
  float inv_s;
  {
    float x[KS][8], mx = 0.f;
    const float* qp = data + (uint64_t)bs.q[head] + (uint64_t)(t0 + min(n, rows - 1u)) * q_stride + 8u * g;
#pragma unroll
    for (int st = 0; st < KS; st++) {
      const f4pu_t a = *(const f4pu_t*)(qp + 32 * st), b = *(const f4pu_t*)(qp + 32 * st + 4);
      x[st][0] = a.x; x[st][1] = a.y; x[st][2] = a.z; x[st][3] = a.w; x[st][4] = b.x; x[st][5] = b.y; x[st][6] = b.z; x[st][7] = b.w;
#pragma unroll
      for (int t = 0; t < 8; t++) { if (n >= rows) x[st][t] = 0.f; mx = fmaxf(mx, fabsf(x[st][t])); }
    }
    mx = fmaxf(mx, __shfl_xor(mx, 16, 64)); mx = fmaxf(mx, __shfl_xor(mx, 32, 64));
    const uint32_t e = (__float_as_uint(mx) >> 23) & 0xFFu;
    float s = 1.f;
    inv_s = 1.f;
    if (e >= 14u && e <= 254u) { s = __uint_as_float((267u - e) << 23); inv_s = __uint_as_float((e - 13u) << 23); }
#pragma unroll
    for (int st = 0; st < KS; st++)
#pragma unroll
      for (int t = 0; t < 8; t++) {
        const float xs = x[st][t] * s;
        const _Float16 hi = (_Float16)xs;
        qh[st][t] = hi;
        ql[st][t] = (_Float16)(xs - (float)hi);
      }
  }
  const uint32_t lim = n < rows ? seq0 + t0 + n : 0u;     // cache rows this lane's query sees
  const float c2 = inv_s * scale * 1.44269504f;          // (inv_s is a power of two)
  const bool last = live && n < rows && t0 + n == m - 1u;
  const uint64_t sc_row = bs.sc[head];

  f4p_t acc[NB];
#pragma unroll
  for (int b = 0; b < NB; b++) acc[b] = (f4p_t){0.f, 0.f, 0.f, 0.f};
  float m_run = ATTP_NEG, l_run = 0.f;

  struct Tile { uint4 k[2][KS]; uint4 v[NB]; };
  auto fetch = [&](Tile& t, uint32_t T) {
#pragma unroll
    for (int kb = 0; kb < 2; kb++)
#pragma unroll
      for (int st = 0; st < KS; st++) t.k[kb][st] = kbase[((uint64_t)T * (2 * KS) + 2 * st + kb) * 64u];
#pragma unroll
    for (int b = 0; b < NB; b++) t.v[b] = vbase[((uint64_t)T * NB + b) * 64u];
  };
  // One tile's arithmetic, with the loads of tile Tn (into nx) spread between its matrix instructions, one 16-byte
  // load per lane in front of every pair: a wave issues in order, and sixteen loads in a row ahead of the arithmetic
  // keep it at its load instructions for as long as the CU's one address unit, shared by the four waves, takes to
  // accept them (16 clocks each: ~1000 clocks per tile during which no wave of the CU multiplies).
  auto compute = [&](const Tile& t, uint32_t T, Tile& nx, uint32_t Tn) {
    f4p_t s[2][2];
#pragma unroll
    for (int kb = 0; kb < 2; kb++) { s[kb][0] = (f4p_t){0.f, 0.f, 0.f, 0.f}; s[kb][1] = s[kb][0]; }
    const uint4* kn = kbase + (uint64_t)Tn * (2 * KS) * 64u;
    const uint4* vn = vbase + (uint64_t)Tn * NB * 64u;
#pragma unroll
    for (int st = 0; st < KS; st++)
#pragma unroll
      for (int kb = 0; kb < 2; kb++) {
        nx.k[kb][st] = kn[(2 * st + kb) * 64];
        __builtin_amdgcn_sched_barrier(0);
        const h8p_t ka = __builtin_bit_cast(h8p_t, t.k[kb][st]);
        s[kb][0] = ATTP_MFMA32(ka, qh[st], s[kb][0]);
        s[kb][1] = ATTP_MFMA32(ka, ql[st], s[kb][1]);
        __builtin_amdgcn_sched_barrier(0);
      }
    // The softmax runs on base-2 exponents: without a soft cap the scores' power-of-two scale, the softmax scale and
    // log2(e) are one factor (one rounding, as scale alone would take), a masked score is a large negative number
    // whose power is exactly 0, and the only branches of a tile are wave-uniform and rarely taken (the raw scores
    // of the chunk's last token, a maximum that moved).
    float v[8], mt = ATTP_NEG;
    const uint32_t key0 = 32u * T + 4u * g;
#pragma unroll
    for (int kb = 0; kb < 2; kb++)
#pragma unroll
      for (int r = 0; r < 4; r++) {
        const float sum = s[kb][0][r] + s[kb][1][r];
        const float x = CAP ? prep(sum * inv_s, scale, cap) * 1.44269504f : sum * c2;
        v[4 * kb + r] = key0 + 16u * kb + r < lim ? x : ATTP_NEG;
        mt = fmaxf(mt, v[4 * kb + r]);
      }
    if (__builtin_expect(__any(last), 0)) {
#pragma unroll
      for (int kb = 0; kb < 2; kb++)
#pragma unroll
        for (int r = 0; r < 4; r++) {
          const uint32_t key = key0 + 16u * kb + r;
          if (key < lim && last) out[sc_row + key] = (s[kb][0][r] + s[kb][1][r]) * inv_s;
        }
    }
    mt = fmaxf(mt, __shfl_xor(mt, 16, 64)); mt = fmaxf(mt, __shfl_xor(mt, 32, 64));
    const float m_new = fmaxf(m_run, mt);
    const float alpha = __builtin_amdgcn_exp2f(m_run - m_new);
    const bool moved = m_new > m_run;
    m_run = m_new;
    h8p_t ph, pl;
    float psum = 0.f;
#pragma unroll
    for (int j = 0; j < 8; j++) {
      const float pj = __builtin_amdgcn_exp2f(v[j] - m_new);
      psum += pj;
      const _Float16 hi = (_Float16)pj;
      ph[j] = hi;
      pl[j] = (_Float16)(pj - (float)hi);
    }
    l_run = l_run * alpha + psum;
    if (__builtin_expect(__any(moved), 0)) {   // wave-uniform: most tiles after the first few leave every maximum where it was
      float a4[4];
#pragma unroll
      for (int r = 0; r < 4; r++) a4[r] = __shfl(alpha, (int)(4u * g + r), 64);
#pragma unroll
      for (int b = 0; b < NB; b++)
#pragma unroll
        for (int r = 0; r < 4; r++) acc[b][r] *= a4[r];
    }
#pragma unroll
    for (int b = 0; b < NB; b++) {
      nx.v[b] = vn[b * 64];
      __builtin_amdgcn_sched_barrier(0);
      const h8p_t vb = __builtin_bit_cast(h8p_t, t.v[b]);
      acc[b] = ATTP_MFMA32(ph, vb, acc[b]);
      acc[b] = ATTP_MFMA32(pl, vb, acc[b]);
      __builtin_amdgcn_sched_barrier(0);
    }
  };

  Tile A, B;
  if (T_lo < T_hi) fetch(A, T_lo);
  for (uint32_t T = T_lo; T < T_hi; T += 2u) {
    compute(A, T, B, min(T + 1u, T_hi - 1u));            // (past the end: the last tile again, not used)
    if (T + 1u >= T_hi) break;
    compute(B, T + 1u, A, min(T + 2u, T_hi - 1u));
  }

  if (WPH == 2) {
    // the second wave of a head hands (maximum, sum, accumulators) to the first, which merges: both rescaled to the
    // common maximum (a wave without tiles hands over maximum -1e30, sum 0: factor exactly 0)
    __shared__ float xch[4 * (2 + 4 * NB) * 64];
    float* mine = xch + (wave & 3u) * ((2 + 4 * NB) * 64) + lane;
    if (half) {
      mine[0] = m_run; mine[64] = l_run;
#pragma unroll
      for (int b = 0; b < NB; b++)
#pragma unroll
        for (int r = 0; r < 4; r++) mine[(2 + 4 * b + r) * 64] = acc[b][r];
    }
    __syncthreads();
    if (half || !live) return;
    const float m1 = mine[0], l1 = mine[64];
    const float mm = fmaxf(m_run, m1);
    const float f0 = __builtin_amdgcn_exp2f(m_run - mm), f1 = __builtin_amdgcn_exp2f(m1 - mm);
    l_run = l_run * f0 + l1 * f1;
    float g0[4], g1[4];
#pragma unroll
    for (int r = 0; r < 4; r++) { g0[r] = __shfl(f0, (int)(4u * g + r), 64); g1[r] = __shfl(f1, (int)(4u * g + r), 64); }
#pragma unroll
    for (int b = 0; b < NB; b++)
#pragma unroll
      for (int r = 0; r < 4; r++) acc[b][r] = acc[b][r] * g0[r] + mine[(2 + 4 * b + r) * 64] * g1[r];
  }

  float l_tot = l_run + __shfl_xor(l_run, 16, 64);
  l_tot += __shfl_xor(l_tot, 32, 64);
  const float inv_l = 1.0f / l_tot;
  float il[4];
#pragma unroll
  for (int r = 0; r < 4; r++) il[r] = __shfl(inv_l, (int)(4u * g + r), 64);
#pragma unroll
  for (int r = 0; r < 4; r++) {
    const uint32_t qr = 4u * g + r;
    if (qr >= rows) continue;
    float* dst = out + (uint64_t)bs.o[head] + (uint64_t)(t0 + qr) * o_stride + n;
#pragma unroll
    for (int b = 0; b < NB; b++) dst[16 * b] = acc[b][r] * il[r];
  }
}

// transposed V tiles of the chunk launches: grown on demand, released at shutdown
static uint4* g_vt = nullptr;
static size_t g_vt_bytes = 0;
void attn_prefill_release() {
  if (g_vt) hipFree(g_vt);
  g_vt = nullptr; g_vt_bytes = 0;
}

static bool disjoint_iv(uint64_t a0, uint64_t a1, uint64_t b0, uint64_t b1) { return a1 <= b0 || b1 <= a0; }

// The run of (scores, softmax . V) pairs that starts at q[i]: launches it as one chunk and returns the
// number of queue entries consumed, or 0 when the entries do not form such a run (nothing launched).
size_t launch_attn_chunk(const std::vector<PendOp>& q, size_t i, int* rc) {
  *rc = ADAMAH_OK;
  if (tuning("ADAMAH_ATTN_CHUNK", 1) == 0) return 0;
  const size_t n = q.size();
  if (i + 3 >= n || !attn_foldable(q[i], q[i + 1])) return 0;
  const PendOp &s0 = q[i], &a0 = q[i + 1];
  // cheap way out first: the next token sees one more row of the same cache
  if (q[i + 2].kind != PK_SCORES || q[i + 3].kind != PK_ATTN || q[i + 2].n != s0.n + 1 || q[i + 2].h[0] == s0.h[0]) return 0;
  Map* mp = get_f32_map(a0.map_act);
  const uint32_t H = a0.rpg, D = a0.k;
  if (!mp || !mp->kv16 || H == 0 || H > ATTP_MAX_HEADS || s0.k != D || (D != 64 && D != 128 && D != 256)) return 0;
  const uint32_t *q0 = res_host(s0.h[0], H), *kb = res_host(s0.h[1], H), *sc = res_host(s0.h[2], H);
  const uint32_t *vb = res_host(a0.h[1], H), *o0 = res_host(a0.h[2], H);
  if (!q0 || !kb || !sc || !vb || !o0) return 0;
  // tokens 1 .. m-1: same cache, score rows and parameters, one more visible row each, query and output
  // rows moved by a fixed stride
  uint32_t m = 1, qs = 0, os = 0;
  while (i + 2 * m + 1 < n) {
    const PendOp &st = q[i + 2 * m], &at = q[i + 2 * m + 1];
    if (!attn_foldable(st, at) || st.map_act != s0.map_act || st.rpg != H || at.k != D || st.k != D ||
        st.n != s0.n + m || at.eps != a0.eps || at.f2 != a0.f2)
      break;
    const uint32_t *qt = res_host(st.h[0], H), *kt = res_host(st.h[1], H), *ct = res_host(st.h[2], H);
    const uint32_t *vt = res_host(at.h[1], H), *ot = res_host(at.h[2], H);
    if (!qt || !kt || !ct || !vt || !ot) break;
    if (m == 1) { qs = qt[0] - q0[0]; os = ot[0] - o0[0]; }
    bool same = qt[0] > q0[0] && ot[0] > o0[0];
    for (uint32_t h = 0; same && h < H; h++)
      same = kt[h] == kb[h] && vt[h] == vb[h] && ct[h] == sc[h] && qt[h] == q0[h] + m * qs && ot[h] == o0[h] + m * os;
    if (!same) break;
    m++;
  }
  if (m < 2) return 0;
  // every K / V base inside the fp16 copy on a 16-byte boundary (the queued ops were checked one by
  // one; the copy's alignment is what the 16-byte loads of this kernel need)
  const uint32_t seq_last = s0.n + m - 1;
  for (uint32_t h = 0; h < H; h++) {
    if (kb[h] < mp->kv_start || vb[h] < mp->kv_start || (kb[h] - mp->kv_start) % 8u || (vb[h] - mp->kv_start) % 8u) return 0;
    if ((uint64_t)kb[h] - mp->kv_start + (uint64_t)seq_last * D > mp->kv_count ||
        (uint64_t)vb[h] - mp->kv_start + (uint64_t)seq_last * D > mp->kv_count)
      return 0;
  }
  // The launch reads all queries before or while it writes outputs and scores: none of what it writes
  // may overlap what it reads, nor another token's output.
  uint64_t qlo = ~0ull, qhi = 0, olo = ~0ull, ohi = 0;
  for (uint32_t h = 0; h < H; h++) {
    qlo = std::min<uint64_t>(qlo, q0[h]); qhi = std::max<uint64_t>(qhi, (uint64_t)q0[h] + (uint64_t)(m - 1) * qs + D);
    olo = std::min<uint64_t>(olo, o0[h]); ohi = std::max<uint64_t>(ohi, (uint64_t)o0[h] + (uint64_t)(m - 1) * os + D);
  }
  if (qhi > mp->n_elems || ohi > mp->n_elems || os < D) return 0;
  if (!disjoint_iv(qlo, qhi, olo, ohi)) return 0;
  const uint64_t kv0 = mp->kv_start, kv1 = mp->kv_start + mp->kv_count;
  if (!disjoint_iv(olo, ohi, kv0, kv1)) return 0;
  for (uint32_t h = 0; h < H; h++) {
    const uint64_t s_lo = sc[h], s_hi = (uint64_t)sc[h] + seq_last;
    if (!disjoint_iv(s_lo, s_hi, qlo, qhi) || !disjoint_iv(s_lo, s_hi, olo, ohi) || !disjoint_iv(s_lo, s_hi, kv0, kv1)) return 0;
    for (uint32_t h2 = 0; h2 < h; h2++)        // output rows of different heads must not collide within a token
      if (!disjoint_iv(o0[h], (uint64_t)o0[h] + D, o0[h2], (uint64_t)o0[h2] + D)) return 0;
  }
  AttpBases bs;
  for (uint32_t h = 0; h < H; h++) { bs.q[h] = q0[h]; bs.sc[h] = sc[h]; bs.o[h] = o0[h]; bs.kb[h] = kb[h]; bs.vb[h] = vb[h]; }
  float* d = (float*)mp->buf;
  // Both products on the matrix cores (a wave per head and 16-token tile) when that gives at least half the CUs a
  // workgroup; a chunk with few heads or few tokens (Gemma-3-1B: 4 heads, 32 workgroups for 512 tokens) spreads wider on
  // the kernel above, whose workgroups are one head each and split the cache between their waves.
  // ADAMAH_ATTN_PREFILL_MFMA: 0 never, 1 by that rule (default), 2 always.
  const int mfma_mode = tuning("ADAMAH_ATTN_PREFILL_MFMA", 1);
  if (mfma_mode == 2 || (mfma_mode == 1 && cdiv(H, 4u) * cdiv(m, 16u) * 2u >= (uint32_t)g.n_cu)) {
    // the visible V rows of every KV head transposed into tiles first
    AttpVt gv; AttpVtSrc src;
    uint32_t n_grp = 0;
    for (uint32_t h = 0; h < H; h++) {
      uint32_t gi = 0;
      while (gi < n_grp && (src.vb[gi] != vb[h] || src.kb[gi] != kb[h])) gi++;
      if (gi == n_grp) { src.vb[n_grp] = vb[h]; src.kb[n_grp++] = kb[h]; }
      gv.grp[h] = gi;
    }
    const uint32_t tiles = cdiv(seq_last, 32u);
    const size_t plane = (size_t)n_grp * tiles * 32u * D * sizeof(__half);   // V tiles, then K tiles
    const size_t need = 2 * plane;
    bool ok = true;
    if (need > g_vt_bytes) {
      hipStreamSynchronize(g.stream);
      if (g_vt) hipFree(g_vt);
      g_vt = nullptr; g_vt_bytes = 0;
      const size_t want = std::max(need + need / 2, (size_t)8 << 20);
      if (hipMalloc((void**)&g_vt, want) == hipSuccess) g_vt_bytes = want;
      else { (void)hipGetLastError(); ok = false; }
      layout_changed();
    }
    if (ok) {
      const uint32_t n_quads = cdiv(H, 4u), n_tt = cdiv(m, 16u);
      uint4* const g_kt = (uint4*)((char*)g_vt + plane);
      // two waves per head where the launch has at most one workgroup per CU (ADAMAH_ATTN_PREFILL_WPH: 1 / 2 force)
      const int wph_mode = tuning("ADAMAH_ATTN_PREFILL_WPH", 0);
      const int wph = wph_mode == 1 || wph_mode == 2 ? wph_mode : (n_quads * n_tt <= (uint32_t)g.n_cu ? 2 : 1);
#define APM_ARGS d, d, g_kt, g_vt, bs, gv, H, n_quads, n_tt, m, s0.n, qs, os, a0.eps, a0.f2, tiles
#define APM(DD)                                                                                                   \
  do {                                                                                                            \
    k_kv_tile_arrange<DD><<<dim3(tiles, n_grp), 256, 0, g.stream>>>(mp->kv16, mp->kv_start, src, seq_last, tiles, g_vt, g_kt); \
    const dim3 gr_(n_quads * n_tt);                                                                               \
    if (wph == 2 && DD <= 128) {   /* (D = 256 needs more registers than two waves per SIMD have) */              \
      constexpr int D2_ = DD <= 128 ? DD : 128;                                                                   \
      if (a0.f2 > 0.0f) k_attn_prefill_mfma<D2_, true, 2><<<gr_, 512, 0, g.stream>>>(APM_ARGS);                  \
      else k_attn_prefill_mfma<D2_, false, 2><<<gr_, 512, 0, g.stream>>>(APM_ARGS);                              \
    } else {                                                                                                      \
      if (a0.f2 > 0.0f) k_attn_prefill_mfma<DD, true, 1><<<gr_, 256, 0, g.stream>>>(APM_ARGS);                   \
      else k_attn_prefill_mfma<DD, false, 1><<<gr_, 256, 0, g.stream>>>(APM_ARGS);                               \
    }                                                                                                             \
  } while (0)
      if (D == 64) APM(64); else if (D == 128) APM(128); else APM(256);
#undef APM
#undef APM_ARGS
      count_launch(2);
      *rc = check_launch();
      return 2 * (size_t)m;
    }
  }
  dim3 grid(cdiv(m, 16u), H);
#define APL(DD, NW) k_attn_prefill<DD, NW><<<grid, NW * 64, 0, g.stream>>>(d, d, mp->kv16, mp->kv_start, bs, m, s0.n, qs, os, a0.eps, a0.f2)
  if (D == 64) APL(64, 4); else if (D == 128) APL(128, 4); else APL(256, 2);
#undef APL
  count_launch();
  *rc = check_launch();
  return 2 * (size_t)m;
}

}  // namespace adamah
