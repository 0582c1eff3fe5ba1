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
  dim3 grid(cdiv(m, 16u), H);
#define APL(DD, NW) k_attn_prefill<DD, NW><<<grid, NW * 64, 0, g.stream>>>(d, d, mp->kv16, mp->kv_start, bs, m, s0.n, qs, os, a0.eps, a0.f2)
  if (D == 64) APL(64, 4); else if (D == 128) APL(128, 4); else APL(256, 2);
#undef APL
  count_launch();
  *rc = check_launch();
  return 2 * (size_t)m;
}

}  // namespace adamah
