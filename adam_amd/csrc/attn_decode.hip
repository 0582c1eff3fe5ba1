// Grouped decode attention: scores and softmax . V of one token for all query heads that share a
// KV head, in one pass over the fp16 K and V rows.
//
// Reference: the pair map_matmul_t_dev (scores, shaders/src/f32/map_matmul_t.comp) and
// map_attn_softmax_value_dev (map_attn_softmax_value.comp:39-89; dispatch adamah.c:6682-6781,
// 7894-8059) as the decode loop issues them (adam/models/engine.py:2428-2441 for the arithmetic).
// The reference runs one workgroup per query head, so every KV row is fetched once per head of its
// group and twice more through the score row; here a workgroup owns (KV head, slice of the sequence)
// and reads each K and V row once for the whole group.
//
// Workgroup = NW (4 or 8) waves; a wave takes 16-row tiles of the slice.  Per tile a lane issues its K and V
// loads together (16 bytes each, rows contiguous across lanes), then
//   scores  v_mfma_f32_16x16x16_f16 with A = queries (matrix row = head, zero beyond the group) and
//           B = K tile (column = row of the tile).  The queries are scaled per head by a power of two
//           into fp16 range and split into a high and a low fp16 part, so the products are exact and
//           the sum is fp32: the raw scores stored to the score rows match a float32 dot product.
//   softmax online per wave (running maximum m, sum l), weights handed to the V phase through LDS
//   values  every lane owns D/64 dims of the output and sees all 16 rows of the tile: fp32 FMAs, one
//           accumulator set per head of the group, no reduction across lanes.
// With more than one tile per wave (PF) the next tile's loads are issued before the current tile's
// arithmetic (two register sets).  The queries reach the lanes through LDS, so their rows need no
// alignment.  The waves merge through LDS; slices merge through partials (m, l, o[D]) per head and slice, by
// the consumer when they are few, else by the merge kernel.  (A merge by the last workgroup to
// finish, found with an atomic ticket, needs a device-scope release and acquire in every workgroup;
// each of those writes back and invalidates the L2 of its XCD and the kernel got 4x slower.)
#include "attn_common.h"
#include "gemv_common.h"
#include <algorithm>
#include <string.h>
#include <utility>
#include <vector>

namespace adamah {

typedef _Float16 h4a_t __attribute__((ext_vector_type(4)));
typedef float f4a_t __attribute__((ext_vector_type(4)));
typedef uint32_t u2a_t __attribute__((ext_vector_type(2)));


#define ATTD_NEG (-1.0e30f)
#define ATTD_MAX_SPLITS 256u
#define ATTD_MAX_GROUPS 128u

// Operand bases by value (the handles' host copies): saves a dependent load before the first K row.
#define ATTD_MAX_OPS 64u
struct AttdBases { uint32_t q[ATTD_MAX_OPS], sc[ATTD_MAX_OPS], o[ATTD_MAX_OPS], kb[ATTD_MAX_OPS], vb[ATTD_MAX_OPS]; };

// Row preparation done by the attention launch itself (RP): the rotation (after the optional per-head RMSNorm) of
// the token's new Q and K rows and the append of its K and V rows to the cache, which otherwise are a launch of
// their own just before (rowprep.hip; same arithmetic in the same order, so the results are the same bits).
// Every workgroup of a KV head prepares the group's queries for itself from the raw rows; the workgroup that
// owns the last slice of the sequence also prepares the new K and V rows, stores them to the cache (float32 row
// and fp16 copy) and uses them from LDS in place of the cache row it loaded.  The prepared queries usually go back
// over the raw ones, which other workgroups of the group may not have read yet.  With one slice they are stored
// at once; with more, the first slice's workgroup puts them into scratch memory and the launch that merges the
// slices (the merge kernel, or the GEMV that merges while staging) copies them to their place.  (Counting the
// workgroups in with an atomic and letting the last one store cost 2 us per launch: the atomic's reply comes back
// in order with the wave's K / V tiles, which then wait for the contended counter.)
struct AttdRowPrep {
  uint32_t flags;                        // 1 = RMSNorm (eps 1e-6) before the rotation
  uint32_t pos;                          // position the rotation is for; the new cache row is row_size - 1
  float base;
  uint32_t q_src, k_src, k_dst, v_src;   // element offsets: head h of Q at q_src + h D, KV head g at k_src + g D, ...;
                                         // k_dst = ROWT_NONE: the rotated K row goes to the cache only
  uint32_t q_w, k_w;                     // norm weights (flags & 1)
  float* q_scratch;                      // n_splits > 1: the prepared queries, head h at q_scratch + h D
  const float* inv_freq;                 // 1 / base^(2i/D) for i < D/2, as the stand-alone rotation computes it
};

#define ATTD_DPP(v, ctrl) __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), ctrl, 0xF, 0xF, false))
// all-reduce over each 16-lane row: quad_perm [1,0,3,2], [2,3,0,1], row_half_mirror, row_mirror
__device__ __forceinline__ float row16_max(float v) {
  v = fmaxf(v, ATTD_DPP(v, 0xB1)); v = fmaxf(v, ATTD_DPP(v, 0x4E));
  v = fmaxf(v, ATTD_DPP(v, 0x141)); v = fmaxf(v, ATTD_DPP(v, 0x140));
  return v;
}
__device__ __forceinline__ float row16_sum(float v) {
  v += ATTD_DPP(v, 0xB1); v += ATTD_DPP(v, 0x4E); v += ATTD_DPP(v, 0x141); v += ATTD_DPP(v, 0x140);
  return v;
}

template <int D, int G, int NW, bool PF, bool EXT, bool RP>
__global__ void __launch_bounds__(NW * 64)
k_attn_decode(const float* data, const __half* kv, uint64_t kv_shift, uint32_t row_size, uint32_t chunk, uint32_t splits_share,
              uint32_t rp_q_src, uint32_t rp_k_src, uint32_t rp_v_src, const void* early_ptr,
              float* out, float scale, float cap, float* partial, const AttdBases bs, const AttdRowPrep rp) {
  // splits_share = slices | log2(share) << 16.  share > 1: the launch's groups are narrower than the KV groups --
  // `share` consecutive groups of G heads read the same K / V rows (a short launch spread over more workgroups, each
  // with fewer heads to work through between its barriers); with the row preparation they share one raw K / V row,
  // every one of them prepares it for its own use and the first of them stores it to the cache.
  const uint32_t n_splits = splits_share & 0xFFFFu, share_log = splits_share >> 16;
  // (the first 14 dwords of the arguments are in registers when a wave starts: what the first loads need stands in
  // front -- with the row preparation the raw rows' places and the frequency table, copies of rp's fields; with
  // the operand bases in device memory, the table's address)
  const float* rp_inv_freq = (const float*)early_ptr;
  const uint32_t* __restrict__ ext = (const uint32_t*)early_ptr;
  constexpr int NI = D / 32;           // 16-byte K loads per lane and tile
  constexpr int DPL = D / 64;          // V dims per lane (every lane sees all 16 rows of the tile)
  constexpr int DW = DPL > 2 ? DPL / 2 : 1;
  constexpr uint32_t NT = NW * 64;     // threads
  __shared__ float pbuf[NW][16][G];    // softmax weights of the wave's tile, [row][head]
  __shared__ float abuf[NW][G];        // per head: rescale factor of the tile
  __shared__ float obuf[NW][G][D];     // wave results; first the queries of the group, [head][dim]
  __shared__ float mlbuf[NW][G][2];
  __shared__ h4a_t qop[2 * NI][2][64]; // query operands of the matrix product: [k-step][hi, lo][lane]
  __shared__ uint32_t hmax[G];         // per head: bits of max |q|
  __shared__ float qinv[G];            // per head: 1 / (power-of-two scale of the queries)
  // RP: sums of squares per 64 elements of the raw Q rows and of the raw K row; the new K and V rows as fp16
  __shared__ float ssq[RP ? G * D / 64 : 1], ssk[RP ? D / 64 : 1], kraw_s[RP ? D : 1];
  __shared__ __attribute__((aligned(16))) __half knew[RP ? D : 8], vnew[RP ? D : 8];

  const uint32_t tid = threadIdx.x, lane = tid & 63u;
  const uint32_t wave = (uint32_t)__builtin_amdgcn_readfirstlane((int)(tid >> 6));   // scalar: row numbers below are too
  const uint32_t c = lane & 15u, kc = lane >> 4;
  const uint32_t split = blockIdx.x, group = blockIdx.y, op0 = group * G;
  const uint32_t kvg = group >> share_log;                          // RP: index of the raw K / V row
  const bool kv_writer = (group & ((1u << share_log) - 1u)) == 0u;  // RP: stores the new rows to the cache
  const uint32_t t0 = split * chunk, t1 = min(row_size, t0 + chunk);
  // wave-uniform bases plus 32-bit byte offsets: the V row of a load is the same for all lanes
  // EXT (several sets of heads in one launch, too many for the argument block): the bases come from
  // device memory as [q | score rows | out rows] per head, then [K | V] per group; a score row of
  // 0xFFFFFFFF is not stored.
  const uint32_t n_all = gridDim.y * (uint32_t)G;
  const uint32_t *e_q = ext, *e_sc = ext + n_all, *e_o = ext + 2u * n_all, *e_kb = ext + 3u * n_all, *e_vb = e_kb + gridDim.y;
  // (set where the first tile is asked for: with the row preparation the bases come from the part of the argument
  // block that is not in registers at the start, and the raw rows' loads go out before anything waits for it)
  const char *kbase = nullptr, *vbase = nullptr;
  const uint32_t kb_g = EXT ? e_kb[group] : bs.kb[group], vb_g = EXT ? e_vb[group] : bs.vb[group];   // asked for here
  auto set_bases = [&]() {                                                                           // waited for here
    kbase = (const char*)(kv + ((uint64_t)kb_g - kv_shift));
    vbase = (const char*)(kv + ((uint64_t)vb_g - kv_shift));
  };
  if (!RP) set_bases();
  const uint32_t klane = 16u * kc, vlane = 2u * (uint32_t)DPL * lane;

  auto fetch = [&](uint4 (&kr)[NI], uint32_t (&vr)[16][DW], uint32_t rb) {
    const uint32_t koff = min(rb + c, t1 - 1u) * (2u * D) + klane;
#pragma unroll
    for (int i = 0; i < NI; i++) kr[i] = *(const uint4*)(kbase + koff + 64u * i);
#pragma unroll
    for (int u = 0; u < 16; u++) {
      const char* src = vbase + (uint64_t)(min(rb + u, t1 - 1u) * (2u * D)) + vlane;
      if (DPL == 1) vr[u][0] = *(const uint16_t*)src;
      else if (DPL == 2) vr[u][0] = *(const uint32_t*)src;
      else { const uint2 t = *(const uint2*)src; vr[u][0] = t.x; vr[u][DW - 1] = t.y; }
    }
  };

  // Queries: coalesced scalar loads into LDS (obuf[0] is free until the end) with the per-head
  // maximum on the way; then the first tile's K and V loads go out; then the matrix-A operands (lane
  // (head c, kc) of operand 2i+j: dims 32i + 8kc + 4j .. +3 of head c, zero beyond the group), scaled
  // by 2^e into [2^13, 2^14) and split hi + lo, are written to LDS once for all waves.
  uint4 kA[NI], kB[NI];
  uint32_t vA[16][DW], vB[16][DW];
  uint32_t rbase = t0 + wave * 16u;
  const bool any = rbase < t1;
  constexpr uint32_t QN = ((uint32_t)(G * D) + NT - 1u) / NT;        // query elements per thread
  constexpr uint32_t PN = ((uint32_t)(G * D) / 2u + NT - 1u) / NT;   // RP: rotation pairs per thread
  const bool tail_wg = RP && split + 1u == n_splits;                 // RP: this workgroup owns the sequence's last row
  {
    float* qs = &obuf[0][0][0];
    if (tid < (uint32_t)G) hmax[tid] = 0u;
    if (!RP) {
      // the query loads go out first and are waited for first, with the first tile's loads already behind them
      // (every thread issues the same loads, at clamped addresses where it has no element of its own, so that the
      // compiler can count them: see the row preparation below)
      float qraw[QN];
#pragma unroll
      for (uint32_t u = 0; u < QN; u++) {
        const uint32_t i = min(tid + u * NT, (uint32_t)(G * D) - 1u), hq = i / D;   // a wave's 64 elements belong to one head
        qraw[u] = data[(uint64_t)(EXT ? e_q[op0 + hq] : bs.q[op0 + hq]) + i % D];
      }
      __builtin_amdgcn_sched_barrier(0);
      fetch(kA, vA, min(rbase, t1 - 1u));      // a wave without rows asks for the slice's last row: not used
      __builtin_amdgcn_sched_barrier(0);
      __syncthreads();                         // hmax is zero
#pragma unroll
      for (uint32_t u = 0; u < QN; u++) {
        const uint32_t i = tid + u * NT;
        if (i < (uint32_t)(G * D)) {
          qs[i] = qraw[u];
          float m = fabsf(qraw[u]);
#pragma unroll
          for (int o = 32; o > 0; o >>= 1) m = fmaxf(m, __shfl_xor(m, o, 64));
          if (lane == 0u) atomicMax(&hmax[i / D], __float_as_uint(m));
        }
      }
      __syncthreads();
    } else {
      constexpr uint32_t half = (uint32_t)D / 2u;
      // Raw rows first (they are waited for first), then what the rotation needs from memory (frequencies, norm
      // weights), then the first tile.  Every load below is issued by every thread, at an address clamped into its
      // row where the thread has no element of its own: with loads under branches the compiler no longer knows how
      // many are in flight and waited for all of them, K / V tile included, before the queries could be staged.
      float qraw[QN], kraw, vraw;
#pragma unroll
      for (uint32_t u = 0; u < QN; u++)
        qraw[u] = data[(uint64_t)rp_q_src + (uint64_t)op0 * D + min(tid + u * NT, (uint32_t)(G * D) - 1u)];
      {
        const uint32_t d = min(tid, (uint32_t)D - 1u);
        kraw = data[(uint64_t)rp_k_src + (uint64_t)kvg * D + d];
        vraw = data[(uint64_t)rp_v_src + (uint64_t)kvg * D + d];
      }
      float fr[PN], wq[PN][2], wk[2];
#pragma unroll
      for (uint32_t u = 0; u < PN; u++) fr[u] = rp_inv_freq[(tid + u * NT) % half];
      // Everything above is addressed from the arguments that are in registers when the wave starts; what follows
      // needs the rest of the argument block (a trip to memory), and the fence keeps that wait from being scheduled
      // in front of the raw rows' loads.
      __builtin_amdgcn_sched_barrier(0);
      set_bases();
      const bool nrm = (rp.flags & 1u) != 0u;
      {
        const float* wqp = nrm ? data + rp.q_w : rp_inv_freq;     // no norm: any readable address, the value is not used
        const float* wkp = nrm ? data + rp.k_w : rp_inv_freq;
        const uint32_t hs = nrm ? half : 0u;
#pragma unroll
        for (uint32_t u = 0; u < PN; u++) {
          const uint32_t i = (tid + u * NT) % half;
          wq[u][0] = wqp[i]; wq[u][1] = wqp[i + hs];
        }
        wk[0] = wkp[tid % half]; wk[1] = wkp[tid % half + hs];
      }
      __builtin_amdgcn_sched_barrier(0);
      fetch(kA, vA, min(rbase, t1 - 1u));      // a wave without rows asks for the slice's last row: not used
      __builtin_amdgcn_sched_barrier(0);
#pragma unroll
      for (uint32_t u = 0; u < QN; u++) {
        const uint32_t i = tid + u * NT;
        if (i < (uint32_t)(G * D)) {
          qs[i] = qraw[u];
          if (rp.flags & 1u) {
            float ss = fmaf(qraw[u], qraw[u], 0.f);
#pragma unroll
            for (int o = 32; o > 0; o >>= 1) ss += __shfl_xor(ss, o, 64);
            if (lane == 0u) ssq[i >> 6] = ss;
          }
        }
      }
      if (tail_wg && tid < (uint32_t)D) {   // whole waves: D is a multiple of 64
        kraw_s[tid] = kraw;
        if (rp.flags & 1u) {
          float ss = fmaf(kraw, kraw, 0.f);
#pragma unroll
          for (int o = 32; o > 0; o >>= 1) ss += __shfl_xor(ss, o, 64);
          if (lane == 0u) ssk[tid >> 6] = ss;
        }
        // the V row: rounded to fp16 for the copy, and the rounded value into the float32 row
        const __half vh = __float2half(vraw);
        const uint64_t vo = (uint64_t)bs.vb[group] + (uint64_t)(row_size - 1u) * D + tid;
        if (kv_writer) {
          const_cast<__half*>(kv)[vo - kv_shift] = vh;
          out[vo] = __half2float(vh);
        }
        vnew[tid] = vh;
      }
      __syncthreads();
      // sum over a row's 64-element pieces in the order of the stand-alone kernel: (s0 + s1) + (s2 + s3)
      auto row_ss = [&](const float* pc) {
        const float s0 = pc[0], s1 = pc[1], s2 = D >= 256 ? pc[D >= 256 ? 2 : 0] : 0.f, s3 = D >= 256 ? pc[D >= 256 ? 3 : 0] : 0.f;
        return (s0 + s1) + (s2 + s3);
      };
#pragma unroll
      for (uint32_t u = 0; u < PN; u++) {
        const uint32_t pi = tid + u * NT;           // a wave's 64 pairs belong to one head (D >= 128)
        if (pi < (uint32_t)(G * D) / 2u) {
          const uint32_t h = pi / half, i = pi % half;
          float y0 = qs[h * D + i], y1 = qs[h * D + i + half];
          if (rp.flags & 1u) {
            const float inv = 1.0f / sqrtf(row_ss(&ssq[h * (D / 64)]) / (float)D + 1e-6f);
            y0 = y0 * inv * wq[u][0];
            y1 = y1 * inv * wq[u][1];
          }
          const float angle = (float)rp.pos * fr[u];
          const float cs = cosf(angle), sn = sinf(angle);
          const float r0 = y0 * cs - y1 * sn, r1 = y0 * sn + y1 * cs;
          qs[h * D + i] = r0; qs[h * D + i + half] = r1;   // only this thread touches the pair
          if (split == 0u) {
            float* qd = n_splits == 1u ? out + (uint64_t)bs.q[op0 + h] : rp.q_scratch + (uint64_t)(op0 + h) * D;
            qd[i] = r0; qd[i + half] = r1;
          }
          float m = fmaxf(fabsf(r0), fabsf(r1));
#pragma unroll
          for (int o = 32; o > 0; o >>= 1) m = fmaxf(m, __shfl_xor(m, o, 64));
          if (lane == 0u) atomicMax(&hmax[h], __float_as_uint(m));
          if (u == 0u && tail_wg && tid < half) {
            // the new K row: same angle as this thread's query pair (tid = i); stored as the row tasks store it
            float k0 = kraw_s[i], k1 = kraw_s[i + half];
            if (rp.flags & 1u) {
              const float inv = 1.0f / sqrtf(row_ss(&ssk[0]) / (float)D + 1e-6f);
              k0 = k0 * inv * wk[0];
              k1 = k1 * inv * wk[1];
            }
            const float kr0 = k0 * cs - k1 * sn, kr1 = k0 * sn + k1 * cs;
            if (rp.k_dst != ROWT_NONE && kv_writer) {
              out[(uint64_t)rp.k_dst + (uint64_t)kvg * D + i] = kr0;
              out[(uint64_t)rp.k_dst + (uint64_t)kvg * D + i + half] = kr1;
            }
            const __half h0 = __float2half(kr0), h1 = __float2half(kr1);
            const uint64_t ko = (uint64_t)bs.kb[group] + (uint64_t)(row_size - 1u) * D + i;
            if (kv_writer) {
              const_cast<__half*>(kv)[ko - kv_shift] = h0; const_cast<__half*>(kv)[ko - kv_shift + half] = h1;
              out[ko] = __half2float(h0); out[ko + half] = __half2float(h1);
            }
            knew[i] = h0; knew[i + half] = h1;
          }
        }
      }
      __syncthreads();
    }
    const uint32_t e = c < G ? (hmax[c] >> 23) & 0xFFu : 0u;
    float s = 1.f, inv = 1.f;
    if (e >= 14u && e <= 254u) { s = __uint_as_float((267u - e) << 23); inv = __uint_as_float((e - 13u) << 23); }
    if (wave == 0u && c < G && kc == 0u) qinv[c] = inv;
    for (uint32_t idx = wave; idx < 2u * NI; idx += NW) {
      const float4 q4 = c < G ? *(const float4*)(qs + c * D + 32u * (idx >> 1) + 8u * kc + 4u * (idx & 1u))
                              : make_float4(0.f, 0.f, 0.f, 0.f);
      const float x[4] = {q4.x * s, q4.y * s, q4.z * s, q4.w * s};
      h4a_t hi4, lo4;
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
  // RP: the tile that holds the sequence's last row (and the lanes clamped onto it) takes that row from LDS: the
  // cache row was still being written when it was loaded
  auto patch = [&](uint4 (&kr)[NI], uint32_t (&vr)[16][DW], uint32_t rb) {
    if (!RP || !tail_wg || rb + 16u < t1) return;      // wave-uniform
    if (rb + c >= t1 - 1u) {
#pragma unroll
      for (int i = 0; i < NI; i++) kr[i] = *(const uint4*)((const char*)knew + klane + 64u * i);
    }
#pragma unroll
    for (int u = 0; u < 16; u++)
      if (rb + u >= t1 - 1u) {
        const char* src = (const char*)vnew + vlane;
        if (DPL == 1) vr[u][0] = *(const uint16_t*)src;
        else if (DPL == 2) vr[u][0] = *(const uint32_t*)src;
        else { const uint2 t = *(const uint2*)src; vr[u][0] = t.x; vr[u][DW - 1] = t.y; }
      }
  };
  // after the matrix product lane (c, kc) holds heads 4kc..4kc+3 of tile row c
  float inv_s[4], m_run[4], l_run[4];
  bool hval[4];
  uint32_t crow[4];
#pragma unroll
  for (int r = 0; r < 4; r++) {
    hval[r] = 4u * kc + r < (uint32_t)G;
    inv_s[r] = hval[r] ? qinv[4u * kc + r] : 0.f;
    // scalar reads of the arguments, then a per-lane choice
    crow[r] = 0u;
    if (r < G) crow[r] = EXT ? e_sc[op0 + r] : bs.sc[op0 + r];
    if (G > 4 && kc == 1u) crow[r] = EXT ? e_sc[op0 + (4 + r) % G] : bs.sc[op0 + (4 + r) % G];
    m_run[r] = ATTD_NEG;
    l_run[r] = 0.f;
  }

  float acc[G][DPL];
#pragma unroll
  for (int h = 0; h < G; h++)
#pragma unroll
    for (int j = 0; j < DPL; j++) acc[h][j] = 0.f;

  auto tile = [&](const uint4 (&kr)[NI], const uint32_t (&vr)[16][DW], uint32_t rb) {
    // scores of the tile: 2 * NI k-steps, high and low query part each, four independent sums
    f4a_t s0 = {0.f, 0.f, 0.f, 0.f}, s1 = s0, s2 = s0, s3 = s0;
#pragma unroll
    for (int i = 0; i < NI; i++) {
      const u2a_t b0 = {kr[i].x, kr[i].y}, b1 = {kr[i].z, kr[i].w};
      s0 = __builtin_amdgcn_mfma_f32_16x16x16f16(qop[2 * i][0][lane], __builtin_bit_cast(h4a_t, b0), s0, 0, 0, 0);
      s1 = __builtin_amdgcn_mfma_f32_16x16x16f16(qop[2 * i][1][lane], __builtin_bit_cast(h4a_t, b0), s1, 0, 0, 0);
      s2 = __builtin_amdgcn_mfma_f32_16x16x16f16(qop[2 * i + 1][0][lane], __builtin_bit_cast(h4a_t, b1), s2, 0, 0, 0);
      s3 = __builtin_amdgcn_mfma_f32_16x16x16f16(qop[2 * i + 1][1][lane], __builtin_bit_cast(h4a_t, b1), s3, 0, 0, 0);
    }
    const uint32_t row = rb + c;
    const bool rok = row < t1;
    float v[4], mt[4];
#pragma unroll
    for (int r = 0; r < 4; r++) {
      const float raw = ((s0[r] + s2[r]) + (s1[r] + s3[r])) * inv_s[r];
      if (rok && hval[r] && (!EXT || crow[r] != 0xFFFFFFFFu)) out[(uint64_t)crow[r] + row] = raw;
      v[r] = rok && hval[r] ? prep(raw, scale, cap) : ATTD_NEG;
      mt[r] = row16_max(v[r]);
    }
#pragma unroll
    for (int r = 0; r < 4; r++) {
      const float m_new = fmaxf(m_run[r], mt[r]);
      const float alpha = __expf(m_run[r] - m_new);
      const float p = rok && hval[r] ? __expf(v[r] - m_new) : 0.f;
      l_run[r] = l_run[r] * alpha + p;
      m_run[r] = m_new;
      if (hval[r]) {
        pbuf[wave][c][4u * kc + r] = p;
        if (c == 0u) abuf[wave][4u * kc + r] = alpha;
      }
    }
    __builtin_amdgcn_wave_barrier();
    // values: rescale the running sums, then the sixteen rows of the tile
#pragma unroll
    for (int h = 0; h < G; h++) {
      const float al = abuf[wave][h];
#pragma unroll
      for (int j = 0; j < DPL; j++) acc[h][j] *= al;
    }
#pragma unroll
    for (int u = 0; u < 16; u++) {
      float f[DPL];
      if (DPL == 1) f[0] = __half2float(__ushort_as_half((unsigned short)vr[u][0]));
      else {
#pragma unroll
        for (int w = 0; w < DW; w++) {
          const float2 t = __half22float2(*(const __half2*)&vr[u][w]);
          f[2 * w] = t.x; f[(2 * w + 1) % DPL] = t.y;
        }
      }
#pragma unroll
      for (int h = 0; h < G; h++) {
        const float pw = pbuf[wave][u][h];
#pragma unroll
        for (int j = 0; j < DPL; j++) acc[h][j] = fmaf(pw, f[j], acc[h][j]);
      }
    }
    __builtin_amdgcn_wave_barrier();
  };

  if (any) {
    if (PF) {
      while (true) {
        fetch(kB, vB, rbase + NW * 16u);     // next tile (clamped into the slice when there is none)
        __builtin_amdgcn_sched_barrier(0);
        patch(kA, vA, rbase);
        tile(kA, vA, rbase);
        rbase += NW * 16u;
        if (rbase >= t1) break;
        fetch(kA, vA, rbase + NW * 16u);
        __builtin_amdgcn_sched_barrier(0);
        patch(kB, vB, rbase);
        tile(kB, vB, rbase);
        rbase += NW * 16u;
        if (rbase >= t1) break;
      }
    } else {
      while (true) {
        patch(kA, vA, rbase);
        tile(kA, vA, rbase);
        rbase += NW * 16u;
        if (rbase >= t1) break;
        fetch(kA, vA, rbase);
      }
    }
  }

  // wave results to LDS: l summed over the 16 tile rows; each lane owns its dims of the output
#pragma unroll
  for (int r = 0; r < 4; r++) l_run[r] = row16_sum(l_run[r]);
#pragma unroll
  for (int h = 0; h < G; h++)
#pragma unroll
    for (int j = 0; j < DPL; j++) obuf[wave][h][(uint32_t)DPL * lane + j] = acc[h][j];
  if (c == 0u) {
#pragma unroll
    for (int r = 0; r < 4; r++)
      if (hval[r]) { mlbuf[wave][4u * kc + r][0] = m_run[r]; mlbuf[wave][4u * kc + r][1] = l_run[r]; }
  }
  __syncthreads();
  for (uint32_t idx = tid; idx < (uint32_t)(G * D); idx += NT) {
    const uint32_t h = idx / D, d = idx % D;
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
    if (n_splits == 1u) {
      out[(uint64_t)(EXT ? e_o[op0 + h] : bs.o[op0 + h]) + d] = o * (1.0f / L);
    } else {
      float* pp = partial + ((uint64_t)(op0 + h) * n_splits + split) * (D + 2);
      pp[2 + d] = o;
      if (d == 0u) { pp[0] = M; pp[1] = L; }
    }
  }
}

template <int D, int NW, bool PF>
static void launch_dg(uint32_t G, dim3 grid, const AttnDecodeArgs& a, const AttdBases& bs, uint32_t n_splits,
                      uint32_t chunk, const uint32_t* ext, const AttdRowPrep* rp) {
  const AttdRowPrep none = {};
#define ADL(GG, EE, RR)                                                                                   \
  k_attn_decode<D, GG, NW, PF, EE, RR><<<grid, NW * 64, 0, g.stream>>>(a.data, a.kv, a.kv_shift, a.row_size, chunk, n_splits,                   \
                                                                       (RR ? *rp : none).q_src, (RR ? *rp : none).k_src, (RR ? *rp : none).v_src, \
                                                                       EE ? (const void*)ext : (const void*)(RR ? *rp : none).inv_freq,         \
                                                                       a.data, a.scale, a.cap, g.attn_scratch, bs, RR ? *rp : none)
  if (ext) { if (G == 1) ADL(1, true, false); else if (G == 2) ADL(2, true, false); else if (G == 4) ADL(4, true, false); else ADL(8, true, false); }
  else if (rp && D >= 128) {
    constexpr bool R = D >= 128;   // the row preparation is built for head sizes 128 and 256
    if (G == 1) ADL(1, false, R); else if (G == 2) ADL(2, false, R); else if (G == 4) ADL(4, false, R); else ADL(8, false, R);
  }
  else { if (G == 1) ADL(1, false, false); else if (G == 2) ADL(2, false, false); else if (G == 4) ADL(4, false, false); else ADL(8, false, false); }
#undef ADL
}

template <int D>
static void launch_d(uint32_t G, uint32_t nw, bool pf, dim3 grid, const AttnDecodeArgs& a, const AttdBases& bs,
                     uint32_t n_splits, uint32_t chunk, const uint32_t* ext = nullptr, const AttdRowPrep* rp = nullptr) {
  if (nw == 8) launch_dg<D, 8, false>(G, grid, a, bs, n_splits, chunk, ext, rp);
  else if (pf) launch_dg<D, 4, true>(G, grid, a, bs, n_splits, chunk, ext, rp);
  else launch_dg<D, 4, false>(G, grid, a, bs, n_splits, chunk, ext, rp);
}

// 1 / base^(2i/dim), i < dim / 2, with the arithmetic of the stand-alone rotation (rope_cs2), so that a kernel
// that reads the table rotates to the same bits.  One table per (base, dim) seen, built on the device at first use.
__global__ void k_rope_inv_freq(float* t, uint32_t dim, float base) {
  const uint32_t i = blockIdx.x * 64u + threadIdx.x;
  if (i >= dim / 2u) return;
  const float e = (float)(2u * i) / (float)dim;
  const float p = (float)pow((double)base, (double)e);
  t[i] = 1.0f / p;
}
static struct { float base; uint32_t dim; float* dev; } g_freq[8];
static int g_freq_n = 0;
static const float* rope_inv_freq(float base, uint32_t dim) {
  for (int i = 0; i < g_freq_n; i++)
    if (g_freq[i].dim == dim && __builtin_bit_cast(uint32_t, g_freq[i].base) == __builtin_bit_cast(uint32_t, base)) return g_freq[i].dev;
  if (g_freq_n == 8 || dim < 2) return nullptr;
  float* dev = nullptr;
  if (hipMalloc((void**)&dev, (size_t)(dim / 2u) * 4) != hipSuccess) { (void)hipGetLastError(); return nullptr; }
  k_rope_inv_freq<<<cdiv(dim / 2u, 64u), 64, 0, g.stream>>>(dev, dim, base);
  g_freq[g_freq_n++] = {base, dim, dev};
  return dev;
}

// Are the queued row tasks exactly the preparation of this launch's operands?  Expected, in queue order: one
// rotation task per query head (destination = the head's query row, sources one after the other), one per KV head
// for the new K row (cache row = last row of the head's K rows), one copy per KV head for the new V row.
static bool match_prep(const std::vector<RowTask>& T, const AttnDecodeArgs& a, uint32_t G, uint32_t n_groups, AttdRowPrep* rp) {
  const uint32_t D = a.head_dim, n_ops = a.n_ops;
  if (T.size() != (size_t)n_ops + 2u * n_groups || a.row_size == 0) return false;
  const RowTask &q0 = T[0], &k0 = T[n_ops], &v0 = T[n_ops + n_groups];
  const uint32_t F = q0.flags;
  if (!(F & 2u) || k0.flags != F || v0.flags != 0u) return false;
  const uint64_t last = (uint64_t)(a.row_size - 1u) * D;
  for (uint32_t h = 0; h < n_ops; h++) {
    const RowTask& t = T[h];
    if (t.flags != F || t.dim != D || t.pos != q0.pos || t.base != q0.base || t.cache != ROWT_NONE || t.w != q0.w ||
        t.dst != a.ha[h] || (uint64_t)t.src != (uint64_t)q0.src + (uint64_t)h * D || (uint64_t)t.dst != (uint64_t)q0.dst + (uint64_t)h * D)
      return false;
  }
  for (uint32_t gi = 0; gi < n_groups; gi++) {
    const RowTask &t = T[n_ops + gi], &v = T[n_ops + n_groups + gi];
    if (t.flags != F || t.dim != D || t.pos != q0.pos || t.base != q0.base || t.w != k0.w ||
        (uint64_t)t.src != (uint64_t)k0.src + (uint64_t)gi * D || (uint64_t)t.cache != (uint64_t)a.hb[gi * G] + last)
      return false;
    if ((k0.dst == ROWT_NONE) != (t.dst == ROWT_NONE) || (t.dst != ROWT_NONE && (uint64_t)t.dst != (uint64_t)k0.dst + (uint64_t)gi * D))
      return false;
    if (v.flags != 0u || v.dim != D || v.dst != ROWT_NONE || v.w != ROWT_NONE ||
        (uint64_t)v.src != (uint64_t)v0.src + (uint64_t)gi * D || (uint64_t)v.cache != (uint64_t)a.hv[gi * G] + last)
      return false;
    // the new rows lie in the fp16 copy
    if ((uint64_t)t.cache < a.kv_shift || (uint64_t)v.cache < a.kv_shift) return false;
  }
  if ((F & 1u) && (q0.w == ROWT_NONE || k0.w == ROWT_NONE)) return false;
  // What the launch reads (raw rows, norm weights) against what it writes (prepared rows, cache rows, score rows,
  // outputs).  A prepared row may go back over its own raw row (the usual case); nothing else may meet.
  struct Iv { uint64_t lo, n; int own; };   // own: > 0 marks a raw row / prepared row pair that may coincide
  std::vector<Iv> rd, wr;
  rd.push_back({v0.src, (uint64_t)n_groups * D, 0});
  if (F & 1u) { rd.push_back({q0.w, D, 0}); rd.push_back({k0.w, D, 0}); }
  for (uint32_t h = 0; h < n_ops; h++) { rd.push_back({T[h].src, D, 1 + (int)h}); wr.push_back({T[h].dst, D, 1 + (int)h}); }
  for (uint32_t gi = 0; gi < n_groups; gi++) {
    const RowTask &t = T[n_ops + gi], &v = T[n_ops + n_groups + gi];
    rd.push_back({t.src, D, 1000 + (int)gi});
    if (t.dst != ROWT_NONE) wr.push_back({t.dst, D, 1000 + (int)gi});
    wr.push_back({t.cache, D, 0}); wr.push_back({v.cache, D, 0});
  }
  for (uint32_t h = 0; h < n_ops; h++) { wr.push_back({a.hc[h], a.row_size, 0}); wr.push_back({a.ho[h], D, 0}); }
  auto meet = [](const Iv& x, const Iv& y) { return !(x.lo + x.n <= y.lo || y.lo + y.n <= x.lo); };
  for (const Iv& w : wr)
    for (const Iv& r : rd)
      if (meet(w, r) && !(w.own && w.own == r.own && w.lo == r.lo)) return false;
  for (size_t x = 0; x < wr.size(); x++)
    for (size_t y = x + 1; y < wr.size(); y++)
      if (meet(wr[x], wr[y])) return false;
  const float* inv_freq = rope_inv_freq(q0.base, D);
  if (!inv_freq) return false;
  *rp = AttdRowPrep{F & 1u, q0.pos, q0.base, q0.src, k0.src, k0.dst, v0.src, (F & 1u) ? q0.w : 0u, (F & 1u) ? k0.w : 0u,
                    nullptr, inv_freq};
  return true;
}

bool launch_attn_decode(const AttnDecodeArgs& a, AttnPartials* ap, bool* left, int* rc) {
  if (tuning("ADAMAH_ATTN_IMPL", 1) == 0) return false;
  const uint32_t D = a.head_dim, n_ops = a.n_ops;
  if (D != 64 && D != 128 && D != 256) return false;
  if (!a.ha || !a.hb || !a.hc || !a.hv || !a.ho || !a.kv || n_ops == 0 || n_ops > ATTD_MAX_OPS || a.row_size == 0) return false;
  uint32_t G = 1;
  while (G < n_ops && G < 8 && a.hb[G] == a.hb[0] && a.hv[G] == a.hv[0]) G++;
  if (G != 1 && G != 2 && G != 4 && G != 8) G = G > 4 ? 4 : G == 3 ? 2 : 1;
  while (G > 1 && n_ops % G) G >>= 1;
  for (uint32_t op = 0; op < n_ops; op++) {
    const uint32_t o0 = op - op % G;
    if (a.hb[op] != a.hb[o0] || a.hv[op] != a.hv[o0]) return false;
    if ((a.hb[op] - a.kv_shift) % 8u || (a.hv[op] - a.kv_shift) % 8u) return false;
  }
  const uint32_t n_groups = n_ops / G;
  if (n_groups > ATTD_MAX_GROUPS) return false;
  AttdRowPrep rp = {};
  if (a.prep) {   // with the row preparation inside the launch, or no launch at all
    if (!a.prep_done || (D != 128 && D != 256) || tuning("ADAMAH_ATTN_ROWPREP", 1) == 0 ||
        !match_prep(*a.prep, a, G, n_groups, &rp))
      return false;
  }

  // Slices of the sequence.  Short sequences (at most one 16-row tile per wave with eight waves on every CU):
  // workgroups of 8 waves, one tile each, every tile asked for at the start; longer ones: 4 waves (four per CU) and
  // as many tiles per wave as it takes, the next tile asked for while one is worked on.  (One tile per wave up to
  // eight waves per CU instead of four: Llama shape at context 4096 547 -> 554 tok/s, the pair alone 11.0 -> 10.6 us.)
  const uint32_t target = (uint32_t)std::max(1, knob("ADAMAH_ATTN_WAVES", 4 * g.n_cu));
  const uint64_t tiles = (uint64_t)n_groups * cdiv(a.row_size, 16u);
  uint32_t nw = (tiles <= 2u * target && G * D <= 1024u) ? 8u : 4u;
  nw = (uint32_t)knob("ADAMAH_ATTN_NW", (int)nw) == 8u && G * D <= 1024u ? 8u : 4u;
  const uint32_t step = nw * 16u;
  uint32_t chunk = step * std::max<uint32_t>(1u, cdiv(tiles, nw == 8u ? 2u * target : target));
  while (cdiv(a.row_size, chunk) > ATTD_MAX_SPLITS) chunk += step;
  bool leave = a.leave_partials;
  if (leave) {
    uint32_t cf = chunk;
    while (cf < 4096u && (uint64_t)n_ops * cdiv(a.row_size, cf) * (D + 2) > a.fold_floats) cf += step;
    if ((uint64_t)n_ops * cdiv(a.row_size, cf) * (D + 2) <= a.fold_floats) chunk = cf; else leave = false;
  }
  if (nw == 8u && chunk > step) { nw = 4u; }   // several tiles per wave: the prefetching 4-wave form
  const bool pf = chunk > nw * 16u;
  const uint32_t n_splits = cdiv(a.row_size, chunk);
  if ((uint64_t)n_ops * n_splits * (D + 2) > g.attn_scratch_floats) return false;
  // A launch of few workgroups (short context, few KV heads): one query head per workgroup instead of the whole
  // group -- G times the workgroups, each with a G-th of the vector work between its barriers; the heads of a group
  // ask for the same K / V tiles (Gemma shape at context 640: 5 -> 20 workgroups).
  uint32_t Gl = G, share_log = 0;
  {
    const int hs = tuning("ADAMAH_ATTN_HEADSPLIT", 1);
    const bool small = (uint64_t)n_ops * cdiv(a.row_size, chunk) <= (uint64_t)g.n_cu;
    if (G > 1 && n_ops <= ATTD_MAX_GROUPS && (hs == 2 || (hs == 1 && small))) {
      Gl = 1;
      while ((1u << share_log) < G) share_log++;
    }
  }
  const uint32_t n_groups_l = n_ops / Gl;
  AttdBases bs;
  for (uint32_t op = 0; op < n_ops; op++) { bs.q[op] = a.ha[op]; bs.sc[op] = a.hc[op]; bs.o[op] = a.ho[op]; }
  for (uint32_t gi = 0; gi < n_groups_l; gi++) { bs.kb[gi] = a.hb[gi * Gl]; bs.vb[gi] = a.hv[gi * Gl]; }
  // the slices are merged by the consumer (leave) or by the caller's merge kernel
  dim3 grid(n_splits, n_groups_l);
  const uint32_t splits_share = n_splits | (share_log << 16);
  const AttdRowPrep* rpp = a.prep ? &rp : nullptr;
  // the prepared queries wait behind the partials until the merge copies them to their rows
  const uint64_t part_floats = (uint64_t)n_ops * n_splits * (D + 2);
  if (a.prep && n_splits > 1) {
    if (part_floats + (uint64_t)n_ops * D > g.attn_scratch_floats) return false;
    rp.q_scratch = g.attn_scratch + part_floats;
  }
  if (D == 64) launch_d<64>(Gl, nw, pf, grid, a, bs, splits_share, chunk);
  else if (D == 128) launch_d<128>(Gl, nw, pf, grid, a, bs, splits_share, chunk, nullptr, rpp);
  else launch_d<256>(Gl, nw, pf, grid, a, bs, splits_share, chunk, nullptr, rpp);
  if (a.prep) *a.prep_done = true;
  count_launch();
  *rc = check_launch();
  *ap = AttnPartials{g.attn_scratch, *rc == 0 ? n_splits : 1u, D, n_ops, 0, nullptr, 0, 0};
  if (a.prep && n_splits > 1 && *rc == 0) { ap->q_src = rp.q_scratch; ap->q_dst = (*a.prep)[0].dst; ap->q_n = n_ops * D; }
  *left = leave;
  return true;
}


// ---- several sequences in lockstep ----------------------------------------------------------------
// A batched decode step issues one (scores, softmax . V) pair per sequence: same length, head count and
// parameters, the same score rows, but queries, outputs and KV cache of its own.  A run of such pairs
// becomes one launch of the kernel above over all their heads (bases in device memory); only the
// last pair stores raw scores, which is what the shared score rows hold after the pairs ran one by one.
// The table of operand bases of a launch.  A decode loop comes back with the same tables step after step (one per
// layer), so each distinct table is uploaded once and kept: no copy in the step, and a step without copies from the
// host can be recorded into a graph.
struct ExtTable { std::vector<uint32_t> host; uint32_t* dev; };
static std::vector<ExtTable> g_ext_tables;
#define ATTD_EXT_TABLES 1024u

void attn_decode_release() {
  for (int i = 0; i < g_freq_n; i++) hipFree(g_freq[i].dev);
  g_freq_n = 0;
  for (ExtTable& t : g_ext_tables) hipFree(t.dev);
  g_ext_tables.clear();
}

// Device copy of the table, uploaded on first sight; nullptr: out of memory.
static const uint32_t* ext_table(const std::vector<uint32_t>& ext, int* rc) {
  for (const ExtTable& t : g_ext_tables)
    if (t.host.size() == ext.size() && memcmp(t.host.data(), ext.data(), ext.size() * 4) == 0) return t.dev;
  if (g_ext_tables.size() >= ATTD_EXT_TABLES) {   // a caller that never repeats itself: start over
    hipStreamSynchronize(g.stream);
    for (ExtTable& t : g_ext_tables) hipFree(t.dev);
    g_ext_tables.clear();
    layout_changed();
  }
  uint32_t* dev = nullptr;
  if (hipMalloc((void**)&dev, ext.size() * 4) != hipSuccess) { (void)hipGetLastError(); *rc = ADAMAH_ERR_MEMORY; return nullptr; }
  if ((*rc = h2d(dev, ext.data(), ext.size() * 4)) != ADAMAH_OK) { hipFree(dev); return nullptr; }
  g_ext_tables.push_back({ext, dev});
  return dev;
}

size_t launch_attn_batch(const std::vector<PendOp>& q, size_t i, int* rc) {
  *rc = ADAMAH_OK;
  if (tuning("ADAMAH_ATTN_BATCH", 1) == 0) return 0;
  const size_t n = q.size();
  if (i + 3 >= n || !attn_foldable(q[i], q[i + 1])) return 0;
  const PendOp &s0 = q[i], &a0 = q[i + 1];
  // cheap way out first: the next pair has to bring its own query, output and cache handles
  if (q[i + 2].kind != PK_SCORES || q[i + 3].kind != PK_ATTN || q[i + 2].h[0] == s0.h[0] || q[i + 3].h[2] == a0.h[2] ||
      q[i + 2].h[1] == s0.h[1] || q[i + 2].n != s0.n)
    return 0;
  Map* mp = get_f32_map(a0.map_act);
  const uint32_t H = a0.rpg, D = a0.k, rows = a0.n;
  if (!mp || !mp->kv16 || H == 0 || s0.k != D || (D != 64 && D != 128 && D != 256) || rows == 0) return 0;
  const uint32_t* sc0 = res_host(s0.h[2], H);
  if (!sc0) return 0;
  std::vector<const uint32_t*> hq, hk, hv, ho;
  size_t B = 0;
  while (i + 2 * B + 1 < n) {
    const PendOp &st = q[i + 2 * B], &at = q[i + 2 * B + 1];
    if (!attn_foldable(st, at) || st.map_act != s0.map_act || st.rpg != H || st.k != D || at.k != D || st.n != rows ||
        at.eps != a0.eps || at.f2 != a0.f2)
      break;
    const uint32_t *qt = res_host(st.h[0], H), *kt = res_host(st.h[1], H), *ct = res_host(st.h[2], H);
    const uint32_t *vt = res_host(at.h[1], H), *ot = res_host(at.h[2], H);
    if (!qt || !kt || !ct || !vt || !ot) break;
    bool same = true;
    for (uint32_t h = 0; same && h < H; h++) same = ct[h] == sc0[h];
    if (!same) break;
    hq.push_back(qt); hk.push_back(kt); hv.push_back(vt); ho.push_back(ot);
    B++;
  }
  if (B < 2) return 0;
  // group structure of the first pair, required of all
  uint32_t G = 1;
  while (G < H && G < 8 && hk[0][G] == hk[0][0] && hv[0][G] == hv[0][0]) G++;
  if (G != 1 && G != 2 && G != 4 && G != 8) G = G > 4 ? 4 : G == 3 ? 2 : 1;
  while (G > 1 && H % G) G >>= 1;
  const uint64_t need_rows = (uint64_t)rows * D;
  for (size_t b = 0; b < B; b++)
    for (uint32_t op = 0; op < H; op++) {
      const uint32_t o0 = op - op % G;
      if (hk[b][op] != hk[b][o0] || hv[b][op] != hv[b][o0]) return 0;
      if (hk[b][op] < mp->kv_start || hv[b][op] < mp->kv_start || (hk[b][op] - mp->kv_start) % 8u || (hv[b][op] - mp->kv_start) % 8u) return 0;
      if (hk[b][op] - mp->kv_start + need_rows > mp->kv_count || hv[b][op] - mp->kv_start + need_rows > mp->kv_count) return 0;
      if (!in_range(hq[b][op], D, mp->n_elems) || !in_range(ho[b][op], D, mp->n_elems)) return 0;
    }
  // no pair may write what another reads: outputs apart from all queries and from each other
  {
    std::vector<std::pair<uint64_t, uint64_t>> qs, os;
    for (size_t b = 0; b < B; b++)
      for (uint32_t op = 0; op < H; op++) { qs.push_back({hq[b][op], (uint64_t)hq[b][op] + D}); os.push_back({ho[b][op], (uint64_t)ho[b][op] + D}); }
    std::sort(os.begin(), os.end());
    for (size_t k = 1; k < os.size(); k++) if (os[k].first < os[k - 1].second) return 0;
    std::sort(qs.begin(), qs.end());
    size_t j = 0;
    for (const auto& o : os) {
      while (j < qs.size() && qs[j].second <= o.first) j++;
      if (j < qs.size() && qs[j].first < o.second) return 0;
    }
    const uint64_t kv0 = mp->kv_start, kv1 = mp->kv_start + mp->kv_count;
    for (const auto& o : os) if (!(o.second <= kv0 || kv1 <= o.first)) return 0;
    for (uint32_t h = 0; h < H; h++) {
      const uint64_t s_lo = sc0[h], s_hi = (uint64_t)sc0[h] + rows;
      if (!in_range(sc0[h], rows, mp->n_elems) || !(s_hi <= kv0 || kv1 <= s_lo)) return 0;
      for (const auto& o : os) if (!(o.second <= s_lo || s_hi <= o.first)) return 0;
      for (const auto& qq : qs) if (!(qq.second <= s_lo || s_hi <= qq.first)) return 0;
    }
  }
  const uint32_t n_all = (uint32_t)(B * H), n_groups = n_all / G;
  // slices as for a single pair, sized for all the groups
  const uint32_t target = (uint32_t)std::max(1, knob("ADAMAH_ATTN_WAVES", 4 * g.n_cu));
  const uint64_t tiles = (uint64_t)n_groups * cdiv(rows, 16u);
  uint32_t nw = (tiles <= 2u * target && G * D <= 1024u) ? 8u : 4u;
  const uint32_t step = nw * 16u;
  uint32_t chunk = step * std::max<uint32_t>(1u, cdiv(tiles, nw == 8u ? 2u * target : target));
  while (cdiv(rows, chunk) > ATTD_MAX_SPLITS) chunk += step;
  if (nw == 8u && chunk > step) nw = 4u;
  const bool pf = chunk > nw * 16u;
  const uint32_t n_splits = cdiv(rows, chunk);
  if (n_groups > 65535u || (uint64_t)n_all * n_splits * (D + 2) > g.attn_scratch_floats) return 0;
  const size_t words = 3 * (size_t)n_all + 2 * (size_t)n_groups;
  std::vector<uint32_t> ext(words);
  for (size_t b = 0; b < B; b++)
    for (uint32_t op = 0; op < H; op++) {
      const size_t k = b * H + op;
      ext[k] = hq[b][op];
      ext[n_all + k] = b + 1 == B ? sc0[op] : 0xFFFFFFFFu;
      ext[2 * (size_t)n_all + k] = ho[b][op];
      if (op % G == 0) { ext[3 * (size_t)n_all + k / G] = hk[b][op]; ext[3 * (size_t)n_all + n_groups + k / G] = hv[b][op]; }
    }
  const uint32_t* ext_dev = ext_table(ext, rc);
  if (!ext_dev) return 2 * B;
  AttnDecodeArgs da = {(float*)mp->buf, mp->kv16, mp->kv_start, nullptr, nullptr, nullptr, nullptr, nullptr,
                       nullptr, nullptr, nullptr, nullptr, nullptr, n_all, D, rows, a0.eps, a0.f2, false, 0};
  AttdBases bs = {};
  dim3 grid(n_splits, n_groups);
  if (D == 64) launch_d<64>(G, nw, pf, grid, da, bs, n_splits, chunk, ext_dev);
  else if (D == 128) launch_d<128>(G, nw, pf, grid, da, bs, n_splits, chunk, ext_dev);
  else launch_d<256>(G, nw, pf, grid, da, bs, n_splits, chunk, ext_dev);
  count_launch();
  *rc = check_launch();
  if (*rc == ADAMAH_OK && n_splits > 1) {
    // The O-projection of all sequences next in the queue, over the heads' outputs as rows [B, H D]: the merge of
    // the slices also writes the fp16 form of those rows, and the matmul skips its conversion launch.
    bool merged = false;
    const size_t nx = i + 2 * B;
    if (n_splits <= 8 && nx < n && q[nx].kind == PK_GEMM && q[nx].map_act == s0.map_act && q[nx].rpg == B && q[nx].k == H * D &&
        q[nx].a == ho[0][0] && tuning("ADAMAH_ATTN_MERGE_EMIT", 1) != 0) {
      bool rows = true;
      for (size_t b = 0; rows && b < B; b++)
        for (uint32_t op = 0; rows && op < H; op++) rows = ho[b][op] == ho[0][0] + (b * H + op) * D;
      if (rows && launch_attn_merge_rows_f16(mp, g.attn_scratch, ho[0][0], (uint32_t)B, H * D, D, n_splits)) {
        merged = true;
        *rc = check_launch();
      }
    }
    if (!merged) *rc = launch_attn_combine_dev(mp, g.attn_scratch, ext_dev + 2 * (size_t)n_all, n_all, D, n_splits);
  }
  return 2 * B;
}

}  // namespace adamah

