// Block-quantised dequant-GEMV (float32 activation x Q4/Q8 weight rows) and the fused
// GEMV + argmax LM-head tail.
//
// Reference semantics: y[n] = sum_k x[k] * (float(code(b + n*K + k)) * scale[g] + zp[g]),
// g = (b + n*K + k) / group_size over the whole weight map
// (shaders/src/f32/map_matvec_t_xq4.comp:49-135, map_matvec_t_xq8.comp:47-132,
//  map_matmul_t_xq4.comp:33-73; dispatch adamah.c:8606-8803, 9834-9910);
// argmax tail: per group of `rows_per_group` rows the best (value, row), then a pair
// reduction (map_matvec_argmax_t_xq4.comp:66-158, map_argmax_pairs.comp:34-67,
// adamah.c:9558-9721).
//
// Fast path ("block" kernels): group_size 32, rows aligned to blocks.  One lane owns one
// 32-weight block per step: a 16-byte (Q4) or 2x16-byte (Q8) load of codes that the wave
// reads as one contiguous 1 KiB / 2 KiB row segment, plus the block's scale.  The activation
// vector lives in LDS (XOR-swizzled 16-byte chunks, conflict-free for the one-block-per-lane
// access), read once per step and reused for ROWS weight rows.  Per block the kernel
// accumulates  scale * sum(code*x) + zp * sum(x)  with sum(x) per block precomputed, so the
// inner loop is one byte->float convert and one FMA per weight, fp32 throughout.
#include "gemv_common.h"
#include "../../include/adamah_hip.h"
#include <algorithm>
#include <stdlib.h>

namespace adamah {

// sum_j code[j] * x[j] for the 8 nibbles of one word; x = two float4 (elements 0..7)
__device__ __forceinline__ float dot_q4_word(uint32_t w, const float4& xa, const float4& xb, float acc) {
  uint32_t lo = w & 0x0F0F0F0Fu;          // elements 0,2,4,6
  uint32_t hi = (w >> 4) & 0x0F0F0F0Fu;   // elements 1,3,5,7
  acc = fmaf(ubyte_f32<0>(lo), xa.x, acc);
  acc = fmaf(ubyte_f32<0>(hi), xa.y, acc);
  acc = fmaf(ubyte_f32<1>(lo), xa.z, acc);
  acc = fmaf(ubyte_f32<1>(hi), xa.w, acc);
  acc = fmaf(ubyte_f32<2>(lo), xb.x, acc);
  acc = fmaf(ubyte_f32<2>(hi), xb.y, acc);
  acc = fmaf(ubyte_f32<3>(lo), xb.z, acc);
  acc = fmaf(ubyte_f32<3>(hi), xb.w, acc);
  return acc;
}
__device__ __forceinline__ float dot_q8_word(uint32_t w, const float4& x, float acc) {
  acc = fmaf(ubyte_f32<0>(w), x.x, acc);
  acc = fmaf(ubyte_f32<1>(w), x.y, acc);
  acc = fmaf(ubyte_f32<2>(w), x.z, acc);
  acc = fmaf(ubyte_f32<3>(w), x.w, acc);
  return acc;
}

// LDS position (in float4 units) of 16-byte chunk j (0..7) of activation block blk
__device__ __forceinline__ uint32_t xs_slot(uint32_t blk, uint32_t j) { return blk * 8u + (j ^ (blk & 7u)); }

template <int FMT, int EPI, int ROWS>
__global__ void __launch_bounds__(256)
k_gemv_block(const float* act, float* act_out, const uint8_t* __restrict__ W,
             const float2* __restrict__ qp, const __half* __restrict__ d16, const uint32_t* __restrict__ la,
             const uint32_t* __restrict__ lb, const uint32_t* __restrict__ lc, const uint32_t* __restrict__ lidx,
             const uint32_t* __restrict__ lval, uint32_t K, uint32_t N, uint32_t rows_per_group, uint32_t n_groups) {
  constexpr bool Q4 = (FMT == FMT_Q4_B16 || FMT == FMT_Q4_AFF);
  constexpr bool B16 = (FMT == FMT_Q4_B16 || FMT == FMT_Q8_B16);
  constexpr float OFF = Q4 ? 8.0f : 128.0f;
  extern __shared__ float4 smem4[];
  const uint32_t nblk = K >> 5;
  float4* xs = smem4;                               // nblk * 8 float4
  float* sx = (float*)(smem4 + (size_t)nblk * 8);   // nblk block sums
  __shared__ float red_v[4];
  __shared__ uint32_t red_i[4];

  const uint32_t tid = threadIdx.x, lane = tid & 63u, wave = tid >> 6;
  const uint64_t a = la[0], b = lb[0];

  // stage x (swizzled) and per-block sums
  for (uint32_t i = tid; i < nblk * 8u; i += 256u) {
    const float* p = act + a + (uint64_t)i * 4u;
    xs[xs_slot(i >> 3, i & 7u)] = make_float4(p[0], p[1], p[2], p[3]);
  }
  __syncthreads();
  for (uint32_t blk = tid; blk < nblk; blk += 256u) {
    float s = 0.f;
#pragma unroll
    for (uint32_t j = 0; j < 8; j++) {
      float4 v = xs[xs_slot(blk, j)];
      s += (v.x + v.y) + (v.z + v.w);
    }
    sx[blk] = s;
  }
  __syncthreads();

  const uint64_t gbase = b >> 5;                    // first group of the matrix
  for (uint32_t grp = blockIdx.x; grp < n_groups; grp += gridDim.x) {
    const uint32_t row0 = grp * rows_per_group;
    const uint32_t row1 = min(N, row0 + rows_per_group);
    float best_v = NEG_FLT_MAX;
    uint32_t best_i = INVALID_IDX;
    for (uint32_t r = row0 + wave * ROWS; r < row1; r += 4u * ROWS) {
      float acc[ROWS];
#pragma unroll
      for (int i = 0; i < ROWS; i++) acc[i] = 0.f;
      for (uint32_t blk = lane; blk < nblk; blk += 64u) {
        uint4 q0[ROWS], q1[ROWS];
        float sc[ROWS], zp[ROWS];
#pragma unroll
        for (int i = 0; i < ROWS; i++) {
          const uint32_t row = min(r + i, row1 - 1);          // clamp: duplicates are discarded below
          const uint64_t gidx = gbase + (uint64_t)row * nblk + blk;
          if (Q4) {
            q0[i] = *(const uint4*)(W + (gidx << 4));
          } else {
            q0[i] = *(const uint4*)(W + (gidx << 5));
            q1[i] = *(const uint4*)(W + (gidx << 5) + 16);
          }
          if (B16) { sc[i] = __half2float(d16[gidx]); zp[i] = 0.f; }
          else { float2 p = qp[gidx]; sc[i] = p.x; zp[i] = p.y; }
        }
        float4 x[8];
#pragma unroll
        for (uint32_t j = 0; j < 8; j++) x[j] = xs[xs_slot(blk, j)];
        const float sxb = sx[blk];
#pragma unroll
        for (int i = 0; i < ROWS; i++) {
          float d = 0.f;
          if (Q4) {
            d = dot_q4_word(q0[i].x, x[0], x[1], d);
            d = dot_q4_word(q0[i].y, x[2], x[3], d);
            d = dot_q4_word(q0[i].z, x[4], x[5], d);
            d = dot_q4_word(q0[i].w, x[6], x[7], d);
          } else {
            d = dot_q8_word(q0[i].x, x[0], d); d = dot_q8_word(q0[i].y, x[1], d);
            d = dot_q8_word(q0[i].z, x[2], d); d = dot_q8_word(q0[i].w, x[3], d);
            d = dot_q8_word(q1[i].x, x[4], d); d = dot_q8_word(q1[i].y, x[5], d);
            d = dot_q8_word(q1[i].z, x[6], d); d = dot_q8_word(q1[i].w, x[7], d);
          }
          if (B16) acc[i] = fmaf(sc[i], fmaf(-OFF, sxb, d), acc[i]);
          else acc[i] = fmaf(sc[i], d, fmaf(zp[i], sxb, acc[i]));
        }
      }
#pragma unroll
      for (int i = 0; i < ROWS; i++) {
        const float y = wave_sum_to_lane63(acc[i]);   // total valid in lane 63 only
        const uint32_t row = r + i;
        if (row < row1 && lane == 63) {
          if (EPI == EPI_STORE) act_out[(uint64_t)lc[0] + row] = y;
          else if (better(y, row, best_v, best_i)) { best_v = y; best_i = row; }
        }
      }
    }
    if (EPI == EPI_ARGMAX) {
      if (lane == 63) { red_v[wave] = best_v; red_i[wave] = best_i; }
      __syncthreads();
      if (tid == 0) {
        float bv = red_v[0]; uint32_t bi = red_i[0];
        for (int w = 1; w < 4; w++)
          if (better(red_v[w], red_i[w], bv, bi)) { bv = red_v[w]; bi = red_i[w]; }
        act_out[lidx[grp]] = (float)(bi == INVALID_IDX ? 0u : bi);
        act_out[lval[grp]] = bv;
      }
      __syncthreads();
    }
  }
}

// ---- register-resident activation variant --------------------------------------------------
// Each lane keeps the 32 activations (and their sum) of its NB blocks in registers for the whole
// workgroup lifetime, so the row loop touches no LDS: per row it issues NB 16-byte code loads and
// NB scale loads, converts and FMAs.  KS waves share a row when K is long (each takes a slice of
// 64*NB blocks) and meet through 64 bytes of LDS once per row step.
typedef float float4_u __attribute__((ext_vector_type(4), aligned(4)));

template <int FMT, int EPI, int NB, int KS>
__global__ void __launch_bounds__(256)
k_gemv_regx(const float* act, float* act_out, const uint8_t* __restrict__ W, const float2* __restrict__ qp,
            const __half* __restrict__ d16, const uint32_t* __restrict__ la, const uint32_t* __restrict__ lb,
            const uint32_t* __restrict__ lc, const uint32_t* __restrict__ lidx, const uint32_t* __restrict__ lval,
            uint32_t K, uint32_t N, uint32_t rows_per_wg) {
  constexpr bool Q4 = (FMT == FMT_Q4_B16 || FMT == FMT_Q4_AFF);
  constexpr bool B16 = (FMT == FMT_Q4_B16 || FMT == FMT_Q8_B16);
  constexpr float OFF = Q4 ? 8.0f : 128.0f;
  constexpr int R = 4;             // rows in flight per wave
  constexpr int G = 4 / KS;        // row groups per workgroup
  __shared__ float part[G][KS][R];
  __shared__ float red_v[4];
  __shared__ uint32_t red_i[4];

  const uint32_t tid = threadIdx.x, lane = tid & 63u, wave = tid >> 6;
  const uint32_t kpart = wave % KS, grp = wave / KS;
  const uint32_t nblk = K >> 5;
  const uint64_t a = la[0], gbase = (uint64_t)lb[0] >> 5;

  uint32_t blk[NB];
  float x[NB][32], sx[NB];
#pragma unroll
  for (int i = 0; i < NB; i++) {
    blk[i] = (kpart * NB + i) * 64u + lane;
    const bool valid = blk[i] < nblk;
    const float4_u* px = (const float4_u*)(act + a + (uint64_t)(valid ? blk[i] : 0u) * 32u);
    float s = 0.f;
#pragma unroll
    for (int j = 0; j < 8; j++) {
      float4_u v = px[j];
      if (!valid) v = (float4_u)(0.f);
      x[i][4 * j] = v.x; x[i][4 * j + 1] = v.y; x[i][4 * j + 2] = v.z; x[i][4 * j + 3] = v.w;
      s += (v.x + v.y) + (v.z + v.w);
    }
    sx[i] = s;
    if (!valid) blk[i] = nblk - 1;      // keep addresses in range; the zero activations cancel the block
  }

  const uint32_t row_begin = blockIdx.x * rows_per_wg;
  const uint32_t row_end = min(N, row_begin + rows_per_wg);
  const uint32_t iters = (rows_per_wg + G * R - 1) / (G * R);
  float best_v = NEG_FLT_MAX;
  uint32_t best_i = INVALID_IDX;

  for (uint32_t it = 0; it < iters; it++) {
    const uint32_t r0 = row_begin + it * (G * R) + grp * R;
    float acc[R];
#pragma unroll
    for (int j = 0; j < R; j++) acc[j] = 0.f;
    if (r0 < row_end) {
#pragma unroll
      for (int i = 0; i < NB; i++) {
        uint4 q0[R], q1[R];
        float sc[R], zp[R];
#pragma unroll
        for (int j = 0; j < R; j++) {
          const uint32_t row = min(r0 + j, row_end - 1);
          const uint64_t gidx = gbase + (uint64_t)row * nblk + blk[i];
          if (Q4) {
            q0[j] = *(const uint4*)(W + (gidx << 4));
          } else {
            q0[j] = *(const uint4*)(W + (gidx << 5));
            q1[j] = *(const uint4*)(W + (gidx << 5) + 16);
          }
          if (B16) { sc[j] = __half2float(d16[gidx]); zp[j] = 0.f; }
          else { const float2 p = qp[gidx]; sc[j] = p.x; zp[j] = p.y; }
        }
#pragma unroll
        for (int j = 0; j < R; j++) {
          float d = 0.f;
          const float* xv = x[i];
          if (Q4) {
            const uint32_t w[4] = {q0[j].x, q0[j].y, q0[j].z, q0[j].w};
#pragma unroll
            for (int u = 0; u < 4; u++) {
              const uint32_t lo = w[u] & 0x0F0F0F0Fu, hi = (w[u] >> 4) & 0x0F0F0F0Fu;
              d = fmaf(ubyte_f32<0>(lo), xv[8 * u + 0], d); d = fmaf(ubyte_f32<0>(hi), xv[8 * u + 1], d);
              d = fmaf(ubyte_f32<1>(lo), xv[8 * u + 2], d); d = fmaf(ubyte_f32<1>(hi), xv[8 * u + 3], d);
              d = fmaf(ubyte_f32<2>(lo), xv[8 * u + 4], d); d = fmaf(ubyte_f32<2>(hi), xv[8 * u + 5], d);
              d = fmaf(ubyte_f32<3>(lo), xv[8 * u + 6], d); d = fmaf(ubyte_f32<3>(hi), xv[8 * u + 7], d);
            }
          } else {
            const uint32_t w[8] = {q0[j].x, q0[j].y, q0[j].z, q0[j].w, q1[j].x, q1[j].y, q1[j].z, q1[j].w};
#pragma unroll
            for (int u = 0; u < 8; u++) {
              d = fmaf(ubyte_f32<0>(w[u]), xv[4 * u + 0], d); d = fmaf(ubyte_f32<1>(w[u]), xv[4 * u + 1], d);
              d = fmaf(ubyte_f32<2>(w[u]), xv[4 * u + 2], d); d = fmaf(ubyte_f32<3>(w[u]), xv[4 * u + 3], d);
            }
          }
          if (B16) acc[j] = fmaf(sc[j], fmaf(-OFF, sx[i], d), acc[j]);
          else acc[j] = fmaf(sc[j], d, fmaf(zp[j], sx[i], acc[j]));
        }
      }
    }
#pragma unroll
    for (int j = 0; j < R; j++) acc[j] = wave_sum_to_lane63(acc[j]);
    if (KS > 1) {
      if (lane == 63) {
#pragma unroll
        for (int j = 0; j < R; j++) part[grp][kpart][j] = acc[j];
      }
      __syncthreads();
    }
    // one lane per row group finishes the rows: lane 63 of the kpart-0 wave
    if (kpart == 0 && lane == 63 && r0 < row_end) {
#pragma unroll
      for (int j = 0; j < R; j++) {
        float y = acc[j];
        if (KS > 1) {
          y = part[grp][0][j];
#pragma unroll
          for (int p = 1; p < KS; p++) y += part[grp][p][j];
        }
        const uint32_t row = r0 + j;
        if (row < row_end) {
          if (EPI == EPI_STORE) act_out[(uint64_t)lc[0] + row] = y;
          else if (better(y, row, best_v, best_i)) { best_v = y; best_i = row; }
        }
      }
    }
    if (KS > 1) __syncthreads();
  }
  if (EPI == EPI_ARGMAX) {
    if (lane == 63) { red_v[wave] = best_v; red_i[wave] = best_i; }   // waves with kpart != 0 hold INVALID
    __syncthreads();
    if (tid == 0) {
      float bv = red_v[0]; uint32_t bi = red_i[0];
      for (int w = 1; w < 4; w++)
        if (better(red_v[w], red_i[w], bv, bi)) { bv = red_v[w]; bi = red_i[w]; }
      act_out[lidx[blockIdx.x]] = (float)(bi == INVALID_IDX ? 0u : bi);
      act_out[lval[blockIdx.x]] = bv;
    }
  }
}

// ---- generic path: any K, N, M, n_ops, base offset, group size; one wave per output ------------
template <bool Q4, bool TRANSPOSED>
__global__ void __launch_bounds__(256)
k_matmul_xq_generic(const float* act, float* out, const uint8_t* __restrict__ W,
                    const float2* __restrict__ qp, const uint32_t* __restrict__ la, const uint32_t* __restrict__ lb,
                    const uint32_t* __restrict__ lc, uint32_t M, uint32_t K, uint32_t N, uint32_t group,
                    uint64_t act_elems, uint64_t wt_elems) {
  const uint32_t lane = threadIdx.x & 63u, wave = threadIdx.x >> 6;
  const uint32_t col = blockIdx.x * 4u + wave, row = blockIdx.y, op = blockIdx.z;
  if (col >= N) return;
  const uint64_t a = (uint64_t)la[op] + (uint64_t)row * K, b = lb[op], c = (uint64_t)lc[op] + (uint64_t)row * N + col;
  float s = 0.f;
  for (uint32_t k = lane; k < K; k += 64u) {
    const uint64_t wi = TRANSPOSED ? b + (uint64_t)col * K + k : b + (uint64_t)k * N + col;
    if (a + k < act_elems && wi < wt_elems) s = fmaf(act[a + k], deq_elem(W, qp, wi, group, Q4), s);
  }
  s = wave_sum(s);
  if (lane == 0 && c < act_elems) out[c] = s;
}

template <bool Q4>
__global__ void __launch_bounds__(256)
k_matvec_argmax_generic(const float* act, float* out, const uint8_t* __restrict__ W,
                        const float2* __restrict__ qp, const uint32_t* __restrict__ la, const uint32_t* __restrict__ lb,
                        const uint32_t* __restrict__ lidx, const uint32_t* __restrict__ lval, uint32_t K, uint32_t N,
                        uint32_t group, uint32_t rows_per_group, uint64_t act_elems, uint64_t wt_elems) {
  __shared__ float red_v[4];
  __shared__ uint32_t red_i[4];
  const uint32_t lane = threadIdx.x & 63u, wave = threadIdx.x >> 6, grp = blockIdx.x;
  const uint32_t row0 = grp * rows_per_group, row1 = min(N, row0 + rows_per_group);
  const uint64_t a = la[0], b = lb[0];
  float bv = NEG_FLT_MAX; uint32_t bi = INVALID_IDX;
  for (uint32_t r = row0 + wave; r < row1; r += 4u) {
    float s = 0.f;
    for (uint32_t k = lane; k < K; k += 64u) {
      const uint64_t wi = b + (uint64_t)r * K + k;
      if (a + k < act_elems && wi < wt_elems) s = fmaf(act[a + k], deq_elem(W, qp, wi, group, Q4), s);
    }
    s = wave_sum(s);
    if (better(s, r, bv, bi)) { bv = s; bi = r; }
  }
  if (lane == 0) { red_v[wave] = bv; red_i[wave] = bi; }
  __syncthreads();
  if (threadIdx.x == 0) {
    for (int w = 1; w < 4; w++)
      if (better(red_v[w], red_i[w], bv, bi)) { bv = red_v[w]; bi = red_i[w]; }
    if (lidx[grp] < act_elems) out[lidx[grp]] = (float)(bi == INVALID_IDX ? 0u : bi);
    if (lval[grp] < act_elems) out[lval[grp]] = bv;
  }
}

// pass 2 (map_argmax_pairs.comp): best over the per-group (value, index) pairs
__global__ void __launch_bounds__(256)
k_argmax_pairs(float* __restrict__ act, const uint32_t* __restrict__ lidx, const uint32_t* __restrict__ lval,
               const uint32_t* __restrict__ ldst, uint32_t n_groups, uint64_t act_elems) {
  __shared__ float sv[256];
  __shared__ uint32_t si[256];
  const uint32_t tid = threadIdx.x;
  float bv = NEG_FLT_MAX; uint32_t bi = INVALID_IDX;
  for (uint32_t i = tid; i < n_groups; i += 256u) {
    if (lval[i] >= act_elems || lidx[i] >= act_elems) continue;
    float v = act[lval[i]];
    uint32_t idx = (uint32_t)(act[lidx[i]] + 0.5f);
    if (better(v, idx, bv, bi)) { bv = v; bi = idx; }
  }
  sv[tid] = bv; si[tid] = bi;
  __syncthreads();
  for (uint32_t s = 128; s > 0; s >>= 1) {
    if (tid < s && better(sv[tid + s], si[tid + s], sv[tid], si[tid])) { sv[tid] = sv[tid + s]; si[tid] = si[tid + s]; }
    __syncthreads();
  }
  if (tid == 0 && ldst[0] < act_elems) act[ldst[0]] = (float)(si[0] == INVALID_IDX ? 0u : si[0]);
}

// Dequantise with the block kernels' unpack code (one lane per 32-weight block), for tests.
template <int FMT>
__global__ void k_debug_dequant(const uint8_t* __restrict__ W, const float2* __restrict__ qp,
                                const __half* __restrict__ d16, uint64_t start, uint64_t count, float* __restrict__ out) {
  constexpr bool Q4 = (FMT == FMT_Q4_B16 || FMT == FMT_Q4_AFF);
  constexpr bool B16 = (FMT == FMT_Q4_B16 || FMT == FMT_Q8_B16);
  const uint64_t blk = (uint64_t)blockIdx.x * blockDim.x + threadIdx.x;
  const uint64_t g0 = start >> 5;
  if (blk * 32 >= count + (start & 31)) return;
  const uint64_t gidx = g0 + blk;
  float sc, zp;
  if (B16) { sc = __half2float(d16[gidx]); zp = (Q4 ? -8.0f : -128.0f) * sc; }
  else { float2 p = qp[gidx]; sc = p.x; zp = p.y; }
  float v[32];
  if (Q4) {
    uint4 q = *(const uint4*)(W + (gidx << 4));
    uint32_t w[4] = {q.x, q.y, q.z, q.w};
    for (int i = 0; i < 4; i++) {
      uint32_t lo = w[i] & 0x0F0F0F0Fu, hi = (w[i] >> 4) & 0x0F0F0F0Fu;
      v[i * 8 + 0] = ubyte_f32<0>(lo); v[i * 8 + 1] = ubyte_f32<0>(hi);
      v[i * 8 + 2] = ubyte_f32<1>(lo); v[i * 8 + 3] = ubyte_f32<1>(hi);
      v[i * 8 + 4] = ubyte_f32<2>(lo); v[i * 8 + 5] = ubyte_f32<2>(hi);
      v[i * 8 + 6] = ubyte_f32<3>(lo); v[i * 8 + 7] = ubyte_f32<3>(hi);
    }
  } else {
    const uint32_t* p = (const uint32_t*)(W + (gidx << 5));
    for (int i = 0; i < 8; i++) {
      uint32_t w = p[i];
      v[i * 4 + 0] = ubyte_f32<0>(w); v[i * 4 + 1] = ubyte_f32<1>(w);
      v[i * 4 + 2] = ubyte_f32<2>(w); v[i * 4 + 3] = ubyte_f32<3>(w);
    }
  }
  for (int j = 0; j < 32; j++) {
    const uint64_t e = gidx * 32 + j;
    if (e >= start && e - start < count) out[e - start] = __fadd_rn(__fmul_rn(v[j], sc), zp);
  }
}

// ---- host side -----------------------------------------------------------------------------------
struct XqArgs {
  Map *ma, *mw;
  const uint32_t *la, *lb, *lc;
};

// Block-kernel preconditions, checked against the host copies of the handles.
bool block_path_ok(const Map* ma, const Map* mw, uint32_t ha, uint32_t hb, uint32_t K, uint32_t N,
                          uint64_t* a_out, uint64_t* b_out) {
  if (mw->group_size != 32 || mw->pack_size != 1 || ma->pack_size != 1) return false;
  if (K == 0 || (K & 31u) || K > 16384) return false;
  const uint32_t* a = res_host(ha, 1);
  const uint32_t* b = res_host(hb, 1);
  if (!a || !b) return false;
  if (b[0] & 31u) return false;
  if (!in_range(a[0], K, ma->n_elems) || !in_range(b[0], (uint64_t)N * K, mw->n_elems)) return false;
  *a_out = a[0]; *b_out = b[0];
  return true;
}

int fmt_of(const Map* mw, uint64_t b, uint64_t n_w) {
  const bool q4 = mw->dtype == DTYPE_Q4;
  const bool b16 = (b + n_w + 31) / 32 <= mw->block16_groups;
  return q4 ? (b16 ? FMT_Q4_B16 : FMT_Q4_AFF) : (b16 ? FMT_Q8_B16 : FMT_Q8_AFF);
}

// Behaviour switches of the library (each selects between code paths that the parity tests run both ways):
// read from the environment at every call, so a test can flip one between two ops.
int tuning(const char* name, int dflt) {
  const char* v = getenv(name);
  return v ? atoi(v) : dflt;
}
// Launch-shape numbers (waves per workgroup, rows per pass, ...): fixed in the library as built; a build with
// -DADAMAH_TUNING reads them from the environment for sweeps.
int knob(const char* name, int dflt) {
#ifdef ADAMAH_TUNING
  const char* v = getenv(name);
  return v ? atoi(v) : dflt;
#else
  (void)name;
  return dflt;
#endif
}

template <int EPI>
static int launch_block(int fmt, const Map* ma, const Map* mw, const uint32_t* la, const uint32_t* lb,
                        const uint32_t* lc, const uint32_t* lidx, const uint32_t* lval, uint32_t K, uint32_t N,
                        uint32_t rows_per_group) {
  const uint32_t n_groups = cdiv(N, rows_per_group);
  const size_t smem = (size_t)K * 4 + (size_t)(K >> 5) * 4;
  const uint32_t per_cu = (uint32_t)knob("ADAMAH_GEMV_PERCU", smem > 40000 ? 2 : 4);
  const uint32_t grid = std::min<uint32_t>(n_groups, (uint32_t)g.n_cu * per_cu);
  float* act = (float*)ma->buf;
#define LAUNCH(F)                                                                                              \
  k_gemv_block<F, EPI, 4><<<grid, 256, smem, g.stream>>>(act, act, mw->buf, mw->qp, mw->d16, la, lb, lc, lidx,  \
                                                        lval, K, N, rows_per_group, n_groups)
  switch (fmt) {
    case FMT_Q4_B16: LAUNCH(FMT_Q4_B16); break;
    case FMT_Q4_AFF: LAUNCH(FMT_Q4_AFF); break;
    case FMT_Q8_B16: LAUNCH(FMT_Q8_B16); break;
    default: LAUNCH(FMT_Q8_AFF); break;
  }
#undef LAUNCH
  count_launch();
  return check_launch();
}

// Register-resident variant: K up to 16384.  For EPI_STORE rows_per_wg is chosen here; for
// EPI_ARGMAX one workgroup handles one argmax group (rows_per_wg = rows_per_group).
template <int EPI, int FMT>
static int launch_regx_fmt(const Map* ma, const Map* mw, const uint32_t* la, const uint32_t* lb, const uint32_t* lc,
                           const uint32_t* lidx, const uint32_t* lval, uint32_t K, uint32_t N, uint32_t rows_per_wg) {
  float* act = (float*)ma->buf;
  const uint32_t nblk = K >> 5;
  const uint32_t grid = cdiv(N, rows_per_wg);
#define RX(NB, KS)                                                                                             \
  k_gemv_regx<FMT, EPI, NB, KS><<<grid, 256, 0, g.stream>>>(act, act, mw->buf, mw->qp, mw->d16, la, lb, lc, lidx, \
                                                            lval, K, N, rows_per_wg)
  if (nblk <= 64) RX(1, 1);
  else if (nblk <= 128) RX(2, 1);
  else if (nblk <= 256) RX(2, 2);
  else RX(2, 4);
#undef RX
  count_launch();
  return check_launch();
}
template <int EPI>
static int launch_regx(int fmt, const Map* ma, const Map* mw, const uint32_t* la, const uint32_t* lb,
                       const uint32_t* lc, const uint32_t* lidx, const uint32_t* lval, uint32_t K, uint32_t N,
                       uint32_t rows_per_wg) {
  switch (fmt) {
    case FMT_Q4_B16: return launch_regx_fmt<EPI, FMT_Q4_B16>(ma, mw, la, lb, lc, lidx, lval, K, N, rows_per_wg);
    case FMT_Q4_AFF: return launch_regx_fmt<EPI, FMT_Q4_AFF>(ma, mw, la, lb, lc, lidx, lval, K, N, rows_per_wg);
    case FMT_Q8_B16: return launch_regx_fmt<EPI, FMT_Q8_B16>(ma, mw, la, lb, lc, lidx, lval, K, N, rows_per_wg);
    default: return launch_regx_fmt<EPI, FMT_Q8_AFF>(ma, mw, la, lb, lc, lidx, lval, K, N, rows_per_wg);
  }
}

int op_matmul_t_xq(uint32_t dtype, uint32_t map_act, uint32_t map_wt, uint32_t ha, uint32_t hb, uint32_t hc,
                   uint32_t M, uint32_t K, uint32_t N, uint32_t n_ops, bool transposed) {
  Map* ma = get_map(map_act);
  Map* mw = get_map(map_wt);
  if (!ma || !mw) return ADAMAH_ERR_INVALID;
  if (n_ops == 0 || N == 0 || M == 0) return ADAMAH_OK;
  if (ma->dtype != DTYPE_F32 || mw->dtype != dtype || !mw->qp || mw->group_size == 0) return ADAMAH_ERR_INVALID;
  const uint32_t *la = res_u32(ha, n_ops), *lb = res_u32(hb, n_ops), *lc = res_u32(hc, n_ops);
  if (!la || !lb || !lc) return ADAMAH_ERR_INVALID;
  // reject operands the host can see are out of range (handles written by the device are
  // bounds-checked inside the generic kernel instead)
  const uint32_t *ah = res_host(ha, n_ops), *bh = res_host(hb, n_ops), *ch = res_host(hc, n_ops);
  for (uint32_t op = 0; op < n_ops; op++) {
    if (ah && !in_range(ah[op], (uint64_t)M * K, ma->n_elems)) return ADAMAH_ERR_INVALID;
    if (bh && !in_range(bh[op], (uint64_t)N * K, mw->n_elems)) return ADAMAH_ERR_INVALID;
    if (ch && !in_range(ch[op], (uint64_t)M * N, ma->n_elems)) return ADAMAH_ERR_INVALID;
  }
  uint64_t a0 = 0, b0 = 0;
  if (transposed && M == 1 && n_ops == 1 && ch && block_path_ok(ma, mw, ha, hb, K, N, &a0, &b0)) {
    const int fmt = fmt_of(mw, b0, (uint64_t)N * K);
    // Q4: int8 matrix-instruction kernel.  Q8 (and Q4 on request): float32 kernels, activations in
    // registers with waves sharing a row when K > 8192, else staged in LDS
    const int impl = tuning("ADAMAH_GEMV_IMPL", mfma_path_ok(mw, K) ? 3 : K > 8192 ? 1 : 0);
    if (impl == 3 && mfma_path_ok(mw, K)) {
      if (can_defer()) {   // queue it: neighbouring row-wise ops may be folded into the launch
        PendOp p;
        p.kind = PK_GEMV; p.map_act = map_act; p.map_wt = map_wt; p.a = (uint32_t)a0; p.b = (uint32_t)b0; p.c = ch[0];
        p.k = K; p.n = N; p.op = (uint32_t)fmt;
        g.pend.push_back(p);
        return ADAMAH_OK;
      }
      flush_pending();
      return launch_mfma_store(fmt, ma, mw, (uint32_t)a0, (uint32_t)b0, ch[0], K, N);
    }
    flush_pending();
    if (impl == 1) {
      const uint32_t ks = K <= 4096 ? 1 : K <= 8192 ? 2 : 4;
      const uint32_t step = (4 / ks) * 4;                       // rows one workgroup pass covers
      const uint32_t passes = (uint32_t)knob("ADAMAH_GEMV_PASSES", 2);
      return launch_regx<EPI_STORE>(fmt, ma, mw, la, lb, lc, nullptr, nullptr, K, N, step * std::max(1u, passes));
    }
    if ((uint64_t)K * 4 + (K >> 5) * 4 > 64000) goto generic;
    return launch_block<EPI_STORE>(fmt, ma, mw, la, lb, lc, nullptr, nullptr, K, N,
                                   (uint32_t)knob("ADAMAH_GEMV_RPG", 16));
  }
  // several activation rows over Q4_0 blocks: fp16 matrix-core GEMM
  // (Q8_0 blocks: up to 32 rows)
  if (transposed && M > 1 && (dtype == DTYPE_Q4 || M <= 32) && mw->group_size == 32 && K >= 128 && (K & 127u) == 0 && ah && bh &&
      ch && mw->pack_size == 1 && ma->pack_size == 1 && tuning("ADAMAH_GEMM_IMPL", 1) == 1) {
    const int want = dtype == DTYPE_Q4 ? FMT_Q4_B16 : FMT_Q8_B16;
    bool ok = true;
    for (uint32_t op = 0; ok && op < n_ops; op++)
      ok = (bh[op] & 31u) == 0 && fmt_of(mw, bh[op], (uint64_t)N * K) == want;
    if (ok && n_ops == 1 && can_defer() && tuning("ADAMAH_GEMM_MERGE", 1) != 0) {
      // queued: matmuls over the same rows whose matrices lie back to back (Q, K, V; gate, up) become one launch
      PendOp p;
      p.kind = PK_GEMM; p.map_act = map_act; p.map_wt = map_wt; p.a = ah[0]; p.b = bh[0]; p.c = ch[0]; p.rpg = M; p.k = K;
      p.n = N; p.op = (uint32_t)want; p.h[0] = ha; p.h[1] = hb; p.h[2] = hc;
      g.pend.push_back(p);
      return ADAMAH_OK;
    }
    if (ok) {
      flush_pending();
      return launch_gemm_q4_mfma(ma, mw, la, lb, lc, M, K, N, n_ops, dtype == DTYPE_Q8, nullptr,
                                 n_ops == 1 ? (int64_t)ah[0] : -1, n_ops == 1 ? (int64_t)ch[0] : -1);
    }
  }
generic:
  flush_pending();
  dim3 grid(cdiv(N, 4), M, n_ops);
  float* act = (float*)ma->buf;
  const bool q4 = dtype == DTYPE_Q4;
#define GEN(Q, T)                                                                                             \
  k_matmul_xq_generic<Q, T><<<grid, 256, 0, g.stream>>>(act, act, mw->buf, mw->qp, la, lb, lc, M, K, N,        \
                                                        mw->group_size, ma->n_elems, mw->n_elems)
  if (q4) { if (transposed) GEN(true, true); else GEN(true, false); }
  else { if (transposed) GEN(false, true); else GEN(false, false); }
#undef GEN
  count_launch();
  return check_launch();
}

int op_matvec_argmax(uint32_t dtype, uint32_t map_act, uint32_t map_wt, uint32_t ha, uint32_t hb, uint32_t hidx,
                     uint32_t hval, uint32_t hdst, uint32_t K, uint32_t N, uint32_t rows_per_group) {
  Map* ma = get_map(map_act);
  Map* mw = get_map(map_wt);
  if (!ma || !mw) return ADAMAH_ERR_INVALID;
  if (N == 0) return ADAMAH_OK;
  if (rows_per_group == 0) return ADAMAH_ERR_INVALID;
  if (ma->dtype != DTYPE_F32 || mw->dtype != dtype || !mw->qp || mw->group_size == 0) return ADAMAH_ERR_INVALID;
  const uint32_t n_groups = cdiv(N, rows_per_group);
  const uint32_t *la = res_u32(ha, 1), *lb = res_u32(hb, 1), *lidx = res_u32(hidx, n_groups),
                 *lval = res_u32(hval, n_groups), *ldst = res_u32(hdst, 1);
  if (!la || !lb || !lidx || !lval || !ldst) return ADAMAH_ERR_INVALID;
  const uint32_t *ih = res_host(hidx, n_groups), *vh = res_host(hval, n_groups), *dh = res_host(hdst, 1);
  bool locs_ok = ih && vh && dh && dh[0] < ma->n_elems;
  for (uint32_t i = 0; locs_ok && i < n_groups; i++) locs_ok = ih[i] < ma->n_elems && vh[i] < ma->n_elems;
  if (ih && vh && dh && !locs_ok) return ADAMAH_ERR_INVALID;
  uint64_t a0 = 0, b0 = 0;
  int r;
  if (locs_ok && block_path_ok(ma, mw, ha, hb, K, N, &a0, &b0)) {
    const int impl = tuning("ADAMAH_GEMV_IMPL", mfma_path_ok(mw, K) ? 3 : K > 8192 ? 1 : 0);
    if (impl == 3 && mfma_path_ok(mw, K) && can_defer()) {
      PendOp p;
      p.kind = PK_ARGMAX; p.map_act = map_act; p.map_wt = map_wt; p.a = (uint32_t)a0; p.b = (uint32_t)b0; p.k = K; p.n = N;
      p.op = (uint32_t)fmt_of(mw, b0, (uint64_t)N * K); p.h[0] = hidx; p.h[1] = hval; p.h[2] = hdst; p.h[3] = ha; p.h[4] = hb;
      p.rpg = rows_per_group;
      g.pend.push_back(p);
      return ADAMAH_OK;
    }
    if (impl != 3 && fmt_of(mw, b0, (uint64_t)N * K) == FMT_Q8_B16 && K >= 128 && (K & 127u) == 0 && can_defer() &&
        tuning("ADAMAH_ARGMAX_RUN", 1) != 0) {
      // queued so that the LM head passes of several sequences can share one read of the matrix
      PendOp p;
      p.kind = PK_ARGMAX; p.map_act = map_act; p.map_wt = map_wt; p.a = (uint32_t)a0; p.b = (uint32_t)b0; p.k = K; p.n = N;
      p.op = FMT_Q8_B16; p.h[0] = hidx; p.h[1] = hval; p.h[2] = hdst; p.h[3] = ha; p.h[4] = hb; p.rpg = rows_per_group;
      g.pend.push_back(p);
      return ADAMAH_OK;
    }
    flush_pending();
    if (impl == 3 && mfma_path_ok(mw, K))
      r = launch_mfma_argmax(fmt_of(mw, b0, (uint64_t)N * K), ma, mw, (uint32_t)a0, (uint32_t)b0, lidx, lval, K, N,
                             rows_per_group);
    else if (impl == 1)
      r = launch_regx<EPI_ARGMAX>(fmt_of(mw, b0, (uint64_t)N * K), ma, mw, la, lb, nullptr, lidx, lval, K, N,
                                  rows_per_group);
    else
      r = launch_block<EPI_ARGMAX>(fmt_of(mw, b0, (uint64_t)N * K), ma, mw, la, lb, nullptr, lidx, lval, K, N,
                                   rows_per_group);
  } else {
    flush_pending();
    const uint32_t *ah = res_host(ha, 1), *bh = res_host(hb, 1);
    if (ah && !in_range(ah[0], K, ma->n_elems)) return ADAMAH_ERR_INVALID;
    if (bh && !in_range(bh[0], (uint64_t)N * K, mw->n_elems)) return ADAMAH_ERR_INVALID;
    float* act = (float*)ma->buf;
    if (dtype == DTYPE_Q4)
      k_matvec_argmax_generic<true><<<n_groups, 256, 0, g.stream>>>(act, act, mw->buf, mw->qp, la, lb, lidx, lval, K, N,
                                                                    mw->group_size, rows_per_group, ma->n_elems,
                                                                    mw->n_elems);
    else
      k_matvec_argmax_generic<false><<<n_groups, 256, 0, g.stream>>>(act, act, mw->buf, mw->qp, la, lb, lidx, lval, K,
                                                                     N, mw->group_size, rows_per_group, ma->n_elems,
                                                                     mw->n_elems);
    count_launch();
    r = check_launch();
  }
  if (r) return r;
  return launch_argmax_pairs(ma, lidx, lval, ldst, n_groups);
}

// A queued Q8 GEMV + argmax that did not join a run: the float32 block kernels, as when launched at once.
// The block-layout GEMV with its result rows written to `out` (device memory outside the maps: the scratch logits of
// the GEMV + top-k ops) instead of a range of the activation map.  The kernel adds the row number to the word behind
// `lc`: a word of the zero-initialised counter block that no kernel ever writes (ZERO_WORD; the ticket counter of the
// GEMV prologues is word 0 of that block) serves as that word.
int launch_block_store_to(int fmt, const Map* ma, const Map* mw, const uint32_t* la, const uint32_t* lb, uint32_t K,
                          uint32_t N, float* out) {
  const size_t smem = (size_t)K * 4 + (size_t)(K >> 5) * 4;
  if (smem > 64000 || !g.sync_ctr) return ADAMAH_ERR_INVALID;
  const uint32_t rpg = (uint32_t)knob("ADAMAH_GEMV_RPG", 16), n_groups = cdiv(N, rpg);
  const uint32_t per_cu = (uint32_t)knob("ADAMAH_GEMV_PERCU", smem > 40000 ? 2 : 4);
  const uint32_t grid = std::min<uint32_t>(n_groups, (uint32_t)g.n_cu * per_cu);
  const float* act = (const float*)ma->buf;
  const uint32_t* zero = (const uint32_t*)g.sync_ctr + ZERO_WORD;
#define LAUNCH(F)                                                                                                \
  k_gemv_block<F, EPI_STORE, 4><<<grid, 256, smem, g.stream>>>(act, out, mw->buf, mw->qp, mw->d16, la, lb, zero, nullptr, \
                                                              nullptr, K, N, rpg, n_groups)
  switch (fmt) {
    case FMT_Q4_B16: LAUNCH(FMT_Q4_B16); break;
    case FMT_Q4_AFF: LAUNCH(FMT_Q4_AFF); break;
    case FMT_Q8_B16: LAUNCH(FMT_Q8_B16); break;
    default: LAUNCH(FMT_Q8_AFF); break;
  }
#undef LAUNCH
  count_launch();
  return check_launch();
}

int launch_argmax_direct(const PendOp& p) {
  Map* ma = get_f32_map(p.map_act);
  Map* mw = get_map(p.map_wt);
  const uint32_t n_groups = cdiv(p.n, p.rpg);
  const uint32_t *la = res_u32(p.h[3], 1), *lb = res_u32(p.h[4], 1), *lidx = res_u32(p.h[0], n_groups),
                 *lval = res_u32(p.h[1], n_groups), *ldst = res_u32(p.h[2], 1);
  if (!ma || !mw || !la || !lb || !lidx || !lval || !ldst) return ADAMAH_ERR_INVALID;
  int r;
  if (p.k > 8192) r = launch_regx<EPI_ARGMAX>((int)p.op, ma, mw, la, lb, nullptr, lidx, lval, p.k, p.n, p.rpg);
  else r = launch_block<EPI_ARGMAX>((int)p.op, ma, mw, la, lb, nullptr, lidx, lval, p.k, p.n, p.rpg);
  if (r) return r;
  return launch_argmax_pairs(ma, lidx, lval, ldst, n_groups);
}

int launch_argmax_pairs(const Map* ma, const uint32_t* lidx, const uint32_t* lval, const uint32_t* ldst,
                        uint32_t n_groups) {
  k_argmax_pairs<<<1, 256, 0, g.stream>>>((float*)ma->buf, lidx, lval, ldst, n_groups, ma->n_elems);
  count_launch();
  return check_launch();
}

}  // namespace adamah

using namespace adamah;

extern "C" {

int map_matmul_t_xq4_dev(uint32_t ma, uint32_t mw, uint32_t a, uint32_t b, uint32_t c, uint32_t M, uint32_t K,
                         uint32_t N, uint32_t n_ops) {
  return op_matmul_t_xq(DTYPE_Q4, ma, mw, a, b, c, M, K, N, n_ops, true);
}
int map_matmul_xq4_dev(uint32_t ma, uint32_t mw, uint32_t a, uint32_t b, uint32_t c, uint32_t M, uint32_t K,
                       uint32_t N, uint32_t n_ops) {
  return op_matmul_t_xq(DTYPE_Q4, ma, mw, a, b, c, M, K, N, n_ops, false);
}
int map_matmul_t_xq8_dev(uint32_t ma, uint32_t mw, uint32_t a, uint32_t b, uint32_t c, uint32_t M, uint32_t K,
                         uint32_t N, uint32_t n_ops) {
  return op_matmul_t_xq(DTYPE_Q8, ma, mw, a, b, c, M, K, N, n_ops, true);
}
int map_matmul_xq8_dev(uint32_t ma, uint32_t mw, uint32_t a, uint32_t b, uint32_t c, uint32_t M, uint32_t K,
                       uint32_t N, uint32_t n_ops) {
  return op_matmul_t_xq(DTYPE_Q8, ma, mw, a, b, c, M, K, N, n_ops, false);
}
int map_matvec_argmax_t_xq4_dev(uint32_t ma, uint32_t mw, uint32_t a, uint32_t b, uint32_t idx, uint32_t val,
                                uint32_t dst, uint32_t K, uint32_t N, uint32_t rpg) {
  return op_matvec_argmax(DTYPE_Q4, ma, mw, a, b, idx, val, dst, K, N, rpg);
}
int map_matvec_argmax_t_xq8_dev(uint32_t ma, uint32_t mw, uint32_t a, uint32_t b, uint32_t idx, uint32_t val,
                                uint32_t dst, uint32_t K, uint32_t N, uint32_t rpg) {
  return op_matvec_argmax(DTYPE_Q8, ma, mw, a, b, idx, val, dst, K, N, rpg);
}

int adamah_hip_debug_dequant(uint32_t map_id, uint64_t start, uint64_t count, float* out) { ADAMAH_API();
  Map* m = get_map(map_id);
  if (!m || !m->qp || m->group_size != 32 || !out || count == 0 || !in_range(start, count, m->n_elems))
    return ADAMAH_ERR_INVALID;
  float* d = nullptr;
  if (hipMalloc((void**)&d, count * sizeof(float)) != hipSuccess) return ADAMAH_ERR_MEMORY;
  const uint64_t nb = (count + (start & 31) + 31) / 32;
  const int fmt = fmt_of(m, start, count);
  const uint32_t grid = cdiv(nb, 64);
  switch (fmt) {
    case FMT_Q4_B16: k_debug_dequant<FMT_Q4_B16><<<grid, 64, 0, g.stream>>>(m->buf, m->qp, m->d16, start, count, d); break;
    case FMT_Q4_AFF: k_debug_dequant<FMT_Q4_AFF><<<grid, 64, 0, g.stream>>>(m->buf, m->qp, m->d16, start, count, d); break;
    case FMT_Q8_B16: k_debug_dequant<FMT_Q8_B16><<<grid, 64, 0, g.stream>>>(m->buf, m->qp, m->d16, start, count, d); break;
    default: k_debug_dequant<FMT_Q8_AFF><<<grid, 64, 0, g.stream>>>(m->buf, m->qp, m->d16, start, count, d); break;
  }
  int r = check_launch();
  if (!r) r = d2h(out, d, count * sizeof(float));
  hipStreamSynchronize(g.stream);
  hipFree(d);
  return r;
}

}  // extern "C"
