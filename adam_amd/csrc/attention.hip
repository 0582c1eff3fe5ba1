// Decode attention behind the reference's two entry points: score rows (q . K^T per head, through
// map_matmul_t_dev) and softmax(prep(scores)) . V (map_attn_softmax_value_dev).
//
// Reference: shaders/src/f32/map_matmul_t.comp, map_attn_softmax_value.comp:39-89 (dispatch
// adamah.c:6682-6781, 7894-8059), prep(s) = cap*tanh(s*scale/cap) when cap > 0 else s*scale.
// The reference keeps all probabilities of a row in 2048 floats of shared memory and returns
// without output for longer rows; here the row is split over workgroups with an online-softmax
// merge (running max m, sum l, weighted values o), so any length works.  K/V rows are read from
// the fp16 copy of the KV range when the operands lie inside it, else from the float32 map.
#include "common.h"
#include "attn_common.h"
#include "../../include/adamah_hip.h"
#include <algorithm>

extern "C" int map_matmul_t_dev(uint32_t map_id, uint32_t ha, uint32_t hb, uint32_t hc, uint32_t M, uint32_t K, uint32_t N,
                                uint32_t n_ops);

namespace adamah {


__device__ __forceinline__ float ld(const float* p, uint64_t i) { return p[i]; }
__device__ __forceinline__ float ld(const __half* p, uint64_t i) { return __half2float(p[i]); }

__device__ __forceinline__ float wave_sum64(float v) {
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) v += __shfl_xor(v, o, 64);
  return v;
}
__device__ __forceinline__ float wave_max64(float v) {
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) v = fmaxf(v, __shfl_xor(v, o, 64));
  return v;
}

// C[M,N] = A[M,K] . B[N,K]^T per op; one wave per output column, lanes over K.
// B is read through `bsrc` (float map or fp16 KV copy, index = element - b_shift).
template <typename TB>
__global__ void __launch_bounds__(256)
k_matmul_t(const float* A, float* C, const TB* bsrc, uint64_t b_shift, const uint32_t* __restrict__ la,
           const uint32_t* __restrict__ lb, const uint32_t* __restrict__ lc, uint32_t M, uint32_t K, uint32_t N,
           uint64_t a_elems, uint64_t b_elems) {
  const uint32_t lane = threadIdx.x & 63u, wave = threadIdx.x >> 6;
  const uint32_t col = blockIdx.x * 4u + wave, row = blockIdx.y, op = blockIdx.z;
  if (col >= N) return;
  const uint64_t a = (uint64_t)la[op] + (uint64_t)row * K, b = (uint64_t)lb[op] + (uint64_t)col * K;
  const uint64_t c = (uint64_t)lc[op] + (uint64_t)row * N + col;
  float s = 0.f;
  if (a + K <= a_elems && b >= b_shift && b - b_shift + K <= b_elems)
    for (uint32_t k = lane; k < K; k += 64u) s = fmaf(A[a + k], ld(bsrc, b - b_shift + k), s);
  s = wave_sum64(s);
  if (lane == 0 && c < a_elems) C[c] = s;
}

// Decode scores, M == 1: out[op][t] = q_op . B_op[t].  LPR lanes share one B row (VEC contiguous
// elements per 16-byte load, up to 4 loads per lane), 64/LPR rows per wave step; each lane keeps
// its slice of the query in registers.  Needs K % VEC == 0, K <= 4*LPR*VEC and VEC-aligned bases.
template <typename TB, int VEC>
__global__ void __launch_bounds__(256)
k_scores_vec(const float* A, float* C, const TB* bsrc, uint64_t b_shift, const uint32_t* __restrict__ la,
             const uint32_t* __restrict__ lb, const uint32_t* __restrict__ lc, uint32_t K, uint32_t N, uint32_t lpr,
             uint32_t rows_per_wg) {
  const uint32_t lane = threadIdx.x & 63u, wave = threadIdx.x >> 6, op = blockIdx.y;
  const uint32_t sub = lane % lpr, rslot = lane / lpr, rpw = 64u / lpr;   // lane's column slice / row slot
  const uint64_t a = la[op], b = (uint64_t)lb[op] - b_shift, c = lc[op];
  const uint32_t nvec = K / VEC;                                         // vectors per row
  float q[4][VEC];
#pragma unroll
  for (int i = 0; i < 4; i++) {
    const uint32_t v = sub + i * lpr;
#pragma unroll
    for (int j = 0; j < VEC; j++) q[i][j] = v < nvec ? A[a + (uint64_t)v * VEC + j] : 0.f;
  }
  const uint32_t row0 = blockIdx.x * rows_per_wg, row1 = min(N, row0 + rows_per_wg);
  for (uint32_t rb = row0 + wave * rpw; rb < row1; rb += 4u * rpw) {
    const uint32_t r = rb + rslot;
    float s = 0.f;
    if (r < row1) {
#pragma unroll
      for (int i = 0; i < 4; i++) {
        const uint32_t v = sub + i * lpr;
        if (v < nvec) {
          const TB* bp = bsrc + b + (uint64_t)r * K + (uint64_t)v * VEC;
          if (VEC == 8) {
            const uint4 raw = *(const uint4*)bp;
            const __half2* h = (const __half2*)&raw;
#pragma unroll
            for (int j = 0; j < 4; j++) {
              const float2 f = __half22float2(h[j]);
              s = fmaf(q[i][2 * j], f.x, s);
              s = fmaf(q[i][2 * j + 1], f.y, s);
            }
          } else {
            const float4 f = *(const float4*)bp;
            s = fmaf(q[i][0], f.x, s); s = fmaf(q[i][1], f.y, s);
            s = fmaf(q[i][2], f.z, s); s = fmaf(q[i][3], f.w, s);
          }
        }
      }
    }
    for (uint32_t o = lpr >> 1; o > 0; o >>= 1) s += __shfl_xor(s, o, 64);
    if (r < row1 && sub == 0) C[c + r] = s;
  }
}

// C = A[M,K] . B[K,N] (non-transposed B), same indexing conventions.
__global__ void __launch_bounds__(256)
k_matmul_nt(const float* A, float* C, const float* B, const uint32_t* __restrict__ la, const uint32_t* __restrict__ lb,
            const uint32_t* __restrict__ lc, uint32_t M, uint32_t K, uint32_t N, uint64_t a_elems, uint64_t b_elems) {
  const uint32_t lane = threadIdx.x & 63u, wave = threadIdx.x >> 6;
  const uint32_t col = blockIdx.x * 4u + wave, row = blockIdx.y, op = blockIdx.z;
  if (col >= N) return;
  const uint64_t a = (uint64_t)la[op] + (uint64_t)row * K, b = lb[op];
  const uint64_t c = (uint64_t)lc[op] + (uint64_t)row * N + col;
  float s = 0.f;
  for (uint32_t k = lane; k < K; k += 64u) {
    const uint64_t bi = b + (uint64_t)k * N + col;
    if (a + k < a_elems && bi < b_elems) s = fmaf(A[a + k], B[bi], s);
  }
  s = wave_sum64(s);
  if (lane == 0 && c < a_elems) C[c] = s;
}


#define ATT_CHUNK 1024   // most score rows one workgroup handles (LDS array size)

// grid (n_splits, n_ops).  Workgroup (split s, op): rows [s*ATT_CHUNK, ...) of the op's score row.
// Writes either the normalised output (n_splits == 1) or the partial (m, l, o[value_dim]).
template <typename TV, int VEC>
__global__ void __launch_bounds__(256)
k_attn_softmax_value(const float* data, float* out, const TV* vsrc, uint64_t v_shift, const uint32_t* __restrict__ lsc,
                     const uint32_t* __restrict__ lv, const uint32_t* __restrict__ lo, uint32_t row_size,
                     uint32_t value_dim, float scale, float cap, uint32_t n_splits, uint32_t chunk, float* partial,
                     uint64_t n_elems, uint64_t v_elems) {
  __shared__ float p[ATT_CHUNK];
  __shared__ float red[4];
  __shared__ float osum[VEC > 1 ? 2048 : 256];
  const uint32_t tid = threadIdx.x, lane = tid & 63u, wave = tid >> 6;
  const uint32_t split = blockIdx.x, op = blockIdx.y;
  const uint32_t t0 = split * chunk, t1 = min(row_size, t0 + chunk), nt = t1 - t0;
  const uint64_t sb = lsc[op], vb = lv[op], ob = lo[op];
  const bool ok = sb + row_size <= n_elems && vb >= v_shift &&
                  vb - v_shift + (uint64_t)row_size * value_dim <= v_elems && ob + value_dim <= n_elems;
  // pass 1: chunk maximum of prep(score)
  float mx = -9.99999968e+37f;
  if (ok)
    for (uint32_t t = tid; t < nt; t += 256u) {
      const float v = prep(data[sb + t0 + t], scale, cap);
      p[t] = v;
      mx = fmaxf(mx, v);
    }
  mx = wave_max64(mx);
  if (lane == 0) red[wave] = mx;
  __syncthreads();
  mx = fmaxf(fmaxf(red[0], red[1]), fmaxf(red[2], red[3]));
  __syncthreads();
  // pass 2: exponentials and their sum
  float sum = 0.f;
  if (ok)
    for (uint32_t t = tid; t < nt; t += 256u) {
      const float e = expf(p[t] - mx);
      p[t] = e;
      sum += e;
    }
  sum = wave_sum64(sum);
  if (lane == 0) red[wave] = sum;
  __syncthreads();
  sum = (red[0] + red[1]) + (red[2] + red[3]);
  if (VEC > 1) {
    // pass 3, vector form: lpr = value_dim/VEC lanes cover one V row with 16-byte loads, 256/lpr rows
    // are in flight per sweep, four sweeps unrolled; row-slot partials meet in LDS.
    const uint32_t lpr = value_dim / VEC, slots = 256u / lpr, sub = tid % lpr, slot = tid / lpr;
    float acc[VEC];
#pragma unroll
    for (int j = 0; j < VEC; j++) acc[j] = 0.f;
    if (ok && slot < slots) {
      const TV* base = vsrc + (vb - v_shift) + (uint64_t)t0 * value_dim + (uint64_t)sub * VEC;
#pragma unroll 4
      for (uint32_t t = slot; t < nt; t += slots) {
        const float w = p[t];
        if (VEC == 8) {
          const uint4 raw = *(const uint4*)(base + (uint64_t)t * value_dim);
          const __half2* h = (const __half2*)&raw;
#pragma unroll
          for (int j = 0; j < 4; j++) {
            const float2 f = __half22float2(h[j]);
            acc[2 * j] = fmaf(w, f.x, acc[2 * j]);
            acc[2 * j + 1] = fmaf(w, f.y, acc[2 * j + 1]);
          }
        } else {
          const float4 f = *(const float4*)(base + (uint64_t)t * value_dim);
          acc[0] = fmaf(w, f.x, acc[0]); acc[1] = fmaf(w, f.y, acc[1]);
          acc[2] = fmaf(w, f.z, acc[2]); acc[3] = fmaf(w, f.w, acc[3]);
        }
      }
    }
    // reduce the row slots: osum holds up to 2048 floats, so fold slots in rounds of (2048/value_dim)
    const uint32_t fit = 2048u / value_dim;
    float o = 0.f;
    for (uint32_t s0 = 0; s0 < slots; s0 += fit) {
      if (slot >= s0 && slot < s0 + fit && slot < slots) {
#pragma unroll
        for (int j = 0; j < VEC; j++) osum[(slot - s0) * value_dim + sub * VEC + j] = acc[j];
      }
      __syncthreads();
      if (tid < value_dim)
        for (uint32_t s = 0; s < fit && s0 + s < slots; s++) o += osum[s * value_dim + tid];
      __syncthreads();
    }
    if (tid < value_dim && ok) {
      if (n_splits == 1) out[ob + tid] = o * (1.0f / sum);
      else partial[((uint64_t)op * n_splits + split) * (value_dim + 2) + 2 + tid] = o;
    }
    if (n_splits > 1 && tid == 0) {
      float* pp = partial + ((uint64_t)op * n_splits + split) * (value_dim + 2);
      pp[0] = mx;
      pp[1] = sum;
    }
    return;
  }
  // pass 3: o[d] = sum_t p[t] * V[t][d]; thread (slot, d): slot strides the rows
  const uint32_t dpw = min(value_dim, 256u);       // columns handled per sweep
  const uint32_t slots = 256u / dpw;               // rows in flight per sweep
  for (uint32_t d0 = 0; d0 < value_dim; d0 += 256u) {
    const uint32_t d = d0 + tid % dpw, slot = tid / dpw;
    float acc = 0.f;
    if (ok && d < value_dim && slot < slots) {
      const uint64_t base = vb - v_shift + (uint64_t)t0 * value_dim + d;
      for (uint32_t t = slot; t < nt; t += slots) acc = fmaf(p[t], ld(vsrc, base + (uint64_t)t * value_dim), acc);
    }
    osum[tid] = acc;
    __syncthreads();
    if (tid < dpw && d0 + tid < value_dim && ok) {
      float o = 0.f;
      for (uint32_t s = 0; s < slots; s++) {
        o += osum[s * dpw + tid];
      }
      if (n_splits == 1) out[ob + d0 + tid] = o * (1.0f / sum);
      else partial[((uint64_t)op * n_splits + split) * (value_dim + 2) + 2 + d0 + tid] = o;
    }
    __syncthreads();
  }
  if (n_splits > 1 && tid == 0) {
    float* pp = partial + ((uint64_t)op * n_splits + split) * (value_dim + 2);
    pp[0] = mx;
    pp[1] = sum;
  }
}

// Scores and softmax . V of one chunk of the sequence in one launch (fp16 K and V rows, 8 elements
// per 16-byte load): the two kernels above back to back inside a workgroup, with the prepared scores
// handed over in LDS instead of through the score row in memory.  The raw scores are still stored
// where the stand-alone score kernel would put them.  grid (n_splits, n_ops); lpr lanes share a K
// row, vlpr = value_dim / 8 lanes a V row.
template <int LPR>
__global__ void __launch_bounds__(256)
k_attn_fused(const float* data, float* out, const __half* kv, uint64_t kv_shift, const uint32_t* __restrict__ la,
             const uint32_t* __restrict__ lb, const uint32_t* __restrict__ lc, const uint32_t* __restrict__ lv,
             const uint32_t* __restrict__ lo, uint32_t K, uint32_t row_size, uint32_t value_dim, float scale,
             float cap, uint32_t n_splits, uint32_t chunk, float* partial) {
  constexpr int VEC = 8;
  constexpr uint32_t lpr = LPR;
  __shared__ float p[ATT_CHUNK];
  __shared__ float red[4];
  __shared__ float osum[2048];
  const uint32_t tid = threadIdx.x, lane = tid & 63u, wave = tid >> 6;
  const uint32_t split = blockIdx.x, op = blockIdx.y;
  const uint32_t t0 = split * chunk, t1 = min(row_size, t0 + chunk), nt = t1 - t0;
  const uint64_t a = la[op], kb = (uint64_t)lb[op] - kv_shift, c = lc[op], vb = (uint64_t)lv[op] - kv_shift, ob = lo[op];
  // scores: the query slice of this lane in registers, 64/lpr K rows per wave step
  {
    const uint32_t sub = lane % lpr, rslot = lane / lpr, rpw = 64u / lpr, nvec = K / VEC;
    float q[4][VEC];
#pragma unroll
    for (int i = 0; i < 4; i++) {
      const uint32_t v = sub + i * lpr;
#pragma unroll
      for (int j = 0; j < VEC; j++) q[i][j] = v < nvec ? data[a + (uint64_t)v * VEC + j] : 0.f;
    }
    if (lpr >= nvec) {
      // every lane holds one 16-byte slice of a row (head dims up to 512): sixteen row groups per trip,
      // all loads issued before the first is used; rows past the chunk are clamped and dropped
      for (uint32_t rb = t0 + wave * rpw; rb < t1; rb += 64u * rpw) {
        uint4 raw[16];
        const uint32_t v = min(sub, nvec - 1u);
#pragma unroll
        for (int g16 = 0; g16 < 16; g16++) {
          const uint32_t r = min(rb + g16 * 4u * rpw + rslot, t1 - 1u);
          raw[g16] = *(const uint4*)(kv + kb + (uint64_t)r * K + (uint64_t)v * VEC);
        }
        // partial dot products of all sixteen groups, then the lane reductions stage by stage so that
        // the sixteen shuffles of a stage are independent
        float sg[16];
#pragma unroll
        for (int g16 = 0; g16 < 16; g16++) {
          float s = 0.f;
          if (sub < nvec) {
            const __half2* h = (const __half2*)&raw[g16];
#pragma unroll
            for (int j = 0; j < 4; j++) {
              const float2 f = __half22float2(h[j]);
              s = fmaf(q[0][2 * j], f.x, s);
              s = fmaf(q[0][2 * j + 1], f.y, s);
            }
          }
          sg[g16] = s;
        }
#pragma unroll
        for (int o = LPR >> 1; o > 0; o >>= 1) {
#pragma unroll
          for (int g16 = 0; g16 < 16; g16++) sg[g16] += __shfl_xor(sg[g16], o, 64);
        }
#pragma unroll
        for (int g16 = 0; g16 < 16; g16++) {
          const uint32_t r = rb + g16 * 4u * rpw + rslot;
          if (r < t1 && sub == 0) {
            out[c + r] = sg[g16];
            p[r - t0] = sg[g16];   // soft cap and scale are applied below, one row per thread
          }
        }
      }
    } else {
      // long rows: up to four slices per lane, four row groups per trip
      for (uint32_t rb = t0 + wave * rpw; rb < t1; rb += 16u * rpw) {
        uint4 raw[4][4];
#pragma unroll
        for (int g4 = 0; g4 < 4; g4++) {
          const uint32_t r = min(rb + g4 * 4u * rpw + rslot, t1 - 1u);
#pragma unroll
          for (int i = 0; i < 4; i++) {
            if (i * lpr < nvec) {   // uniform: slices the row does not have are skipped
              const uint32_t v = min(sub + i * lpr, nvec - 1u);
              raw[g4][i] = *(const uint4*)(kv + kb + (uint64_t)r * K + (uint64_t)v * VEC);
            }
          }
        }
#pragma unroll
        for (int g4 = 0; g4 < 4; g4++) {
          const uint32_t r = rb + g4 * 4u * rpw + rslot;
          float s = 0.f;
#pragma unroll
          for (int i = 0; i < 4; i++) {
            if (sub + i * lpr < nvec) {
              const __half2* h = (const __half2*)&raw[g4][i];
#pragma unroll
              for (int j = 0; j < 4; j++) {
                const float2 f = __half22float2(h[j]);
                s = fmaf(q[i][2 * j], f.x, s);
                s = fmaf(q[i][2 * j + 1], f.y, s);
              }
            }
          }
          for (uint32_t o = lpr >> 1; o > 0; o >>= 1) s += __shfl_xor(s, o, 64);
          if (r < t1 && sub == 0) {
            out[c + r] = s;
            p[r - t0] = s;
          }
        }
      }
    }
  }
  __syncthreads();
  float mx = -9.99999968e+37f;
  for (uint32_t t = tid; t < nt; t += 256u) {
    const float v = prep(p[t], scale, cap);
    p[t] = v;
    mx = fmaxf(mx, v);
  }
  mx = wave_max64(mx);
  if (lane == 0) red[wave] = mx;
  __syncthreads();
  mx = fmaxf(fmaxf(red[0], red[1]), fmaxf(red[2], red[3]));
  __syncthreads();
  float sum = 0.f;
  for (uint32_t t = tid; t < nt; t += 256u) {
    const float e = expf(p[t] - mx);
    p[t] = e;
    sum += e;
  }
  sum = wave_sum64(sum);
  if (lane == 0) red[wave] = sum;
  __syncthreads();
  sum = (red[0] + red[1]) + (red[2] + red[3]);
  // values: vlpr lanes cover one V row, 256/vlpr rows in flight per sweep; row-slot partials meet in LDS
  const uint32_t vlpr = value_dim / VEC, slots = 256u / vlpr, sub = tid % vlpr, slot = tid / vlpr;
  float acc[VEC];
#pragma unroll
  for (int j = 0; j < VEC; j++) acc[j] = 0.f;
  if (slot < slots) {
    const __half* base = kv + vb + (uint64_t)t0 * value_dim + (uint64_t)sub * VEC;
    // eight V rows per lane and trip, loads first (rows past the chunk: clamped, weight 0)
    for (uint32_t tb = slot; tb < nt; tb += 8u * slots) {
      uint4 raw[8];
      float w[8];
#pragma unroll
      for (int u = 0; u < 8; u++) {
        const uint32_t t = tb + u * slots;
        raw[u] = *(const uint4*)(base + (uint64_t)min(t, nt - 1u) * value_dim);
        w[u] = t < nt ? p[min(t, nt - 1u)] : 0.f;
      }
#pragma unroll
      for (int u = 0; u < 8; u++) {
        const __half2* h = (const __half2*)&raw[u];
#pragma unroll
        for (int j = 0; j < 4; j++) {
          const float2 f = __half22float2(h[j]);
          acc[2 * j] = fmaf(w[u], f.x, acc[2 * j]);
          acc[2 * j + 1] = fmaf(w[u], f.y, acc[2 * j + 1]);
        }
      }
    }
  }
  const uint32_t fit = 2048u / value_dim;
  float o = 0.f;
  for (uint32_t s0 = 0; s0 < slots; s0 += fit) {
    if (slot >= s0 && slot < s0 + fit && slot < slots) {
#pragma unroll
      for (int j = 0; j < VEC; j++) osum[(slot - s0) * value_dim + sub * VEC + j] = acc[j];
    }
    __syncthreads();
    if (tid < value_dim)
      for (uint32_t s = 0; s < fit && s0 + s < slots; s++) o += osum[s * value_dim + tid];
    __syncthreads();
  }
  if (tid < value_dim) {
    if (n_splits == 1) out[ob + tid] = o * (1.0f / sum);
    else partial[((uint64_t)op * n_splits + split) * (value_dim + 2) + 2 + tid] = o;
  }
  if (n_splits > 1 && tid == 0) {
    float* pp = partial + ((uint64_t)op * n_splits + split) * (value_dim + 2);
    pp[0] = mx;
    pp[1] = sum;
  }
}

// Merge the split partials of one op: M = max m_s, w_s = e^(m_s-M), L = sum l_s w_s,
// out = sum_s o_s w_s / L.  n_splits <= 1024.  grid (n_ops, ceil(value_dim / 32)): a workgroup owns 32
// output elements, eight groups of 32 threads take every eighth split each and meet in LDS.
// FEW (n_splits <= 64): everything a thread needs -- its eight values, one split's (max, sum) pair per lane, the
// output base, its element of the prepared queries -- is asked for in one round of loads, clamped rather than
// skipped, and every wave works out M, the weights and L for itself with cross-lane operations: one trip to memory
// and one barrier where the general form below takes three of each.  Same operations in the same order per result.
template <bool FEW>
__global__ void __launch_bounds__(256)
k_attn_combine(float* out, const float* partial, const uint32_t* __restrict__ lo, uint32_t value_dim,
               uint32_t n_splits, uint64_t n_elems, const float* q_src, uint32_t q_dst, uint32_t q_n) {
  __shared__ float w[FEW ? 1 : 1024];
  __shared__ float red[4];
  __shared__ float osum[8][32];
  const uint32_t op = blockIdx.x, tid = threadIdx.x, lane = tid & 63u, wave = tid >> 6;
  const uint32_t stride = value_dim + 2;
  const float* pp = partial + (uint64_t)op * n_splits * stride;
  if (FEW) {
    const uint32_t last = n_splits - 1u, sg = tid >> 5, d = blockIdx.y * 32u + (tid & 31u), dc = min(d, value_dim - 1u);
    const uint32_t threads = gridDim.x * gridDim.y * 256u, gi = (blockIdx.y * gridDim.x + op) * 256u + tid;
    const float* ps = pp + (uint64_t)min(lane, last) * stride;
    const float m_own = ps[0], l_own = ps[1];
    float v[8];
#pragma unroll
    for (uint32_t k = 0; k < 8u; k++) v[k] = pp[(uint64_t)min(sg + 8u * k, last) * stride + 2 + dc];
    const float qv = (q_n ? q_src : partial)[q_n ? min(gi, q_n - 1u) : 0u];   // (a load on every path)
    const uint64_t ob = lo[op];
    const float M = wave_max64(lane < n_splits ? m_own : -9.99999968e+37f);
    const float e = lane < n_splits ? expf(m_own - M) : 0.f;
    const float invL = 1.0f / wave_sum64(lane < n_splits ? fmaf(l_own, e, 0.f) : 0.f);
    float o0 = 0.f, o1 = 0.f;
#pragma unroll
    for (uint32_t k = 0; k < 4u; k++) {
      const uint32_t s0 = sg + 16u * k, s1 = s0 + 8u;
      const float w0 = __shfl(e, (int)s0, 64), w1 = __shfl(e, (int)s1, 64);
      o0 = s0 < n_splits ? fmaf(v[2u * k], w0, o0) : o0;
      o1 = s1 < n_splits ? fmaf(v[2u * k + 1u], w1, o1) : o1;
    }
    osum[sg][tid & 31u] = o0 + o1;
    if (gi < q_n) out[(uint64_t)q_dst + gi] = qv;
    for (uint32_t i = gi + threads; i < q_n; i += threads) out[(uint64_t)q_dst + i] = q_src[i];
    __syncthreads();
    if (tid < 32u && d < value_dim && ob + value_dim <= n_elems) {
      float o = 0.f;
#pragma unroll
      for (int i = 0; i < 8; i++) o += osum[i][tid];
      out[ob + d] = o * invL;
    }
    return;
  }
  // queries the attention launch prepared and could not yet store over the raw ones: each workgroup its share
  for (uint32_t i = (blockIdx.y * gridDim.x + op) * 256u + tid; i < q_n; i += gridDim.x * gridDim.y * 256u)
    out[(uint64_t)q_dst + i] = q_src[i];
  const uint64_t ob = lo[op];
  if (ob + value_dim > n_elems) return;
  float M = -9.99999968e+37f;
  for (uint32_t s = tid; s < n_splits; s += 256u) M = fmaxf(M, pp[(uint64_t)s * stride]);
  M = wave_max64(M);
  if (lane == 0) red[wave] = M;
  __syncthreads();
  M = fmaxf(fmaxf(red[0], red[1]), fmaxf(red[2], red[3]));
  __syncthreads();
  float L = 0.f;
  for (uint32_t s = tid; s < n_splits; s += 256u) {
    const float e = expf(pp[(uint64_t)s * stride] - M);
    w[s] = e;
    L = fmaf(pp[(uint64_t)s * stride + 1], e, L);
  }
  L = wave_sum64(L);
  if (lane == 0) red[wave] = L;
  __syncthreads();
  const float invL = 1.0f / ((red[0] + red[1]) + (red[2] + red[3]));
  const uint32_t d = blockIdx.y * 32u + (tid & 31u), sg = tid >> 5;
  float o0 = 0.f, o1 = 0.f;
  if (d < value_dim) {
    uint32_t s = sg;
    for (; s + 8u < n_splits; s += 16u) {
      o0 = fmaf(pp[(uint64_t)s * stride + 2 + d], w[s], o0);
      o1 = fmaf(pp[(uint64_t)(s + 8u) * stride + 2 + d], w[s + 8u], o1);
    }
    if (s < n_splits) o0 = fmaf(pp[(uint64_t)s * stride + 2 + d], w[s], o0);
  }
  osum[sg][tid & 31u] = o0 + o1;
  __syncthreads();
  if (tid < 32u && d < value_dim) {
    float o = 0.f;
#pragma unroll
    for (int i = 0; i < 8; i++) o += osum[i][tid];
    out[ob + d] = o * invL;
  }
}

// Row softmax family (map_softmax.comp, map_softmax_abs.comp, map_attn_softmax_abs.comp):
// one workgroup per row, source/destination bases from locs (multiplied by row_size when REL).
template <bool REL>
__global__ void __launch_bounds__(256)
k_softmax_rows(float* data, const uint32_t* __restrict__ ls, const uint32_t* __restrict__ ldst, uint32_t row_size,
               float scale, float cap, uint64_t n_elems) {
  __shared__ float red[4];
  const uint32_t tid = threadIdx.x, lane = tid & 63u, wave = tid >> 6, ri = blockIdx.x;
  const uint64_t sb = REL ? (uint64_t)ls[ri] * row_size : ls[ri], db = REL ? (uint64_t)ldst[ri] * row_size : ldst[ri];
  if (sb + row_size > n_elems || db + row_size > n_elems) return;
  float mx = -9.99999968e+37f;
  for (uint32_t i = tid; i < row_size; i += 256u) mx = fmaxf(mx, prep(data[sb + i], scale, cap));
  mx = wave_max64(mx);
  if (lane == 0) red[wave] = mx;
  __syncthreads();
  mx = fmaxf(fmaxf(red[0], red[1]), fmaxf(red[2], red[3]));
  __syncthreads();
  float sum = 0.f;
  for (uint32_t i = tid; i < row_size; i += 256u) sum += expf(prep(data[sb + i], scale, cap) - mx);
  sum = wave_sum64(sum);
  if (lane == 0) red[wave] = sum;
  __syncthreads();
  sum = (red[0] + red[1]) + (red[2] + red[3]);
  const float inv = 1.0f / sum;
  // src may equal dst: every thread rereads only the elements it then overwrites
  for (uint32_t i = tid; i < row_size; i += 256u) data[db + i] = expf(prep(data[sb + i], scale, cap) - mx) * inv;
}

// All ops of a handle inside the fp16 KV range?  Needs the host copy of the locs.
static bool all_in_kv(const Map* m, uint32_t h, uint32_t n_ops, uint64_t span) {
  if (!m->kv16) return false;
  const uint32_t* v = res_host(h, n_ops);
  if (!v) return false;
  for (uint32_t i = 0; i < n_ops; i++)
    if (v[i] < m->kv_start || v[i] - m->kv_start + span > m->kv_count) return false;
  return true;
}


// Sequence split of softmax . V: rows per workgroup so that about two workgroups per CU exist over
// all heads, 32..1024 rows each.
#define ATT_FOLD_FLOATS 8192u   // most partial floats a consumer is asked to merge by itself
static void attn_split(uint32_t n_ops, uint32_t row_size, uint32_t value_dim, bool few, uint32_t* chunk,
                       uint32_t* n_splits) {
  const uint32_t want_splits = std::max<uint32_t>(1u, cdiv(2u * (uint32_t)g.n_cu, n_ops));
  uint32_t c = std::min<uint32_t>(ATT_CHUNK, std::max<uint32_t>(32u, cdiv(row_size, want_splits)));
  c = (c + 31u) & ~31u;
  // `few`: the consumer will merge the partials, every one of its workgroups reads all of them, so
  // keep them few (longer chunks) as long as a chunk still fits a workgroup
  if (few) {
    uint32_t cf = c;
    while (cf < ATT_CHUNK && (uint64_t)n_ops * cdiv(row_size, cf) * (value_dim + 2) > ATT_FOLD_FLOATS) cf += 32u;
    // partials still too many at the longest chunk: the consumer will not merge them, keep the wide split
    if ((uint64_t)n_ops * cdiv(row_size, cf) * (value_dim + 2) <= ATT_FOLD_FLOATS) c = cf;
  }
  *chunk = c;
  *n_splits = cdiv(row_size, c);
}

// Operand checks of softmax . V against the host copies of the handles; *kv = K/V rows in the fp16
// copy, *fast = whole 16-byte vectors and everything in range.
static int attn_check(uint32_t map_id, uint32_t hs, uint32_t hv, uint32_t ho, uint32_t n_ops, uint32_t row_size,
                      uint32_t value_dim, bool* kv, bool* fast) {
  Map* m = get_f32_map(map_id);
  if (!m) return ADAMAH_ERR_INVALID;
  if (!res_u32(hs, n_ops) || !res_u32(hv, n_ops) || !res_u32(ho, n_ops)) return ADAMAH_ERR_INVALID;
  uint32_t chunk, n_splits;
  attn_split(n_ops, row_size, value_dim, false, &chunk, &n_splits);
  if ((uint64_t)n_ops * n_splits * (value_dim + 2) > g.attn_scratch_floats || n_splits > 1024) return ADAMAH_ERR_INVALID;
  *kv = all_in_kv(m, hv, n_ops, (uint64_t)row_size * value_dim);
  const uint32_t vec = *kv ? 8u : 4u;
  const uint32_t *sh = res_host(hs, n_ops), *vh = res_host(hv, n_ops), *oh = res_host(ho, n_ops);
  bool f = sh && vh && oh && value_dim % vec == 0 && value_dim / vec <= 256 && 256u % (value_dim / vec) == 0 &&
           value_dim <= 256;
  for (uint32_t op = 0; f && op < n_ops; op++)
    f = in_range(sh[op], row_size, m->n_elems) && in_range(vh[op], (uint64_t)row_size * value_dim, m->n_elems) &&
        in_range(oh[op], value_dim, m->n_elems) && (vh[op] - (*kv ? m->kv_start : 0)) % vec == 0;
  *fast = f;
  return ADAMAH_OK;
}

int launch_scores(const PendOp& sc) {
  g.no_defer++;
  const int r = map_matmul_t_dev(sc.map_act, sc.h[0], sc.h[1], sc.h[2], 1, sc.k, sc.n, sc.rpg);
  g.no_defer--;
  return r;
}

// Can the queued score op be computed inside the softmax . V launch?  Same heads and length, the
// score rows it writes are the ones softmax . V reads, K rows in the fp16 copy.
bool attn_foldable(const PendOp& sc, const PendOp& at) {
  if (sc.kind != PK_SCORES || at.kind != PK_ATTN || sc.map_act != at.map_act || sc.rpg != at.rpg || sc.n != at.n) return false;
  const uint32_t *c = res_host(sc.h[2], sc.rpg), *s = res_host(at.h[0], at.rpg);
  if (!c || !s) return false;
  for (uint32_t i = 0; i < sc.rpg; i++) if (c[i] != s[i]) return false;
  return true;
}

int launch_attn(const PendOp* sc, const PendOp& at, bool leave_partials, AttnPartials* ap, const RowPrepCtx* prep) {
  Map* m = get_f32_map(at.map_act);
  // the row ops offered with the pair: launched here, ahead of the attention, unless the decode kernel takes them
  auto rows_first = [&]() {
    int rc = ADAMAH_OK;
    if (prep) launch_row_run(*prep->q, prep->i0, &rc);
    prep = nullptr;
    return rc;
  };
  if (!m) { rows_first(); return ADAMAH_ERR_INVALID; }
  const uint32_t n_ops = at.rpg, row_size = at.n, value_dim = at.k;
  bool kv = false, fast = false;
  int r = attn_check(at.map_act, at.h[0], at.h[1], at.h[2], n_ops, row_size, value_dim, &kv, &fast);
  if (r) { rows_first(); return r; }
  const uint32_t *ls = res_u32(at.h[0], n_ops), *lv = res_u32(at.h[1], n_ops), *lo = res_u32(at.h[2], n_ops);
  uint32_t chunk, n_splits;
  attn_split(n_ops, row_size, value_dim, leave_partials, &chunk, &n_splits);
  if ((uint64_t)n_ops * n_splits * (value_dim + 2) > ATT_FOLD_FLOATS) leave_partials = false;
  float* d = (float*)m->buf;
  dim3 grid(n_splits, n_ops);
  if (sc && fast && kv && sc->k == value_dim) {
    // all query heads of a KV head in one workgroup, K and V rows read once
    AttnDecodeArgs da = {d, m->kv16, m->kv_start,
                         res_u32(sc->h[0], n_ops), res_u32(sc->h[1], n_ops), ls, lv, lo,
                         res_host(sc->h[0], n_ops), res_host(sc->h[1], n_ops), res_host(at.h[0], n_ops),
                         res_host(at.h[1], n_ops), res_host(at.h[2], n_ops),
                         n_ops, value_dim, row_size, at.eps, at.f2, leave_partials, ATT_FOLD_FLOATS, nullptr, nullptr};
    int drc = 0;
    bool left = false, prep_done = false;
    AttnPartials dp = {};
    auto finish = [&]() {
      if (ap) ap->n_splits = 1;
      if (drc || dp.n_splits == 1) return drc;
      if (left && ap) { *ap = dp; return (int)ADAMAH_OK; }
      return launch_attn_combine(at, dp);
    };
    if (prep) {
      // with the preparation inside the launch, or not at all (nothing is launched then)
      da.prep = &prep->tasks; da.prep_done = &prep_done;
      if (launch_attn_decode(da, &dp, &left, &drc)) return finish();
      da.prep = nullptr; da.prep_done = nullptr;
      if ((r = rows_first())) return r;
    }
    if (launch_attn_decode(da, &dp, &left, &drc)) return finish();
  }
  if ((r = rows_first())) return r;
  if (sc && fast && kv) {
    const uint32_t *la = res_u32(sc->h[0], n_ops), *lb = res_u32(sc->h[1], n_ops);
    uint32_t lpr = 8;
    while (lpr < 64 && lpr * 8u < sc->k) lpr <<= 1;
#define AF(L)                                                                                                      \
  k_attn_fused<L><<<grid, 256, 0, g.stream>>>(d, d, m->kv16, m->kv_start, la, lb, ls, lv, lo, sc->k, row_size, value_dim, \
                                              at.eps, at.f2, n_splits, chunk, g.attn_scratch)
    if (lpr == 8) AF(8); else if (lpr == 16) AF(16); else if (lpr == 32) AF(32); else AF(64);
#undef AF
  } else {
    if (sc && (r = launch_scores(*sc))) return r;
    const float scale = at.eps, cap = at.f2;
#define ASV(T, V, src, shift, elems)                                                                             \
  k_attn_softmax_value<T, V><<<grid, 256, 0, g.stream>>>(d, d, src, shift, ls, lv, lo, row_size, value_dim, scale, \
                                                         cap, n_splits, chunk, g.attn_scratch, m->n_elems, elems)
    if (kv) { if (fast) ASV(__half, 8, m->kv16, m->kv_start, m->kv_count); else ASV(__half, 1, m->kv16, m->kv_start, m->kv_count); }
    else { if (fast) ASV(float, 4, d, 0, m->n_elems); else ASV(float, 1, d, 0, m->n_elems); }
#undef ASV
  }
  count_launch();
  r = check_launch();
  if (r || n_splits == 1) { if (ap) ap->n_splits = 1; return r; }
  AttnPartials loc = {g.attn_scratch, n_splits, value_dim, n_ops, 0, nullptr, 0, 0};
  if (leave_partials && ap) { *ap = loc; return ADAMAH_OK; }
  if (ap) ap->n_splits = 1;
  return launch_attn_combine(at, loc);
}

int launch_attn_combine(const PendOp& at, const AttnPartials& ap) {
  Map* m = get_f32_map(at.map_act);
  const uint32_t* lo = res_u32(at.h[2], at.rpg);
  if (!m || !lo) return ADAMAH_ERR_INVALID;
  const dim3 grid(at.rpg, cdiv(ap.value_dim, 32));
  if (ap.n_splits <= 64u)
    k_attn_combine<true><<<grid, 256, 0, g.stream>>>((float*)m->buf, ap.base, lo, ap.value_dim, ap.n_splits, m->n_elems, ap.q_src,
                                                     ap.q_dst, ap.q_n);
  else
    k_attn_combine<false><<<grid, 256, 0, g.stream>>>((float*)m->buf, ap.base, lo, ap.value_dim, ap.n_splits, m->n_elems, ap.q_src,
                                                      ap.q_dst, ap.q_n);
  count_launch();
  return check_launch();
}

// Merge of the sequence slices for output rows listed in device memory.
int launch_attn_combine_dev(Map* m, const float* partial, const uint32_t* lo_dev, uint32_t n_ops, uint32_t value_dim,
                            uint32_t n_splits) {
  const dim3 grid(n_ops, cdiv(value_dim, 32));
  if (n_splits <= 64u)
    k_attn_combine<true><<<grid, 256, 0, g.stream>>>((float*)m->buf, partial, lo_dev, value_dim, n_splits, m->n_elems, nullptr, 0u, 0u);
  else
    k_attn_combine<false><<<grid, 256, 0, g.stream>>>((float*)m->buf, partial, lo_dev, value_dim, n_splits, m->n_elems, nullptr, 0u,
                                                      0u);
  count_launch();
  return check_launch();
}

}  // namespace adamah


using namespace adamah;

extern "C" {

int map_matmul_t_dev(uint32_t map_id, uint32_t ha, uint32_t hb, uint32_t hc, uint32_t M, uint32_t K, uint32_t N,
                     uint32_t n_ops) {
  Map* m = get_f32_map(map_id);
  if (!m) { flush_pending(); return ADAMAH_ERR_INVALID; }
  if (n_ops == 0 || M == 0 || N == 0) { flush_pending(); return ADAMAH_OK; }
  const uint32_t *la = res_u32(ha, n_ops), *lb = res_u32(hb, n_ops), *lc = res_u32(hc, n_ops);
  if (!la || !lb || !lc) { flush_pending(); return ADAMAH_ERR_INVALID; }
  dim3 grid(cdiv(N, 4), M, n_ops);
  float* d = (float*)m->buf;
  const bool kv = all_in_kv(m, hb, n_ops, (uint64_t)N * K);
  // decode-score fast path: one query row per op, whole 16-byte vectors, operands verified on the host
  const uint32_t vec = kv ? 8u : 4u;
  const uint32_t *ah = res_host(ha, n_ops), *bh = res_host(hb, n_ops), *ch = res_host(hc, n_ops);
  bool fast = M == 1 && ah && bh && ch && K % vec == 0 && K >= vec && K <= 4u * 64u * vec;
  uint32_t lpr = 1;
  if (fast) {
    while (lpr < 64 && lpr * vec < K) lpr <<= 1;        // lanes per row: a power of two, at most 64
    for (uint32_t op = 0; fast && op < n_ops; op++)
      fast = in_range(ah[op], K, m->n_elems) && in_range(bh[op], (uint64_t)N * K, m->n_elems) &&
             in_range(ch[op], N, m->n_elems) && (bh[op] - (kv ? m->kv_start : 0)) % vec == 0;
  }
  if (fast && kv && can_defer()) {   // decode scores over the fp16 cache: queue, softmax . V may absorb them
    PendOp p;
    p.kind = PK_SCORES; p.map_act = map_id; p.h[0] = ha; p.h[1] = hb; p.h[2] = hc; p.k = K; p.n = N; p.rpg = n_ops;
    g.pend.push_back(p);
    return ADAMAH_OK;
  }
  flush_pending();
  if (fast) {
    // rows per workgroup: about two workgroups per CU over all ops, at least one wave step each
    const uint32_t want_wg = std::max<uint32_t>(1u, cdiv(2u * (uint32_t)g.n_cu, n_ops));
    const uint32_t rows_per_wg = std::max<uint32_t>(4u * (64u / lpr), std::min<uint32_t>(1024u, cdiv(N, want_wg)));
    dim3 g2(cdiv(N, rows_per_wg), n_ops);
    if (kv)
      k_scores_vec<__half, 8><<<g2, 256, 0, g.stream>>>(d, d, m->kv16, m->kv_start, la, lb, lc, K, N, lpr, rows_per_wg);
    else
      k_scores_vec<float, 4><<<g2, 256, 0, g.stream>>>(d, d, d, 0, la, lb, lc, K, N, lpr, rows_per_wg);
  } else if (kv)
    k_matmul_t<__half><<<grid, 256, 0, g.stream>>>(d, d, m->kv16, m->kv_start, la, lb, lc, M, K, N, m->n_elems,
                                                   m->kv_count);
  else
    k_matmul_t<float><<<grid, 256, 0, g.stream>>>(d, d, d, 0, la, lb, lc, M, K, N, m->n_elems, m->n_elems);
  count_launch();
  return check_launch();
}

int map_matmul_t_x_dev(uint32_t map_act, uint32_t map_wt, uint32_t ha, uint32_t hb, uint32_t hc, uint32_t M, uint32_t K,
                       uint32_t N, uint32_t n_ops) { ADAMAH_API();
  Map* ma = get_f32_map(map_act);
  Map* mw = get_f32_map(map_wt);
  if (!ma || !mw) return ADAMAH_ERR_INVALID;
  if (n_ops == 0 || M == 0 || N == 0) return ADAMAH_OK;
  const uint32_t *la = res_u32(ha, n_ops), *lb = res_u32(hb, n_ops), *lc = res_u32(hc, n_ops);
  if (!la || !lb || !lc) return ADAMAH_ERR_INVALID;
  dim3 grid(cdiv(N, 4), M, n_ops);
  k_matmul_t<float><<<grid, 256, 0, g.stream>>>((const float*)ma->buf, (float*)ma->buf, (const float*)mw->buf, 0, la, lb,
                                                lc, M, K, N, ma->n_elems, mw->n_elems);
  count_launch();
  return check_launch();
}

static int matmul_nt(uint32_t map_act, uint32_t map_wt, uint32_t ha, uint32_t hb, uint32_t hc, uint32_t M, uint32_t K,
                     uint32_t N, uint32_t n_ops) { ADAMAH_API();
  Map* ma = get_f32_map(map_act);
  Map* mw = get_f32_map(map_wt);
  if (!ma || !mw) return ADAMAH_ERR_INVALID;
  if (n_ops == 0 || M == 0 || N == 0) return ADAMAH_OK;
  const uint32_t *la = res_u32(ha, n_ops), *lb = res_u32(hb, n_ops), *lc = res_u32(hc, n_ops);
  if (!la || !lb || !lc) return ADAMAH_ERR_INVALID;
  dim3 grid(cdiv(N, 4), M, n_ops);
  k_matmul_nt<<<grid, 256, 0, g.stream>>>((const float*)ma->buf, (float*)ma->buf, (const float*)mw->buf, la, lb, lc, M,
                                          K, N, ma->n_elems, mw->n_elems);
  count_launch();
  return check_launch();
}
int map_matmul_x_dev(uint32_t map_act, uint32_t map_wt, uint32_t ha, uint32_t hb, uint32_t hc, uint32_t M, uint32_t K,
                     uint32_t N, uint32_t n_ops) { ADAMAH_API();
  return matmul_nt(map_act, map_wt, ha, hb, hc, M, K, N, n_ops);
}
int map_matmul_dev(uint32_t map_id, uint32_t ha, uint32_t hb, uint32_t hc, uint32_t M, uint32_t K, uint32_t N,
                   uint32_t n_ops) { ADAMAH_API();
  return matmul_nt(map_id, map_id, ha, hb, hc, M, K, N, n_ops);
}

int map_attn_softmax_value_dev(uint32_t map_id, uint32_t hs, uint32_t hv, uint32_t ho, uint32_t n_ops,
                               uint32_t row_size, uint32_t value_dim, float scale, float cap) {
  if (n_ops == 0 || row_size == 0 || value_dim == 0) { flush_pending(); return get_f32_map(map_id) ? ADAMAH_OK : ADAMAH_ERR_INVALID; }
  bool kv = false, fast = false;
  int r = attn_check(map_id, hs, hv, ho, n_ops, row_size, value_dim, &kv, &fast);
  if (r) { flush_pending(); return r; }
  PendOp p;
  p.kind = PK_ATTN; p.map_act = map_id; p.h[0] = hs; p.h[1] = hv; p.h[2] = ho; p.rpg = n_ops; p.n = row_size;
  p.k = value_dim; p.eps = scale; p.f2 = cap;
  if (fast && kv && can_defer()) {   // queue: the scores before it and the GEMV after it may be folded in
    g.pend.push_back(p);
    return ADAMAH_OK;
  }
  flush_pending();
  return launch_attn(nullptr, p, false, nullptr);
}

static int softmax_rows(uint32_t map_id, uint32_t hs, uint32_t hd, uint32_t n_rows, uint32_t row_size, float scale,
                        float cap, bool rel) { ADAMAH_API();
  Map* m = get_f32_map(map_id);
  if (!m) return ADAMAH_ERR_INVALID;
  if (n_rows == 0 || row_size == 0) return ADAMAH_OK;
  const uint32_t *ls = res_u32(hs, n_rows), *ld = res_u32(hd, n_rows);
  if (!ls || !ld) return ADAMAH_ERR_INVALID;
  if (rel)
    k_softmax_rows<true><<<n_rows, 256, 0, g.stream>>>((float*)m->buf, ls, ld, row_size, scale, cap, m->n_elems);
  else
    k_softmax_rows<false><<<n_rows, 256, 0, g.stream>>>((float*)m->buf, ls, ld, row_size, scale, cap, m->n_elems);
  count_launch();
  return check_launch();
}
int map_softmax_dev(uint32_t map_id, uint32_t hs, uint32_t hd, uint32_t n_rows, uint32_t row_size) { ADAMAH_API();
  return softmax_rows(map_id, hs, hd, n_rows, row_size, 1.0f, 0.0f, true);
}
int map_softmax_abs_dev(uint32_t map_id, uint32_t hs, uint32_t hd, uint32_t n_rows, uint32_t row_size) { ADAMAH_API();
  return softmax_rows(map_id, hs, hd, n_rows, row_size, 1.0f, 0.0f, false);
}
int map_attn_softmax_abs_dev(uint32_t map_id, uint32_t hs, uint32_t hd, uint32_t n_rows, uint32_t row_size, float scale,
                             float cap) { ADAMAH_API();
  return softmax_rows(map_id, hs, hd, n_rows, row_size, scale, cap, false);
}

int adamah_attn_causal_rows_dev(uint32_t map_id, const uint32_t* q_handles, uint32_t locs_k, uint32_t locs_scores,
                                uint32_t locs_v, const uint32_t* out_handles, uint32_t m, uint32_t head_dim,
                                uint32_t n_keys0, uint32_t n_heads, uint32_t value_dim, float scale, float softcap) {
  if (m == 0) return ADAMAH_OK;
  if (!q_handles || !out_handles) return ADAMAH_ERR_INVALID;
  for (uint32_t t = 0; t < m; t++) {
    int r = map_matmul_t_dev(map_id, q_handles[t], locs_k, locs_scores, 1, head_dim, n_keys0 + t, n_heads);
    if (r != ADAMAH_OK) return r;
    r = map_attn_softmax_value_dev(map_id, locs_scores, locs_v, out_handles[t], n_heads, n_keys0 + t, value_dim, scale, softcap);
    if (r != ADAMAH_OK) return r;
  }
  return ADAMAH_OK;
}

}  // extern "C"
