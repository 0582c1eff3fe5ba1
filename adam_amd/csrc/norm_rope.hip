// RMSNorm (+ residual), half-split RoPE, fused per-head QK-norm + RoPE, and row copy (KV append).
//
// Reference kernels: shaders/src/f32/map_rmsnorm.comp, map_rmsnorm_x.comp:26-48,
// map_rmsnorm_add.comp:14-44, map_rope.comp:11-37, map_qk_norm_rope_x.comp:32-84,
// map_row_copy.comp:13-24; dispatchers adamah.c:7610-7878, 8476-8604, 8061-8085.
// Row bases come from device-resident loc arrays, one entry per row, as in the reference.
#include "common.h"
#include "gemv_common.h"
#include "../../include/adamah_hip.h"

namespace adamah {

__device__ __forceinline__ float block_sum_256(float v, float* sh) {
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) v += __shfl_xor(v, o, 64);
  if ((threadIdx.x & 63u) == 0) sh[threadIdx.x >> 6] = v;
  __syncthreads();
  float t = (sh[0] + sh[1]) + (sh[2] + sh[3]);
  __syncthreads();
  return t;
}

// y = x * (1/sqrt(sum(x^2)/dim + eps)) * w (+ r); one 256-thread workgroup per row
template <bool ADD>
__global__ void __launch_bounds__(256)
k_rmsnorm(const float* act, const float* wt, float* out, const uint32_t* __restrict__ ls,
          const uint32_t* __restrict__ lw, const uint32_t* __restrict__ lr, const uint32_t* __restrict__ ld,
          uint32_t dim, float eps, uint64_t act_elems, uint64_t wt_elems) {
  __shared__ float sh[4];
  const uint32_t ri = blockIdx.x, tid = threadIdx.x;
  const uint64_t sb = ls[ri], wb = lw[ri], db = ld[ri], rb = ADD ? (uint64_t)lr[ri] : 0;
  if (sb + dim > act_elems || db + dim > act_elems || wb + dim > wt_elems || (ADD && rb + dim > act_elems)) return;
  float ss = 0.f;
  for (uint32_t i = tid; i < dim; i += 256u) { float x = act[sb + i]; ss = fmaf(x, x, ss); }
  ss = block_sum_256(ss, sh);
  const float inv = 1.0f / sqrtf(ss / (float)dim + eps);
  for (uint32_t i = tid; i < dim; i += 256u) {
    float y = act[sb + i] * inv * wt[wb + i];
    if (ADD) y += act[rb + i];
    out[db + i] = y;
  }
}

// The same row op with the row held in registers (dim <= 256 NU): one trip to memory instead of two
// dependent passes.  Thread t owns elements t, t + 256, ... and sums their squares in that order, as the
// kernel above does, so the results are the same bits.  EMIT: the rows are [n_rows, dim] back to back and a
// batched matmul follows; its fp16 operand form (row scaled by a power of two, two planes, 8-element words in the
// order (0,4)(1,5)(2,6)(3,7), plus (s, 1/s) per row) is written here as well, which spares that
// matmul its conversion launch.
struct RowsByValue { uint32_t on, s0, ss, w0, ws, d0, ds, r0, rs; };   // host side only
template <bool ADD, bool EMIT, int NU>
__global__ void __launch_bounds__(256)
k_rmsnorm_rows(const float* act, const float* wt, uint32_t dim_on, float eps, uint32_t s0, uint32_t ss_, uint32_t w0, uint32_t ws,
               uint32_t d0, uint32_t ds, uint32_t r0, uint32_t rs, float* out,
               const uint32_t* __restrict__ ls, const uint32_t* __restrict__ lw, const uint32_t* __restrict__ lr,
               const uint32_t* __restrict__ ld, uint64_t act_elems, uint64_t wt_elems, float* scale, __half* xh, __half* xl) {
  // (these 14 dwords are in registers when a wave starts.  Top bit of dim_on: row i's source / weights / destination /
  // residual start at x0 + i xs -- the host found the rows evenly spaced -- instead of four loads from the row
  // tables, which the rows' own loads would have to wait for)
  __shared__ float sh[4];
  const uint32_t ri = blockIdx.x, tid = threadIdx.x, dim = dim_on & 0x7FFFFFFFu;
  uint64_t sb, wb, db, rb = 0;
  if (dim_on >> 31) {
    sb = (uint64_t)s0 + (uint64_t)ri * ss_; wb = (uint64_t)w0 + (uint64_t)ri * ws;
    db = (uint64_t)d0 + (uint64_t)ri * ds; if (ADD) rb = (uint64_t)r0 + (uint64_t)ri * rs;
  } else {
    sb = ls[ri]; wb = lw[ri]; db = ld[ri]; if (ADD) rb = lr[ri];
  }
  if (sb + dim > act_elems || db + dim > act_elems || wb + dim > wt_elems || (ADD && rb + dim > act_elems)) return;
  float x[NU], w[NU], r[NU];
#pragma unroll
  for (int u = 0; u < NU; u++) {
    const uint32_t i = tid + 256u * u;
    const bool in = i < dim;
    x[u] = in ? act[sb + i] : 0.f;
    w[u] = in ? wt[wb + i] : 0.f;
    r[u] = (ADD && in) ? act[rb + i] : 0.f;
  }
  float ss = 0.f;
#pragma unroll
  for (int u = 0; u < NU; u++)
    if (tid + 256u * u < dim) ss = fmaf(x[u], x[u], ss);
  ss = block_sum_256(ss, sh);
  const float inv = 1.0f / sqrtf(ss / (float)dim + eps);
  float m = 0.f;
#pragma unroll
  for (int u = 0; u < NU; u++) {
    float y = x[u] * inv * w[u];
    if (ADD) y += r[u];
    x[u] = y;
    if (tid + 256u * u < dim) { out[db + tid + 256u * u] = y; m = fmaxf(m, fabsf(y)); }
  }
  if (!EMIT) return;
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) m = fmaxf(m, __shfl_xor(m, o, 64));
  if ((tid & 63u) == 0) sh[tid >> 6] = m;
  __syncthreads();
  m = fmaxf(fmaxf(sh[0], sh[1]), fmaxf(sh[2], sh[3]));
  const uint32_t e = (__float_as_uint(m) >> 23) & 0xFFu;
  float s = 1.f, si = 1.f;
  if (e >= 14u && e <= 254u) { s = __uint_as_float((267u - e) << 23); si = __uint_as_float((e - 13u) << 23); }
  if (tid == 0) { scale[2 * ri] = s; scale[2 * ri + 1] = si; }
  // two planes: fp16(x s) and the fp16 remainder x s - fp16(x s), as the matmul's own conversion writes them
  __half* dst = xh + (uint64_t)ri * dim;
  __half* dstl = xl + (uint64_t)ri * dim;
#pragma unroll
  for (int u = 0; u < NU; u++) {
    const uint32_t i = tid + 256u * u, q = i & 7u;
    if (i < dim) {
      const uint32_t at = (i & ~7u) + (q < 4u ? 2u * q : 2u * (q - 4u) + 1u);
      const float v = x[u] * s;
      const __half h = __float2half(v);
      dst[at] = h;
      dstl[at] = __float2half(v - __half2float(h));
    }
  }
}

// theta_i = pos * (1 / base^(2i/dim)).  The exponent and the reciprocal are float32 operations as
// in the shader; the power itself is evaluated in double and rounded once, which makes the
// frequency independent of the float32 pow implementation.
__device__ __forceinline__ void rope_cs(uint32_t i, uint32_t dim, uint32_t pos, float base, float* c, float* s) {
  const float e = (float)(2u * i) / (float)dim;
  const float p = (float)pow((double)base, (double)e);
  const float angle = (float)pos * (1.0f / p);
  *c = cosf(angle);
  *s = sinf(angle);
}

__global__ void __launch_bounds__(256)
k_rope(float* data, const uint32_t* __restrict__ ls, const uint32_t* __restrict__ ld, uint32_t n_tokens,
       uint32_t n_heads, uint32_t head_dim, uint32_t pos_offset, float base, uint64_t n_elems) {
  const uint32_t half = head_dim >> 1;
  const uint64_t tid = (uint64_t)blockIdx.x * 256u + threadIdx.x;
  if (tid >= (uint64_t)n_tokens * n_heads * half) return;
  const uint32_t token = (uint32_t)(tid / ((uint64_t)n_heads * half));
  const uint32_t rem = (uint32_t)(tid % ((uint64_t)n_heads * half));
  const uint32_t head = rem / half, d = rem % half;
  const uint64_t bs = (uint64_t)ls[token] + (uint64_t)head * head_dim, bd = (uint64_t)ld[token] + (uint64_t)head * head_dim;
  if (bs + head_dim > n_elems || bd + head_dim > n_elems) return;
  float c, s;
  rope_cs(d, head_dim, pos_offset + token, base, &c, &s);
  const float x0 = data[bs + d], x1 = data[bs + d + half];
  data[bd + d] = x0 * c - x1 * s;
  data[bd + d + half] = x0 * s + x1 * c;
}

// One workgroup per Q or K row: RMSNorm with eps = 1e-6 (fixed in the shader), weight per row from
// map_wt, then RoPE; rows written contiguously (Q rows, then K rows) from locs_qk_dst[0].
__global__ void __launch_bounds__(256)
k_qk_norm_rope(float* act, const float* wt, const uint32_t* __restrict__ lqs, const uint32_t* __restrict__ lqw,
               const uint32_t* __restrict__ lks, const uint32_t* __restrict__ lkw, const uint32_t* __restrict__ ldst,
               uint32_t q_rows, uint32_t q_dim, uint32_t k_rows, uint32_t k_dim, uint32_t pos, float base,
               uint64_t act_elems, uint64_t wt_elems) {
  __shared__ float sh[4];
  const uint32_t row = blockIdx.x, tid = threadIdx.x;
  const bool is_q = row < q_rows;
  const uint32_t lr = is_q ? row : row - q_rows;
  const uint32_t dim = is_q ? q_dim : k_dim, half = dim >> 1;
  if (half == 0) return;
  const uint64_t sb = is_q ? lqs[lr] : lks[lr], wb = is_q ? lqw[lr] : lkw[lr];
  const uint64_t db = (uint64_t)ldst[0] + (is_q ? (uint64_t)lr * q_dim : (uint64_t)q_rows * q_dim + (uint64_t)lr * k_dim);
  if (sb + dim > act_elems || db + dim > act_elems || wb + dim > wt_elems) return;
  float ss = 0.f;
  for (uint32_t i = tid; i < dim; i += 256u) { float x = act[sb + i]; ss = fmaf(x, x, ss); }
  ss = block_sum_256(ss, sh);
  const float inv = 1.0f / sqrtf(ss / (float)dim + 1e-6f);
  for (uint32_t i = tid; i < half; i += 256u) {
    const float y0 = act[sb + i] * inv * wt[wb + i];
    const float y1 = act[sb + i + half] * inv * wt[wb + i + half];
    float c, s;
    rope_cs(i, dim, pos, base, &c, &s);
    act[db + i] = y0 * c - y1 * s;
    act[db + i + half] = y0 * s + y1 * c;
  }
}

// spec = [src_row, dst_row] pairs; src = src_base[0] + src_row*row_size; dst = (dst_row+offset)*row_size.
// Destinations inside the map's fp16 KV range are rounded to fp16 and mirrored.
__global__ void __launch_bounds__(256)
k_row_copy(float* data, const uint32_t* __restrict__ spec, const uint32_t* __restrict__ src_base, uint32_t n_copies,
           uint32_t row_size, uint32_t dst_row_offset, uint64_t n_elems, __half* kv16, uint64_t kv_start,
           uint64_t kv_count) {
  const uint64_t tid = (uint64_t)blockIdx.x * 256u + threadIdx.x;
  const uint32_t ci = (uint32_t)(tid / row_size), ei = (uint32_t)(tid % row_size);
  if (ci >= n_copies) return;
  const uint64_t so = (uint64_t)src_base[0] + (uint64_t)spec[2 * ci] * row_size + ei;
  const uint64_t dof = ((uint64_t)spec[2 * ci + 1] + dst_row_offset) * row_size + ei;
  if (so >= n_elems || dof >= n_elems) return;
  float v = data[so];
  if (kv16 && dof >= kv_start && dof - kv_start < kv_count) {
    const __half h = __float2half(v);
    kv16[dof - kv_start] = h;
    v = __half2float(h);
  }
  data[dof] = v;
}

static int rmsnorm_impl(uint32_t map_act, uint32_t map_wt, uint32_t hs, uint32_t hw, uint32_t hr, uint32_t hd,
                        uint32_t n_rows, uint32_t dim, float eps, bool add) {
  Map* ma = get_f32_map(map_act);
  Map* mw = get_f32_map(map_wt);
  if (!ma || !mw) return ADAMAH_ERR_INVALID;
  if (n_rows == 0) return ADAMAH_OK;
  if (n_rows == 1 && dim > 0 && can_defer()) {
    // single row with operands known on the host: queue it, a neighbouring GEMV may absorb it
    PendOp p;
    if (res_scalar(hs, &p.a) && res_scalar(hw, &p.b) && res_scalar(hd, &p.c) && (!add || res_scalar(hr, &p.d)) &&
        in_range(p.a, dim, ma->n_elems) && in_range(p.c, dim, ma->n_elems) && in_range(p.b, dim, mw->n_elems) &&
        (!add || in_range(p.d, dim, ma->n_elems))) {
      p.kind = PK_RMSNORM; p.map_act = map_act; p.map_wt = map_wt; p.n = dim; p.op = add ? 1u : 0u; p.eps = eps;
      g.pend.push_back(p);
      return ADAMAH_OK;
    }
  }
  flush_pending();
  const uint32_t *ls = res_u32(hs, n_rows), *lw = res_u32(hw, n_rows), *ld = res_u32(hd, n_rows);
  const uint32_t* lr = add ? res_u32(hr, n_rows) : ls;
  if (!ls || !lw || !ld || !lr) return ADAMAH_ERR_INVALID;
  float* a = (float*)ma->buf;
  if (n_rows > 1 && dim <= 8192 && tuning("ADAMAH_RMSNORM_ROWS", 1) != 0) {
    // rows in registers; when the results are the rows of a matrix [n_rows, dim], also in the form the
    // batched matmul reads
    const uint32_t* dh = res_host(hd, n_rows);
    bool emit = dh && dim >= 128 && (dim & 127u) == 0 && n_rows <= 4096 && tuning("ADAMAH_RMSNORM_EMIT", 1) != 0;
    for (uint32_t i = 1; emit && i < n_rows; i++) emit = (uint64_t)dh[i] == (uint64_t)dh[0] + (uint64_t)i * dim;
    // the kernel skips a row whose operands are out of range: only rows the host can vouch for are marked
    const uint32_t *sh = res_host(hs, n_rows), *wh = res_host(hw, n_rows), *rh = add ? res_host(hr, n_rows) : nullptr;
    emit = emit && sh && wh && (!add || rh);
    for (uint32_t i = 0; emit && i < n_rows; i++)
      emit = in_range(sh[i], dim, ma->n_elems) && in_range(dh[i], dim, ma->n_elems) && in_range(wh[i], dim, mw->n_elems) &&
             (!add || in_range(rh[i], dim, ma->n_elems));
    float* scale = nullptr;
    __half *xh = nullptr, *xl = nullptr;
    if (emit) emit = gemm_act_slots(n_rows, dim, &scale, &xh, &xl);
    const float* w = (const float*)mw->buf;
    // evenly spaced rows (the usual case: rows of a matrix, one weight vector): their places go by value
    RowsByValue rv = {};
    {
      const uint32_t *s_h = res_host(hs, n_rows), *w_h = res_host(hw, n_rows), *d_h = res_host(hd, n_rows);
      const uint32_t* r_h = add ? res_host(hr, n_rows) : s_h;
      bool even = s_h && w_h && d_h && r_h && s_h[1] >= s_h[0] && w_h[1] >= w_h[0] && d_h[1] >= d_h[0] && r_h[1] >= r_h[0];
      if (even) {
        rv = {1u, s_h[0], s_h[1] - s_h[0], w_h[0], w_h[1] - w_h[0], d_h[0], d_h[1] - d_h[0], r_h[0], r_h[1] - r_h[0]};
        for (uint32_t i = 1; even && i < n_rows; i++)
          even = s_h[i] == s_h[0] + i * rv.ss && w_h[i] == w_h[0] + i * rv.ws && d_h[i] == d_h[0] + i * rv.ds &&
                 r_h[i] == r_h[0] + i * rv.rs;
      }
      if (!even) rv.on = 0u;
    }
#define RR(A, E, NU) k_rmsnorm_rows<A, E, NU><<<n_rows, 256, 0, g.stream>>>(a, w, dim | (rv.on << 31), eps, rv.s0, rv.ss, rv.w0, rv.ws, rv.d0, rv.ds, rv.r0, rv.rs, a, ls, lw, lr, ld, ma->n_elems, mw->n_elems, scale, xh, xl)
#define RN(A, E) do { if (dim <= 2048) RR(A, E, 8); else if (dim <= 4096) RR(A, E, 16); else RR(A, E, 32); } while (0)
    if (add) { if (emit) RN(true, true); else RN(true, false); }
    else { if (emit) RN(false, true); else RN(false, false); }
#undef RN
#undef RR
    count_launch();
    if (emit) gemm_act_mark(ma->buf, dh[0], n_rows, dim);
    return check_launch();
  }
  if (add)
    k_rmsnorm<true><<<n_rows, 256, 0, g.stream>>>(a, (const float*)mw->buf, a, ls, lw, lr, ld, dim, eps, ma->n_elems,
                                                  mw->n_elems);
  else
    k_rmsnorm<false><<<n_rows, 256, 0, g.stream>>>(a, (const float*)mw->buf, a, ls, lw, lr, ld, dim, eps, ma->n_elems,
                                                   mw->n_elems);
  count_launch();
  return check_launch();
}

// One token of many sequences in lockstep: the rotation of all their Q heads, the rotation of all their K heads and the
// append of the K and V rows to the caches (three ops, issued in that order) in one launch.  One workgroup per
// row: the Q rows, then the K rows, then the copies.  A copy whose source is a K row of the launch is done by that
// row's workgroup, which finds it in the copy list and stores the rotated row twice (in place, and to the cache with
// the cache's fp16 rounding); its own workgroup leaves at once.  The host has checked that every copy's source is
// either exactly one such K row (each at most once) or lies clear of both rotated ranges, and that all destinations
// lie in the fp16 KV range, which holds no source.  Arithmetic of the three stand-alone kernels.
__global__ void __launch_bounds__(256)
k_rope2_copy(float* data, uint32_t qa, uint32_t q_rows, uint32_t q_dim, uint32_t ka, uint32_t k_rows, uint32_t k_dim,
             uint32_t pos, float base, const uint32_t* __restrict__ spec, uint32_t src_base, uint32_t n_copies,
             uint32_t dst_row_offset, __half* kv16, uint64_t kv_start, uint64_t kv_count) {
  __shared__ uint32_t found;
  const uint32_t b = blockIdx.x, tid = threadIdx.x;
  auto put = [&](uint64_t dof, float v) {     // into the cache: rounded to fp16 and mirrored, as the row copy does
    if (kv16 && dof >= kv_start && dof - kv_start < kv_count) {
      const __half h = __float2half(v);
      kv16[dof - kv_start] = h;
      v = __half2float(h);
    }
    data[dof] = v;
  };
  if (b < q_rows + k_rows) {
    const bool is_q = b < q_rows;
    const uint32_t dim = is_q ? q_dim : k_dim, half = dim >> 1;
    const uint64_t row = is_q ? (uint64_t)qa + (uint64_t)b * q_dim : (uint64_t)ka + (uint64_t)(b - q_rows) * k_dim;
    uint32_t dst_row = 0xFFFFFFFFu;
    if (!is_q) {
      if (tid == 0) found = 0xFFFFFFFFu;
      __syncthreads();
      for (uint32_t ci = tid; ci < n_copies; ci += 256u)
        if ((uint64_t)src_base + (uint64_t)spec[2 * ci] * k_dim == row) found = spec[2 * ci + 1];   // at most one
      __syncthreads();
      dst_row = found;
    }
    for (uint32_t d = tid; d < half; d += 256u) {
      float c, s;
      rope_cs(d, dim, pos, base, &c, &s);
      const float x0 = data[row + d], x1 = data[row + d + half];
      const float r0 = x0 * c - x1 * s, r1 = x0 * s + x1 * c;
      data[row + d] = r0;
      data[row + d + half] = r1;
      if (dst_row != 0xFFFFFFFFu) {
        const uint64_t dof = ((uint64_t)dst_row + dst_row_offset) * k_dim;
        put(dof + d, r0);
        put(dof + d + half, r1);
      }
    }
    return;
  }
  const uint32_t ci = b - q_rows - k_rows;
  const uint64_t so = (uint64_t)src_base + (uint64_t)spec[2 * ci] * k_dim;
  if (so >= ka && so < (uint64_t)ka + (uint64_t)k_rows * k_dim) return;     // done by the K row's workgroup
  const uint64_t dof = ((uint64_t)spec[2 * ci + 1] + dst_row_offset) * k_dim;
  for (uint32_t e = tid; e < k_dim; e += 256u) put(dof + e, data[so + e]);
}

// A queued rotation (one token, more heads than a row run holds) or row copy (more copies than that) by itself.
static int launch_wide_alone(const PendOp& p, Map* m) {
  if (p.kind == PK_ROPE) {
    const uint32_t *ls = res_u32(p.h[0], 1), *ld = res_u32(p.h[1], 1);
    if (!ls || !ld) return ADAMAH_ERR_INVALID;
    const uint64_t pairs = (uint64_t)p.rpg * (p.k / 2);
    k_rope<<<cdiv(pairs, 256), 256, 0, g.stream>>>((float*)m->buf, ls, ld, 1, p.rpg, p.k, p.n, p.eps, m->n_elems);
  } else {
    const uint32_t *spec = res_u32(p.h[0], 2ull * p.rpg), *base = res_u32(p.h[1], 1);
    if (!spec || !base) return ADAMAH_ERR_INVALID;
    k_row_copy<<<cdiv((uint64_t)p.rpg * p.k, 256), 256, 0, g.stream>>>((float*)m->buf, spec, base, p.rpg, p.k, p.n, m->n_elems, m->kv16,
                                                                    m->kv_start, m->kv_count);
  }
  count_launch();
  return check_launch();
}

// q[i] is a wide rotation or row copy (op == 1).  Rotation of the Q heads, rotation of the K heads in place and the
// KV append behind them, all of one position: one launch; anything else: q[i] by itself.  Returns the entries used.
size_t launch_wide_rows(const std::vector<PendOp>& q, size_t i, int* rc) {
  Map* m = get_f32_map(q[i].map_act);
  if (!m) { *rc = ADAMAH_ERR_INVALID; return 1; }
  auto fold = [&]() -> bool {
    if (i + 2 >= q.size()) return false;
    const PendOp &pq = q[i], &pk = q[i + 1], &pc = q[i + 2];
    if (pq.kind != PK_ROPE || pk.kind != PK_ROPE || pc.kind != PK_ROWCOPY || pk.op != 1u || pc.op != 1u ||
        pk.map_act != pq.map_act || pc.map_act != pq.map_act || pq.a != pq.c || pk.a != pk.c || pk.n != pq.n || pk.eps != pq.eps ||
        pc.k != pk.k || !m->kv16)
      return false;
    const uint64_t q0 = pq.a, q1 = q0 + (uint64_t)pq.rpg * pq.k, k0 = pk.a, k1 = k0 + (uint64_t)pk.rpg * pk.k;
    const uint64_t c0 = m->kv_start, c1 = c0 + m->kv_count;
    auto apart = [](uint64_t a0, uint64_t a1, uint64_t b0, uint64_t b1) { return a1 <= b0 || b1 <= a0; };
    if (!apart(q0, q1, k0, k1) || !apart(q0, q1, c0, c1) || !apart(k0, k1, c0, c1)) return false;
    const uint32_t *spec = res_host(pc.h[0], 2ull * pc.rpg), *base = res_host(pc.h[1], 1);
    if (!spec || !base || !res_u32(pc.h[0], 2ull * pc.rpg)) return false;
    std::vector<uint8_t> seen(pk.rpg, 0);
    for (uint32_t ci = 0; ci < pc.rpg; ci++) {
      const uint64_t so = (uint64_t)base[0] + (uint64_t)spec[2 * ci] * pc.k, s1 = so + pc.k;
      const uint64_t d0 = ((uint64_t)spec[2 * ci + 1] + pc.n) * pc.k, d1 = d0 + pc.k;
      if (d0 < c0 || d1 > c1 || s1 > m->n_elems) return false;
      if (so >= k0 && so < k1) {
        if ((so - k0) % pk.k) return false;
        const uint64_t j = (so - k0) / pk.k;
        if (seen[j]) return false;
        seen[j] = 1;
      } else if (!apart(so, s1, k0, k1) || !apart(so, s1, q0, q1) || !apart(so, s1, c0, c1)) return false;
    }
    k_rope2_copy<<<pq.rpg + pk.rpg + pc.rpg, 256, 0, g.stream>>>((float*)m->buf, pq.a, pq.rpg, pq.k, pk.a, pk.rpg, pk.k, pq.n, pq.eps,
                                                              res_u32(pc.h[0], 2ull * pc.rpg), base[0], pc.rpg, pc.n, m->kv16,
                                                              m->kv_start, m->kv_count);
    count_launch();
    *rc = check_launch();
    return true;
  };
  if (q[i].kind == PK_ROPE && fold()) return 3;
  *rc = launch_wide_alone(q[i], m);
  return 1;
}

}  // namespace adamah

using namespace adamah;

extern "C" {

int map_rmsnorm_dev(uint32_t map_id, uint32_t hs, uint32_t hw, uint32_t hd, uint32_t n_rows, uint32_t dim, float eps) {
  return rmsnorm_impl(map_id, map_id, hs, hw, 0, hd, n_rows, dim, eps, false);
}
int map_rmsnorm_x_dev(uint32_t map_act, uint32_t map_wt, uint32_t hs, uint32_t hw, uint32_t hd, uint32_t n_rows,
                      uint32_t dim, float eps) {
  return rmsnorm_impl(map_act, map_wt, hs, hw, 0, hd, n_rows, dim, eps, false);
}
int map_rmsnorm_add_dev(uint32_t map_id, uint32_t hs, uint32_t hw, uint32_t hr, uint32_t hd, uint32_t n_rows,
                        uint32_t dim, float eps) {
  return rmsnorm_impl(map_id, map_id, hs, hw, hr, hd, n_rows, dim, eps, true);
}

int map_rope_dev(uint32_t map_id, uint32_t hs, uint32_t hd, uint32_t n_tokens, uint32_t n_heads, uint32_t head_dim,
                 uint32_t pos_offset, float freq_base) {
  Map* m = get_f32_map(map_id);
  if (!m) return ADAMAH_ERR_INVALID;
  const uint64_t pairs = (uint64_t)n_tokens * n_heads * (head_dim / 2);
  if (pairs == 0) return ADAMAH_OK;
  if (n_tokens == 1 && can_defer()) {
    // one token with operands known on the host: queue it, it may share a launch with the KV append
    PendOp p;
    p.kind = PK_ROPE; p.map_act = map_id; p.rpg = n_heads; p.k = head_dim; p.n = pos_offset; p.eps = freq_base;
    if (res_scalar(hs, &p.a) && res_scalar(hd, &p.c)) {
      if (row_op_deferrable(p)) { g.pend.push_back(p); return ADAMAH_OK; }
      // more heads than a row run holds (one token of many sequences): queued as well, it may share a launch with
      // the rotation and the KV append next to it
      if (n_heads > ROW_RUN_MAX && (head_dim & 1u) == 0 && in_range(p.a, (uint64_t)n_heads * head_dim, m->n_elems) &&
          in_range(p.c, (uint64_t)n_heads * head_dim, m->n_elems) && tuning("ADAMAH_ROWS_WIDE", 1) != 0) {
        p.op = 1u; p.h[0] = hs; p.h[1] = hd;
        g.pend.push_back(p);
        return ADAMAH_OK;
      }
    }
  }
  flush_pending();
  const uint32_t *ls = res_u32(hs, n_tokens), *ld = res_u32(hd, n_tokens);
  if (!ls || !ld) return ADAMAH_ERR_INVALID;
  k_rope<<<cdiv(pairs, 256), 256, 0, g.stream>>>((float*)m->buf, ls, ld, n_tokens, n_heads, head_dim, pos_offset,
                                                  freq_base, m->n_elems);
  count_launch();
  return check_launch();
}

int map_qk_norm_rope_x_dev(uint32_t map_act, uint32_t map_wt, uint32_t hqs, uint32_t hqw, uint32_t hks, uint32_t hkw,
                           uint32_t hdst, uint32_t q_rows, uint32_t q_dim, uint32_t k_rows, uint32_t k_dim,
                           uint32_t pos_offset, float freq_base) {
  Map* ma = get_f32_map(map_act);
  Map* mw = get_f32_map(map_wt);
  if (!ma || !mw) return ADAMAH_ERR_INVALID;
  if (q_rows + k_rows == 0) return ADAMAH_OK;
  if (map_act == map_wt && can_defer()) {
    PendOp p;
    p.kind = PK_QKNR; p.map_act = map_act; p.map_wt = map_wt; p.rpg = q_rows; p.k = q_dim; p.op = k_rows; p.d = k_dim;
    p.n = pos_offset; p.eps = freq_base;
    p.h[0] = hqs; p.h[1] = hqw; p.h[2] = hks; p.h[3] = hkw; p.h[4] = hdst;
    if (row_op_deferrable(p)) { g.pend.push_back(p); return ADAMAH_OK; }
  }
  flush_pending();
  const uint32_t* one = res_u32(hdst, 1);
  const uint32_t *lqs = q_rows ? res_u32(hqs, q_rows) : one, *lqw = q_rows ? res_u32(hqw, q_rows) : one;
  const uint32_t *lks = k_rows ? res_u32(hks, k_rows) : one, *lkw = k_rows ? res_u32(hkw, k_rows) : one;
  if (!one || !lqs || !lqw || !lks || !lkw) return ADAMAH_ERR_INVALID;
  k_qk_norm_rope<<<q_rows + k_rows, 256, 0, g.stream>>>((float*)ma->buf, (const float*)mw->buf, lqs, lqw, lks, lkw, one,
                                                        q_rows, q_dim, k_rows, k_dim, pos_offset, freq_base,
                                                        ma->n_elems, mw->n_elems);
  count_launch();
  return check_launch();
}

int map_row_copy_offset_dev(uint32_t map_id, uint32_t hspec, uint32_t hbase, uint32_t dst_row_offset, uint32_t n_copies,
                            uint32_t row_size) {
  Map* m = get_f32_map(map_id);
  if (!m) return ADAMAH_ERR_INVALID;
  if (n_copies == 0 || row_size == 0) return ADAMAH_OK;
  if (can_defer()) {
    PendOp p;
    p.kind = PK_ROWCOPY; p.map_act = map_id; p.h[0] = hspec; p.h[1] = hbase; p.rpg = n_copies; p.k = row_size;
    p.n = dst_row_offset;
    if (row_op_deferrable(p)) { g.pend.push_back(p); return ADAMAH_OK; }
    if (n_copies > ROW_RUN_MAX && res_host(hspec, 2ull * n_copies) && res_host(hbase, 1) && tuning("ADAMAH_ROWS_WIDE", 1) != 0) {
      p.op = 1u;     // more copies than a row run holds: queued as well (see map_rope_dev); operands checked at launch
      g.pend.push_back(p);
      return ADAMAH_OK;
    }
  }
  flush_pending();
  const uint32_t *spec = res_u32(hspec, 2ull * n_copies), *base = res_u32(hbase, 1);
  if (!spec || !base) return ADAMAH_ERR_INVALID;
  k_row_copy<<<cdiv((uint64_t)n_copies * row_size, 256), 256, 0, g.stream>>>(
      (float*)m->buf, spec, base, n_copies, row_size, dst_row_offset, m->n_elems, m->kv16, m->kv_start, m->kv_count);
  count_launch();
  return check_launch();
}
int map_row_copy_dev(uint32_t map_id, uint32_t hspec, uint32_t hbase, uint32_t n_copies, uint32_t row_size) {
  return map_row_copy_offset_dev(map_id, hspec, hbase, 0, n_copies, row_size);
}

int adamah_qk_norm_rope_rows_dev(uint32_t map_act, uint32_t map_wt, const uint32_t* q_src_handles, uint32_t locs_q_wt,
                                 const uint32_t* k_src_handles, uint32_t locs_k_wt, const uint32_t* dst_handles,
                                 uint32_t m, uint32_t q_rows, uint32_t q_dim, uint32_t k_rows, uint32_t k_dim,
                                 uint32_t pos0, float freq_base) {
  if (m == 0) return ADAMAH_OK;
  if (!q_src_handles || !k_src_handles || !dst_handles) return ADAMAH_ERR_INVALID;
  for (uint32_t t = 0; t < m; t++) {
    const int r = map_qk_norm_rope_x_dev(map_act, map_wt, q_src_handles[t], locs_q_wt, k_src_handles[t], locs_k_wt,
                                         dst_handles[t], q_rows, q_dim, k_rows, k_dim, pos0 + t, freq_base);
    if (r != ADAMAH_OK) return r;
  }
  return ADAMAH_OK;
}

}  // extern "C"
