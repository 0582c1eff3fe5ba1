// LM-head tail for sampled decoding: logits of a quantised [N, K] matrix reduced on the device to a
// partial top-k list per group of rows (with the repeat penalty applied before ranking), and the exact
// re-scoring of a shortlist of token ids.
//
// Reference: shaders/src/f32/map_matvec_topk_t_xq4.comp:85-208 and map_matvec_topk_t_xq8.comp (one
// workgroup per group of rows: dot products, penalty, insertion into a sorted list of k <= 64),
// map_matvec_rerank_t_xq8.comp:43-82; dispatch adamah.c:9727-9830 (Q4), :9911-10016 (Q8),
// :10018-10110 (rerank).  The callers are the sampled branches of the decode loop
// (adam/models/engine.py:3342-3480, 3573-3680).
//
// Here the dot products run on the ordinary GEMV kernels into a scratch vector owned by the library
// (the int8 matrix-instruction kernel for Q4 block matrices, one wave per row otherwise); a second
// launch ranks every group.  The ranking order is the reference's: larger value first, equal values
// by smaller row index; slots a group cannot fill hold index 0 and the most negative float.  A NaN
// logit ranks as the most negative float (the reference's insertion leaves a NaN wherever it was
// first put, which no caller relies on).  Groups of up to 1024 rows are ranked by counting, for every
// row, the rows that beat it; larger groups by k rounds of a workgroup-wide best-of.
#include "gemv_common.h"
#include <cstdio>
#include <algorithm>
#include "../../include/adamah_hip.h"

// Logit scratch of the entry point that allocates nothing (adamah_matvec_topk_t_xq4_noalloc_dev): part of
// the code object, one copy per GPU at that GPU's own address, held until the process ends.  In host code
// this name is only a stand-in for the symbol: the device address comes from hipGetSymbolAddress
// (topk_noalloc_setup) and only that pointer is ever handed to a kernel.
#define NOALLOC_MAX_ROWS 262144u
static __device__ __align__(256) float scratch[NOALLOC_MAX_ROWS];

namespace adamah {

#define TOPK_MAX 64u
#define NOALLOC_MAX_DEVICES 16

static float* g_noalloc_ptr[NOALLOC_MAX_DEVICES] = {nullptr};

// Called by adamah_init with the library's device current: resolves this device's copy of `scratch`.
int topk_noalloc_setup(int device) {
  if (device < 0 || device >= NOALLOC_MAX_DEVICES) return ADAMAH_ERR_INVALID;
  if (g_noalloc_ptr[device]) return ADAMAH_OK;
  float* p = nullptr;
  if (hipGetSymbolAddress((void**)&p, HIP_SYMBOL(scratch)) != hipSuccess || !p) {
    (void)hipGetLastError();
    return ADAMAH_ERR_BACKEND;
  }
  g_noalloc_ptr[device] = p;
  return ADAMAH_OK;
}

static float* g_logit_buf = nullptr;
static size_t g_logit_cap = 0;   // floats

void topk_fused_release() {
  if (g_logit_buf) hipFree(g_logit_buf);
  g_logit_buf = nullptr;
  g_logit_cap = 0;
}

// out[row] = x . W[row], affine dequantisation; one wave per row, any base / K / group size
template <bool Q4>
__global__ void __launch_bounds__(256)
k_matvec_rows(const float* act, const uint8_t* __restrict__ W, const float2* __restrict__ qp,
              const uint32_t* __restrict__ la, const uint32_t* __restrict__ lb, float* out, uint32_t K, uint32_t N,
              uint32_t group, uint64_t act_elems, uint64_t wt_elems) {
  const uint32_t lane = threadIdx.x & 63u, row = blockIdx.x * 4u + (threadIdx.x >> 6);
  if (row >= N) return;
  const uint64_t a = la[0], b = (uint64_t)lb[0] + (uint64_t)row * K;
  float s = 0.f;
  for (uint32_t k = lane; k < K; k += 64u)
    if (a + k < act_elems && b + k < wt_elems) s = fmaf(act[a + k], deq_elem(W, qp, b + k, group, Q4), s);
  s = wave_sum(s);
  if (lane == 0) out[row] = s;
}

__device__ __forceinline__ float penalised(float v, float rp) { return v > 0.f ? v / rp : v * rp; }

// One workgroup per group of rows.  The penalty is applied in place to the scratch logits (each
// distinct id once, as the reference's membership test does), then k rounds pick the best row that
// ranks strictly after the previous pick.
__global__ void __launch_bounds__(256)
k_group_topk(float* act, float* logits, const uint32_t* __restrict__ pen, const uint32_t* __restrict__ lidx,
             const uint32_t* __restrict__ lval, uint32_t N, uint32_t k, uint32_t n_pen, float rp, uint32_t rows_per_group,
             uint64_t act_elems) {
  __shared__ uint32_t pen_s[TOPK_MAX];
  __shared__ float red_v[4];
  __shared__ uint32_t red_i[4];
  const uint32_t tid = threadIdx.x, lane = tid & 63u, wave = tid >> 6, grp = blockIdx.x;
  const uint32_t row0 = grp * rows_per_group, row1 = min(N, row0 + rows_per_group);
  if (tid < n_pen) pen_s[tid] = pen[tid];
  __syncthreads();
  if (tid < n_pen) {
    const uint32_t id = pen_s[tid];
    bool first = id >= row0 && id < row1;
    for (uint32_t j = 0; j < tid; j++) first = first && pen_s[j] != id;
    if (first) logits[id] = penalised(logits[id], rp);
  }
  __threadfence_block();
  __syncthreads();
  float pv = 0.f;
  uint32_t pi = INVALID_IDX;   // previous pick; INVALID before the first round
  for (uint32_t t = 0; t < k; t++) {
    float bv = NEG_FLT_MAX;
    uint32_t bi = INVALID_IDX;
    for (uint32_t r = row0 + tid; r < row1; r += 256u) {
      float v = logits[r];
      if (v != v) v = NEG_FLT_MAX;
      const bool after = t == 0u || (pi != INVALID_IDX && ((pv > v) || (pv == v && pi < r)));
      if (after && better(v, r, bv, bi)) { bv = v; bi = r; }
    }
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) {
      const float ov = __shfl_xor(bv, o, 64);
      const uint32_t oi = __shfl_xor(bi, o, 64);
      if (better(ov, oi, bv, bi)) { bv = ov; bi = oi; }
    }
    if (lane == 0) { red_v[wave] = bv; red_i[wave] = bi; }
    __syncthreads();
    bv = red_v[0]; bi = red_i[0];
#pragma unroll
    for (int w = 1; w < 4; w++)
      if (better(red_v[w], red_i[w], bv, bi)) { bv = red_v[w]; bi = red_i[w]; }
    __syncthreads();
    if (tid == 0) {
      const uint64_t di = lidx[(uint64_t)grp * k + t], dv = lval[(uint64_t)grp * k + t];
      if (di < act_elems) act[di] = (float)(bi == INVALID_IDX ? 0u : bi);
      if (dv < act_elems) act[dv] = bi == INVALID_IDX ? NEG_FLT_MAX : bv;
    }
    pv = bv; pi = bi;
    if (bi == INVALID_IDX && t > 0u) {   // nothing left: the remaining slots stay empty
      if (tid == 0)
        for (uint32_t u = t + 1; u < k; u++) {
          const uint64_t di = lidx[(uint64_t)grp * k + u], dv = lval[(uint64_t)grp * k + u];
          if (di < act_elems) act[di] = 0.f;
          if (dv < act_elems) act[dv] = NEG_FLT_MAX;
        }
      break;
    }
  }
}

// Groups of at most 1024 rows: the group's (penalised) logits sit in LDS, every thread counts the rows
// that rank before its own and stores those with fewer than k of them straight into their slot.
#define RANK_MAX 1024u
__global__ void __launch_bounds__(256)
k_group_topk_rank(float* act, const float* __restrict__ logits, const uint32_t* __restrict__ pen,
                  const uint32_t* __restrict__ lidx, const uint32_t* __restrict__ lval, uint32_t N, uint32_t k,
                  uint32_t n_pen, float rp, uint32_t rows_per_group, uint64_t act_elems) {
  __shared__ float vs[RANK_MAX];
  __shared__ uint32_t pen_s[TOPK_MAX];
  const uint32_t tid = threadIdx.x, grp = blockIdx.x;
  const uint32_t row0 = grp * rows_per_group, rows = min(N, row0 + rows_per_group) - row0;
  for (uint32_t i = tid; i < rows; i += 256u) {
    const float v = logits[row0 + i];
    vs[i] = v != v ? NEG_FLT_MAX : v;
  }
  // padding of the last quad: NaN compares false both ways, so it is never counted
  for (uint32_t i = rows + tid; i < ((rows + 3u) & ~3u); i += 256u) vs[i] = __uint_as_float(0x7FC00000u);
  if (tid < n_pen) pen_s[tid] = pen[tid];
  __syncthreads();
  if (tid < n_pen) {
    const uint32_t id = pen_s[tid];
    bool first = id >= row0 && id - row0 < rows;
    for (uint32_t j = 0; j < tid; j++) first = first && pen_s[j] != id;
    if (first) vs[id - row0] = penalised(vs[id - row0], rp);
  }
  __syncthreads();
  for (uint32_t i = tid; i < rows; i += 256u) {
    const float v = vs[i];
    uint32_t cnt = 0;
    for (uint32_t j = 0; j < rows; j += 4u) {   // branch-free: rows before i win ties
      const float4 w = *(const float4*)&vs[j];
      cnt += (uint32_t)(w.x > v) | ((uint32_t)(w.x == v) & (uint32_t)(j < i));
      cnt += (uint32_t)(w.y > v) | ((uint32_t)(w.y == v) & (uint32_t)(j + 1u < i));
      cnt += (uint32_t)(w.z > v) | ((uint32_t)(w.z == v) & (uint32_t)(j + 2u < i));
      cnt += (uint32_t)(w.w > v) | ((uint32_t)(w.w == v) & (uint32_t)(j + 3u < i));
    }
    if (cnt < k) {
      const uint64_t di = lidx[(uint64_t)grp * k + cnt], dv = lval[(uint64_t)grp * k + cnt];
      if (di < act_elems) act[di] = (float)(row0 + i);
      if (dv < act_elems) act[dv] = v;
    }
  }
  for (uint32_t t = rows + tid; t < k; t += 256u) {   // slots the group cannot fill
    const uint64_t di = lidx[(uint64_t)grp * k + t], dv = lval[(uint64_t)grp * k + t];
    if (di < act_elems) act[di] = 0.f;
    if (dv < act_elems) act[dv] = NEG_FLT_MAX;
  }
}

// One wave per shortlisted id: token = partial list entry picked by sel, exact logit of its row.
__global__ void __launch_bounds__(64)
k_rerank_q8(float* act, const uint8_t* __restrict__ W, const float2* __restrict__ qp, const uint32_t* __restrict__ la,
            const uint32_t* __restrict__ lb, const uint32_t* __restrict__ lpart, const uint32_t* __restrict__ lsel,
            const uint32_t* __restrict__ pen, const uint32_t* __restrict__ lidx, const uint32_t* __restrict__ lval,
            uint32_t K, uint32_t n_pen, float rp, uint32_t group, uint64_t act_elems, uint64_t wt_elems) {
  const uint32_t row = blockIdx.x, lane = threadIdx.x;
  const uint64_t a = la[0], sl = lsel[row];
  const float selv = sl < act_elems ? act[sl] : 0.f;
  const uint64_t pl = (uint64_t)lpart[0] + (uint32_t)fmaxf(selv, 0.f);
  const float tokv = pl < act_elems ? act[pl] : 0.f;
  const uint32_t tok = (uint32_t)fmaxf(tokv, 0.f);
  const uint64_t b = (uint64_t)lb[0] + (uint64_t)tok * K;
  float s = 0.f;
  for (uint32_t k = lane; k < K; k += 64u)
    if (a + k < act_elems && b + k < wt_elems) s = fmaf(act[a + k], deq_elem(W, qp, b + k, group, false), s);
  s = wave_sum(s);
  if (lane == 0) {
    bool hit = false;
    for (uint32_t i = 0; i < n_pen; i++) hit = hit || pen[i] == tok;
    if (hit) s = penalised(s, rp);
    const uint64_t di = lidx[row], dv = lval[row];
    if (di < act_elems) act[di] = (float)tok;
    if (dv < act_elems) act[dv] = s;
  }
}

static int op_matvec_topk(uint32_t dtype, uint32_t map_act, uint32_t map_wt, uint32_t ha, uint32_t hb, uint32_t hpen,
                          uint32_t hidx, uint32_t hval, uint32_t K, uint32_t N, uint32_t k, uint32_t n_pen, float rp,
                          uint32_t rows_per_group, float* fixed_logits = nullptr) {
  Map* ma = get_map(map_act);
  Map* mw = get_map(map_wt);
  if (!ma || !mw) return ADAMAH_ERR_INVALID;
  if (N == 0 || k == 0) return ADAMAH_OK;
  if (k > TOPK_MAX || n_pen > TOPK_MAX) return ADAMAH_ERR_INVALID;
  if (rows_per_group == 0) return ADAMAH_ERR_INVALID;
  if (ma->dtype != DTYPE_F32 || mw->dtype != dtype || !mw->qp || mw->group_size == 0) return ADAMAH_ERR_INVALID;
  const uint32_t n_groups = cdiv(N, rows_per_group);
  const uint32_t *la = res_u32(ha, 1), *lb = res_u32(hb, 1), *lidx = res_u32(hidx, (uint64_t)n_groups * k),
                 *lval = res_u32(hval, (uint64_t)n_groups * k);
  const uint32_t* pen = n_pen ? res_u32(hpen, n_pen) : nullptr;
  if (!la || !lb || !lidx || !lval || !get_res(hpen) || (n_pen && !pen)) return ADAMAH_ERR_INVALID;
  const uint32_t *ah = res_host(ha, 1), *bh = res_host(hb, 1);
  if (ah && !in_range(ah[0], K, ma->n_elems)) return ADAMAH_ERR_INVALID;
  if (bh && !in_range(bh[0], (uint64_t)N * K, mw->n_elems)) return ADAMAH_ERR_INVALID;
  // fixed_logits: the caller's scratch of at least N floats (the entry point that may not allocate)
  if (!fixed_logits && N > g_logit_cap) {
    layout_changed();
    if (g_logit_buf) { hipStreamSynchronize(g.stream); hipFree(g_logit_buf); }
    g_logit_cap = std::max<size_t>(N, 1u << 16);
    if (hipMalloc((void**)&g_logit_buf, g_logit_cap * sizeof(float)) != hipSuccess) {
      g_logit_buf = nullptr; g_logit_cap = 0;
      return ADAMAH_ERR_MEMORY;
    }
  }
  float* const logits = fixed_logits ? fixed_logits : g_logit_buf;
  float* act = (float*)ma->buf;
  uint64_t a0 = 0, b0 = 0;
  int r;
  if (dtype == DTYPE_Q4 && block_path_ok(ma, mw, ha, hb, K, N, &a0, &b0) && mfma_path_ok(mw, K) &&
      tuning("ADAMAH_GEMV_IMPL", 3) == 3) {
    r = launch_mfma_store(fmt_of(mw, b0, (uint64_t)N * K), ma, mw, (uint32_t)a0, (uint32_t)b0, 0u, K, N, nullptr,
                          logits);
  } else if (block_path_ok(ma, mw, ha, hb, K, N, &a0, &b0) && (uint64_t)K * 4 + (K >> 5) * 4 <= 64000 &&
             tuning("ADAMAH_TOPK_BLOCK", 1) != 0) {
    // block layout without the matrix-instruction kernel (Q8_0 LM heads): the fp32 block GEMV, 5-6 x the rate of
    // the one-wave-per-row kernel below (128256 x 4096 Q8_0: 637 -> 100 us)
    r = launch_block_store_to(fmt_of(mw, b0, (uint64_t)N * K), ma, mw, la, lb, K, N, logits);
  } else {
    if (dtype == DTYPE_Q4)
      k_matvec_rows<true><<<cdiv(N, 4), 256, 0, g.stream>>>(act, mw->buf, mw->qp, la, lb, logits, K, N,
                                                            mw->group_size, ma->n_elems, mw->n_elems);
    else
      k_matvec_rows<false><<<cdiv(N, 4), 256, 0, g.stream>>>(act, mw->buf, mw->qp, la, lb, logits, K, N,
                                                             mw->group_size, ma->n_elems, mw->n_elems);
    count_launch();
    r = check_launch();
  }
  if (r) return r;
  // counting costs rows^2 / 256 comparisons per thread, the rounds k * (rows / 256 + a reduction)
  const uint64_t rws = std::min(rows_per_group, N);
  const bool by_rank = rows_per_group <= RANK_MAX && rws * rws / 256u <= (uint64_t)k * (rws / 256u + 40u);
  if (tuning("ADAMAH_TOPK_RANK", by_rank ? 1 : 0) != 0 && rows_per_group <= RANK_MAX)
    k_group_topk_rank<<<n_groups, 256, 0, g.stream>>>(act, logits, pen, lidx, lval, N, k, n_pen, rp,
                                                      rows_per_group, ma->n_elems);
  else
    k_group_topk<<<n_groups, 256, 0, g.stream>>>(act, logits, pen, lidx, lval, N, k, n_pen, rp, rows_per_group,
                                                 ma->n_elems);
  count_launch();
  return check_launch();
}

// ---- several GEMV + argmax ops over one matrix: one pass over the weights -------------------------
// Lockstep decoding asks for the LM head once per sequence, over consecutive activation rows.  The rows
// go through the matrix-core GEMM together (weights read once instead of once per row), the logits
// [m, N] into the scratch buffer; the two kernels below then produce what every op would have: the
// per-group (index, value) partials -- all ops name the same lists, so the last op's remain -- and
// each op's token.

// best row of group blockIdx.x for activation row blockIdx.y; pairs[row][group] = (value, index bits)
__global__ void __launch_bounds__(256)
k_rows_group_argmax(float* __restrict__ act, const float* __restrict__ logits, const uint32_t* __restrict__ lidx,
                    const uint32_t* __restrict__ lval, float2* __restrict__ pairs, uint32_t N, uint32_t rows_per_group,
                    uint32_t n_groups, uint32_t last, uint64_t act_elems) {
  __shared__ float sv[256];
  __shared__ uint32_t si[256];
  const uint32_t tid = threadIdx.x, grp = blockIdx.x, j = blockIdx.y;
  const uint32_t row0 = grp * rows_per_group, row1 = min(N, row0 + rows_per_group);
  const float* y = logits + (uint64_t)j * N;
  float bv = NEG_FLT_MAX; uint32_t bi = INVALID_IDX;
  for (uint32_t r = row0 + tid; r < row1; r += 256u)
    if (better(y[r], r, bv, bi)) { bv = y[r]; bi = r; }
  sv[tid] = bv; si[tid] = bi;
  __syncthreads();
  for (uint32_t s = 128; s > 0; s >>= 1) {
    if (tid < s && better(sv[tid + s], si[tid + s], sv[tid], si[tid])) { sv[tid] = sv[tid + s]; si[tid] = si[tid + s]; }
    __syncthreads();
  }
  if (tid == 0) {
    pairs[(uint64_t)j * n_groups + grp] = make_float2(sv[0], __uint_as_float(si[0]));
    if (j == last) {
      if (lidx[grp] < act_elems) act[lidx[grp]] = (float)(si[0] == INVALID_IDX ? 0u : si[0]);
      if (lval[grp] < act_elems) act[lval[grp]] = sv[0];
    }
  }
}

struct RowDsts { const uint32_t* p[16]; };

// best pair of activation row blockIdx.x -> its token slot
__global__ void __launch_bounds__(256)
k_rows_argmax_pairs(float* __restrict__ act, const float2* __restrict__ pairs, RowDsts dst, uint32_t n_groups,
                    uint64_t act_elems) {
  __shared__ float sv[256];
  __shared__ uint32_t si[256];
  const uint32_t tid = threadIdx.x, j = blockIdx.x;
  float bv = NEG_FLT_MAX; uint32_t bi = INVALID_IDX;
  for (uint32_t i = tid; i < n_groups; i += 256u) {
    const float2 pr = pairs[(uint64_t)j * n_groups + i];
    if (better(pr.x, __float_as_uint(pr.y), bv, bi)) { bv = pr.x; bi = __float_as_uint(pr.y); }
  }
  sv[tid] = bv; si[tid] = bi;
  __syncthreads();
  for (uint32_t s = 128; s > 0; s >>= 1) {
    if (tid < s && better(sv[tid + s], si[tid + s], sv[tid], si[tid])) { sv[tid] = sv[tid + s]; si[tid] = si[tid + s]; }
    __syncthreads();
  }
  const uint32_t d = dst.p[j][0];
  if (tid == 0 && d < act_elems) act[d] = (float)(si[0] == INVALID_IDX ? 0u : si[0]);
}

// q[i] is a queued GEMV + argmax: when it starts a run of such ops over the same matrix, the same partial
// lists and consecutive activation rows, launches the run and returns its length (0: not a run).
size_t launch_argmax_run(const std::vector<PendOp>& q, size_t i, int* rc) {
  const PendOp& p = q[i];
  if (p.kind != PK_ARGMAX || (p.op != FMT_Q4_B16 && p.op != FMT_Q8_B16) || p.k < 128 || (p.k & 127u) || p.n == 0) return 0;
  if (i + 1 >= q.size() || q[i + 1].kind != PK_ARGMAX || tuning("ADAMAH_ARGMAX_RUN", 1) == 0) return 0;
  size_t m = 1;
  while (i + m < q.size() && m < 16) {
    const PendOp& x = q[i + m];
    if (x.kind != PK_ARGMAX || x.map_act != p.map_act || x.map_wt != p.map_wt || x.b != p.b || x.k != p.k || x.n != p.n ||
        x.rpg != p.rpg || x.op != p.op || x.h[0] != p.h[0] || x.h[1] != p.h[1] ||
        (uint64_t)x.a != (uint64_t)p.a + (uint64_t)m * p.k)
      break;
    m++;
  }
  if (m < 2) return 0;
  Map* ma = get_f32_map(p.map_act);
  Map* mw = get_map(p.map_wt);
  if (!ma || !mw) return 0;
  const uint32_t N = p.n, K = p.k, n_groups = cdiv(N, p.rpg);
  const uint32_t *ih = res_host(p.h[0], n_groups), *vh = res_host(p.h[1], n_groups);
  const uint32_t *lidx = res_u32(p.h[0], n_groups), *lval = res_u32(p.h[1], n_groups);
  const uint32_t *la = res_u32(p.h[3], 1), *lb = res_u32(p.h[4], 1);
  if (!ih || !vh || !lidx || !lval || !la || !lb) return 0;
  // Every op reads its row after the earlier ops have stored their partials and tokens: none of those
  // may land on the rows, and no token slot inside the span of the partial lists (a later op's
  // partials would overwrite it).
  const uint64_t a0 = p.a, a1 = a0 + (uint64_t)m * K;
  uint32_t lo = 0xFFFFFFFFu, hi = 0;
  for (uint32_t gq = 0; gq < n_groups; gq++) {
    lo = std::min(lo, std::min(ih[gq], vh[gq]));
    hi = std::max(hi, std::max(ih[gq], vh[gq]));
  }
  if ((uint64_t)hi >= a0 && (uint64_t)lo < a1) return 0;
  RowDsts dst;
  for (size_t j = 0; j < m; j++) {
    const uint32_t* dh = res_host(q[i + j].h[2], 1);
    dst.p[j] = res_u32(q[i + j].h[2], 1);
    if (!dh || !dst.p[j] || ((uint64_t)dh[0] >= a0 && (uint64_t)dh[0] < a1) || (dh[0] >= lo && dh[0] <= hi)) return 0;
  }
  const size_t need = (size_t)m * N + 2 * (size_t)m * n_groups + 2;
  if (need > g_logit_cap) {
    layout_changed();
    if (g_logit_buf) { hipStreamSynchronize(g.stream); hipFree(g_logit_buf); }
    g_logit_cap = std::max<size_t>(need, 1u << 16);
    if (hipMalloc((void**)&g_logit_buf, g_logit_cap * sizeof(float)) != hipSuccess) {
      g_logit_buf = nullptr; g_logit_cap = 0;
      *rc = ADAMAH_ERR_MEMORY;
      return m;
    }
  }
  float2* pairs = (float2*)(g_logit_buf + (((size_t)m * N + 1) & ~(size_t)1));
  int r = launch_gemm_q4_mfma(ma, mw, la, lb, nullptr, (uint32_t)m, K, N, 1, p.op == FMT_Q8_B16, g_logit_buf, (int64_t)p.a);
  if (r) { *rc = r; return m; }
  k_rows_group_argmax<<<dim3(n_groups, (uint32_t)m), 256, 0, g.stream>>>((float*)ma->buf, g_logit_buf, lidx, lval, pairs, N,
                                                                         p.rpg, n_groups, (uint32_t)m - 1, ma->n_elems);
  count_launch();
  k_rows_argmax_pairs<<<(uint32_t)m, 256, 0, g.stream>>>((float*)ma->buf, pairs, dst, n_groups, ma->n_elems);
  count_launch();
  *rc = check_launch();
  return m;
}


}  // namespace adamah

using namespace adamah;

extern "C" {

int map_matvec_topk_t_xq4_ex_dev(uint32_t ma, uint32_t mw, uint32_t a, uint32_t b, uint32_t pen, uint32_t idx,
                                 uint32_t val, uint32_t K, uint32_t N, uint32_t k, uint32_t n_penalty,
                                 float repeat_penalty, uint32_t rows_per_group) { ADAMAH_API();
  return op_matvec_topk(DTYPE_Q4, ma, mw, a, b, pen, idx, val, K, N, k, n_penalty, repeat_penalty, rows_per_group);
}
int map_matvec_topk_t_xq4_dev(uint32_t ma, uint32_t mw, uint32_t a, uint32_t b, uint32_t pen, uint32_t idx, uint32_t val,
                              uint32_t K, uint32_t N, uint32_t k, uint32_t n_penalty, float repeat_penalty) { ADAMAH_API();
  return op_matvec_topk(DTYPE_Q4, ma, mw, a, b, pen, idx, val, K, N, k, n_penalty, repeat_penalty, 256u);
}
int map_matvec_topk_t_xq8_ex_dev(uint32_t ma, uint32_t mw, uint32_t a, uint32_t b, uint32_t pen, uint32_t idx,
                                 uint32_t val, uint32_t K, uint32_t N, uint32_t k, uint32_t n_penalty,
                                 float repeat_penalty, uint32_t rows_per_group) { ADAMAH_API();
  return op_matvec_topk(DTYPE_Q8, ma, mw, a, b, pen, idx, val, K, N, k, n_penalty, repeat_penalty, rows_per_group);
}
int map_matvec_topk_t_xq8_dev(uint32_t ma, uint32_t mw, uint32_t a, uint32_t b, uint32_t pen, uint32_t idx, uint32_t val,
                              uint32_t K, uint32_t N, uint32_t k, uint32_t n_penalty, float repeat_penalty) { ADAMAH_API();
  return op_matvec_topk(DTYPE_Q8, ma, mw, a, b, pen, idx, val, K, N, k, n_penalty, repeat_penalty, 256u);
}

// The _ex form above for callers that cannot allocate (under HIP graph capture, in serving loops or
// harnesses that forbid hipMalloc): same arguments, same results, but the logits go to the fixed `scratch`
// array of this GPU instead of a buffer the library grows.  No hipMalloc / hipFree on this path.
int adamah_matvec_topk_t_xq4_noalloc_dev(uint32_t ma, uint32_t mw, uint32_t a, uint32_t b, uint32_t pen, uint32_t idx,
                                         uint32_t val, uint32_t K, uint32_t N, uint32_t k, uint32_t n_penalty,
                                         float repeat_penalty, uint32_t rows_per_group) {
  if (!g.initialized) return ADAMAH_ERR_INVALID;
  if (!g.pend.empty()) {
    // launching the queued ops of an open batch could grow library buffers: the caller has them launched first (adamah_sync, batch_end)
    fprintf(stderr, "adamah_matvec_topk_t_xq4_noalloc_dev: ops are queued in the open batch; call adamah_sync or batch_end first\n");
    return ADAMAH_ERR_INVALID;
  }
  if (N > NOALLOC_MAX_ROWS) {
    fprintf(stderr, "adamah_matvec_topk_t_xq4_noalloc_dev: N = %u exceeds the fixed scratch of %u rows\n", N, NOALLOC_MAX_ROWS);
    return ADAMAH_ERR_INVALID;
  }
  float* const sp = (g.device >= 0 && g.device < NOALLOC_MAX_DEVICES) ? g_noalloc_ptr[g.device] : nullptr;
  if (!sp) return ADAMAH_ERR_BACKEND;
  return op_matvec_topk(DTYPE_Q4, ma, mw, a, b, pen, idx, val, K, N, k, n_penalty, repeat_penalty, rows_per_group, sp);
}

int map_matvec_rerank_t_xq8_dev(uint32_t map_act, uint32_t map_wt, uint32_t ha, uint32_t hb, uint32_t hpart,
                                uint32_t hsel, uint32_t hpen, uint32_t hidx, uint32_t hval, uint32_t K, uint32_t n_ids,
                                uint32_t n_penalty, float repeat_penalty) { ADAMAH_API();
  Map* ma = get_map(map_act);
  Map* mw = get_map(map_wt);
  if (!ma || !mw) return ADAMAH_ERR_INVALID;
  if (n_ids == 0) return ADAMAH_OK;
  if (n_ids > TOPK_MAX || n_penalty > TOPK_MAX) return ADAMAH_ERR_INVALID;
  if (ma->dtype != DTYPE_F32 || mw->dtype != DTYPE_Q8 || !mw->qp || mw->group_size == 0) return ADAMAH_ERR_INVALID;
  const uint32_t *la = res_u32(ha, 1), *lb = res_u32(hb, 1), *lp = res_u32(hpart, 1), *ls = res_u32(hsel, n_ids),
                 *li = res_u32(hidx, n_ids), *lv = res_u32(hval, n_ids);
  const uint32_t* pen = n_penalty ? res_u32(hpen, n_penalty) : nullptr;
  if (!la || !lb || !lp || !ls || !li || !lv || !get_res(hpen) || (n_penalty && !pen)) return ADAMAH_ERR_INVALID;
  k_rerank_q8<<<n_ids, 64, 0, g.stream>>>((float*)ma->buf, mw->buf, mw->qp, la, lb, lp, ls, pen, li, lv, K, n_penalty,
                                          repeat_penalty, mw->group_size, ma->n_elems, mw->n_elems);
  count_launch();
  return check_launch();
}

}  // extern "C"
