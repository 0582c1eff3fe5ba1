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
#include "../../include/adamah_hip.h"

namespace adamah {

#define TOPK_MAX 64u

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
                          uint32_t rows_per_group) {
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
  if (N > g_logit_cap) {
    if (g_logit_buf) { hipStreamSynchronize(g.stream); hipFree(g_logit_buf); }
    g_logit_cap = std::max<size_t>(N, 1u << 16);
    if (hipMalloc((void**)&g_logit_buf, g_logit_cap * sizeof(float)) != hipSuccess) {
      g_logit_buf = nullptr; g_logit_cap = 0;
      return ADAMAH_ERR_MEMORY;
    }
  }
  float* act = (float*)ma->buf;
  uint64_t a0 = 0, b0 = 0;
  int r;
  if (dtype == DTYPE_Q4 && block_path_ok(ma, mw, ha, hb, K, N, &a0, &b0) && mfma_path_ok(mw, K) &&
      tuning("ADAMAH_GEMV_IMPL", 3) == 3) {
    r = launch_mfma_store(fmt_of(mw, b0, (uint64_t)N * K), ma, mw, (uint32_t)a0, (uint32_t)b0, 0u, K, N, nullptr,
                          g_logit_buf);
  } else {
    if (dtype == DTYPE_Q4)
      k_matvec_rows<true><<<cdiv(N, 4), 256, 0, g.stream>>>(act, mw->buf, mw->qp, la, lb, g_logit_buf, K, N,
                                                            mw->group_size, ma->n_elems, mw->n_elems);
    else
      k_matvec_rows<false><<<cdiv(N, 4), 256, 0, g.stream>>>(act, mw->buf, mw->qp, la, lb, g_logit_buf, K, N,
                                                             mw->group_size, ma->n_elems, mw->n_elems);
    count_launch();
    r = check_launch();
  }
  if (r) return r;
  // counting costs rows^2 / 256 comparisons per thread, the rounds k * (rows / 256 + a reduction)
  const uint64_t rws = std::min(rows_per_group, N);
  const bool by_rank = rows_per_group <= RANK_MAX && rws * rws / 256u <= (uint64_t)k * (rws / 256u + 40u);
  if (tuning("ADAMAH_TOPK_RANK", by_rank ? 1 : 0) != 0 && rows_per_group <= RANK_MAX)
    k_group_topk_rank<<<n_groups, 256, 0, g.stream>>>(act, g_logit_buf, pen, lidx, lval, N, k, n_pen, rp,
                                                      rows_per_group, ma->n_elems);
  else
    k_group_topk<<<n_groups, 256, 0, g.stream>>>(act, g_logit_buf, pen, lidx, lval, N, k, n_pen, rp, rows_per_group,
                                                 ma->n_elems);
  count_launch();
  return check_launch();
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
