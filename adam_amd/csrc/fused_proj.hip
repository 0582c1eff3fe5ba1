// Single-call forms of the projections that share one activation vector: Q/K/V, gate/up, and gate/up
// with SiLU(gate) * up applied.
//
// Reference: adamah.c:8809-8951 (map_fused_qkv_t_xq4_dev), :8953-9079 (gate/up, Q4), :9081-9351 (the Q8
// twins), :9353-9466 (map_fused_gateup_act_t_xq8_dev); shaders/src/f32/map_fused_qkv_t_xq4.comp,
// map_fused_gateup_t_xq4.comp, map_fused_gateup_act_t_xq8.comp:62-160.  Every handle holds one element
// offset; each projection is y = W x over its own [N, K] matrix.
//
// The projections are queued as ordinary M = 1 GEMVs (also outside a batch); when the queue is
// launched, GEMVs over the same activation vector whose matrices and results lie back to back become
// one launch, and the row-wise ops around them fold in as they do for a single GEMV.  Matrices that
// are not adjacent in the weight map cost one launch each.
#include "gemv_common.h"
#include "../../include/adamah_hip.h"

namespace adamah {

static int fused_projections(uint32_t dtype, uint32_t map_act, uint32_t map_wt, uint32_t ha, const uint32_t* hb,
                             const uint32_t* hc, const uint32_t* n, int cnt, uint32_t K) {
  Map* ma = get_map(map_act);
  Map* mw = get_map(map_wt);
  if (!ma || !mw) return ADAMAH_ERR_INVALID;
  uint32_t any = 0;
  for (int i = 0; i < cnt; i++) any |= n[i];
  if (!any) return ADAMAH_OK;
  if (!mw->qp || mw->group_size == 0) return ADAMAH_ERR_INVALID;
  if (!get_res(ha)) return ADAMAH_ERR_INVALID;
  for (int i = 0; i < cnt; i++)   // every handle has to exist, also of a projection with no rows
    if (!get_res(hb[i]) || !get_res(hc[i])) return ADAMAH_ERR_INVALID;
  g.batch_depth++;
  int r = ADAMAH_OK;
  for (int i = 0; i < cnt && r == ADAMAH_OK; i++)
    if (n[i]) r = op_matmul_t_xq(dtype, map_act, map_wt, ha, hb[i], hc[i], 1, K, n[i], 1, true);
  if (--g.batch_depth == 0) flush_pending();
  return r;
}

// out[row] = silu(x . Wg[row]) * (x . Wu[row]); one wave per row, affine dequantisation
template <bool Q4>
__global__ void __launch_bounds__(256)
k_gateup_act(float* act, const uint8_t* __restrict__ W, const float2* __restrict__ qp, const uint32_t* __restrict__ la,
             const uint32_t* __restrict__ lbg, const uint32_t* __restrict__ lbu, const uint32_t* __restrict__ lco,
             uint32_t K, uint32_t N, uint32_t group, uint64_t act_elems, uint64_t wt_elems) {
  const uint32_t lane = threadIdx.x & 63u, row = blockIdx.x * 4u + (threadIdx.x >> 6);
  if (row >= N) return;
  const uint64_t a = la[0], bg = (uint64_t)lbg[0] + (uint64_t)row * K, bu = (uint64_t)lbu[0] + (uint64_t)row * K;
  float sg = 0.f, su = 0.f;
  for (uint32_t k = lane; k < K; k += 64u) {
    if (a + k >= act_elems) continue;
    const float x = act[a + k];
    if (bg + k < wt_elems) sg = fmaf(x, deq_elem(W, qp, bg + k, group, Q4), sg);
    if (bu + k < wt_elems) su = fmaf(x, deq_elem(W, qp, bu + k, group, Q4), su);
  }
  sg = wave_sum(sg);
  su = wave_sum(su);
  const uint64_t c = (uint64_t)lco[0] + row;
  if (lane == 0 && c < act_elems) act[c] = (sg / (1.0f + expf(-sg))) * su;
}

}  // namespace adamah

using namespace adamah;

extern "C" {

int map_fused_qkv_t_xq4_dev(uint32_t ma, uint32_t mw, uint32_t a, uint32_t bq, uint32_t bk, uint32_t bv, uint32_t cq,
                            uint32_t ck, uint32_t cv, uint32_t K, uint32_t N_q, uint32_t N_k, uint32_t N_v) {
  const uint32_t hb[3] = {bq, bk, bv}, hc[3] = {cq, ck, cv}, n[3] = {N_q, N_k, N_v};
  return fused_projections(DTYPE_Q4, ma, mw, a, hb, hc, n, 3, K);
}
int map_fused_qkv_t_xq8_dev(uint32_t ma, uint32_t mw, uint32_t a, uint32_t bq, uint32_t bk, uint32_t bv, uint32_t cq,
                            uint32_t ck, uint32_t cv, uint32_t K, uint32_t N_q, uint32_t N_k, uint32_t N_v) {
  const uint32_t hb[3] = {bq, bk, bv}, hc[3] = {cq, ck, cv}, n[3] = {N_q, N_k, N_v};
  return fused_projections(DTYPE_Q8, ma, mw, a, hb, hc, n, 3, K);
}
int map_fused_gateup_t_xq4_dev(uint32_t ma, uint32_t mw, uint32_t a, uint32_t bg, uint32_t bu, uint32_t cg, uint32_t cu,
                               uint32_t K, uint32_t N_gate, uint32_t N_up) {
  const uint32_t hb[2] = {bg, bu}, hc[2] = {cg, cu}, n[2] = {N_gate, N_up};
  return fused_projections(DTYPE_Q4, ma, mw, a, hb, hc, n, 2, K);
}
int map_fused_gateup_t_xq8_dev(uint32_t ma, uint32_t mw, uint32_t a, uint32_t bg, uint32_t bu, uint32_t cg, uint32_t cu,
                               uint32_t K, uint32_t N_gate, uint32_t N_up) {
  const uint32_t hb[2] = {bg, bu}, hc[2] = {cg, cu}, n[2] = {N_gate, N_up};
  return fused_projections(DTYPE_Q8, ma, mw, a, hb, hc, n, 2, K);
}

int map_fused_gateup_act_t_xq8_dev(uint32_t map_act, uint32_t map_wt, uint32_t ha, uint32_t hbg, uint32_t hbu,
                                   uint32_t hco, uint32_t K, uint32_t N_ff) { ADAMAH_API();
  Map* ma = get_map(map_act);
  Map* mw = get_map(map_wt);
  if (!ma || !mw) return ADAMAH_ERR_INVALID;
  if (N_ff == 0) return ADAMAH_OK;
  if (ma->dtype != DTYPE_F32 || mw->dtype != DTYPE_Q8 || !mw->qp || mw->group_size == 0) return ADAMAH_ERR_INVALID;
  const uint32_t *la = res_u32(ha, 1), *lbg = res_u32(hbg, 1), *lbu = res_u32(hbu, 1), *lco = res_u32(hco, 1);
  if (!la || !lbg || !lbu || !lco) return ADAMAH_ERR_INVALID;
  const uint32_t *ah = res_host(ha, 1), *gh = res_host(hbg, 1), *uh = res_host(hbu, 1), *ch = res_host(hco, 1);
  if (ah && !in_range(ah[0], K, ma->n_elems)) return ADAMAH_ERR_INVALID;
  if (gh && !in_range(gh[0], (uint64_t)N_ff * K, mw->n_elems)) return ADAMAH_ERR_INVALID;
  if (uh && !in_range(uh[0], (uint64_t)N_ff * K, mw->n_elems)) return ADAMAH_ERR_INVALID;
  if (ch && !in_range(ch[0], N_ff, ma->n_elems)) return ADAMAH_ERR_INVALID;
  k_gateup_act<false><<<cdiv(N_ff, 4), 256, 0, g.stream>>>((float*)ma->buf, mw->buf, mw->qp, la, lbg, lbu, lco, K, N_ff,
                                                           mw->group_size, ma->n_elems, mw->n_elems);
  count_launch();
  return check_launch();
}

}  // extern "C"
