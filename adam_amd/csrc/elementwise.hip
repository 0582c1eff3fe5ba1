// Element-wise ops over loc lists, reductions, argmax, embedding-row fetch, and the host-locs
// variants of the op surface.
//
// Reference kernels: shaders/src/f32/map_op1.comp, map_op2.comp:11-46 (0 ADD ... 34 GEGLU,
// 35 SWIGLU), map_broadcast.comp, map_fma.comp, map_reduce.comp, map_layernorm.comp,
// map_argmax.comp, map_row_gather_xq8.comp; dispatchers adamah.c:5837-6410, 6875-6973,
// 7384-7518, 8086-8178, 10189-10240.  Every op takes one uint32 loc per element (pack index).
#include "common.h"
#include "../../include/adamah_hip.h"

namespace adamah {

#define NEG_FLT_MAX (-3.402823466e+38f)

__device__ __forceinline__ float gelu_tanh(float a) {
  return 0.5f * a * (1.0f + tanhf(0.797884583f * (a + 0.0447149985f * a * a * a)));
}

__device__ float apply_op1(uint32_t op, float v) {
  switch (op) {
    case 0: return -v;
    case 1: return fabsf(v);
    case 2: return sqrtf(fmaxf(v, 0.0f));
    case 3: return expf(v);
    case 4: return logf(fmaxf(v, 1e-7f));
    case 5: return tanhf(v);
    case 6: return fmaxf(0.0f, v);
    case 7: return gelu_tanh(v);
    case 8: return sinf(v);
    case 9: return cosf(v);
    case 10: return tanf(v);
    case 11: return asinf(fminf(fmaxf(v, -1.0f), 1.0f));
    case 12: return acosf(fminf(fmaxf(v, -1.0f), 1.0f));
    case 13: return atanf(v);
    case 14: return sinhf(v);
    case 15: return coshf(v);
    case 16: return 1.0f / (1.0f + expf(-v));
    case 17: return v / (1.0f + expf(-v));
    case 18: return v * tanhf(logf(1.0f + expf(v)));
    case 19: return (v > 0.0f ? v : 1.67325997f * (expf(v) - 1.0f)) * 1.05069995f;
    case 20: return v > 0.0f ? v : expf(v) - 1.0f;
    case 21: return fmaxf(v, 0.01f * v);
    case 22: return ceilf(v);
    case 23: return floorf(v);
    case 24: return rintf(v);
    case 25: return v > 0.0f ? 1.0f : (v < 0.0f ? -1.0f : 0.0f);
    case 26: return 1.0f / v;
    case 27: return v * v;
    case 28: return v * v * v;
    case 29: return logf(1.0f + expf(v));
    case 30: return fminf(fmaxf(0.2f * v + 0.5f, 0.0f), 1.0f);
    case 31: return v * fminf(fmaxf(0.2f * v + 0.5f, 0.0f), 1.0f);
    case 32: return expf(v) - 1.0f;
    case 33: return logf(1.0f + v);
    default: return v;
  }
}

__device__ float apply_op2(uint32_t op, float a, float b) {
  switch (op) {
    case 0: return a + b;
    case 1: return a - b;
    case 2: return a * b;
    case 3: return a / b;
    case 4: return powf(a, b);
    case 5: return fminf(a, b);
    case 6: return fmaxf(a, b);
    case 7: return a - b * floorf(a / b);
    case 8: return a == b ? 1.0f : 0.0f;
    case 9: return a != b ? 1.0f : 0.0f;
    case 10: return a < b ? 1.0f : 0.0f;
    case 11: return a <= b ? 1.0f : 0.0f;
    case 12: return a > b ? 1.0f : 0.0f;
    case 13: return a >= b ? 1.0f : 0.0f;
    case 14: return (a != 0.0f && b != 0.0f) ? 1.0f : 0.0f;
    case 15: return (a != 0.0f || b != 0.0f) ? 1.0f : 0.0f;
    case 16: return ((a != 0.0f) != (b != 0.0f)) ? 1.0f : 0.0f;
    case 17: return atan2f(a, b);
    case 18: return b < a ? 0.0f : 1.0f;
    case 19: { float t = fminf(fmaxf((0.5f - a) / (b - a), 0.0f), 1.0f); return t * t * (3.0f - 2.0f * t); }
    case 34: return gelu_tanh(a) * b;
    case 35: return (a / (1.0f + expf(-a))) * b;
    default: return a;
  }
}

__global__ void __launch_bounds__(256)
k_op1(float* data, uint32_t op, const uint32_t* __restrict__ ls, const uint32_t* __restrict__ ld, uint64_t n,
      uint32_t pack, uint64_t n_elems) {
  const uint64_t tid = (uint64_t)blockIdx.x * 256u + threadIdx.x;
  if (tid >= n * pack) return;
  const uint64_t li = tid / pack, ei = tid % pack;
  const uint64_t s = (uint64_t)ls[li] * pack + ei, d = (uint64_t)ld[li] * pack + ei;
  if (s < n_elems && d < n_elems) data[d] = apply_op1(op, data[s]);
}
__global__ void __launch_bounds__(256)
k_op2(float* data, uint32_t op, const uint32_t* __restrict__ la, const uint32_t* __restrict__ lb,
      const uint32_t* __restrict__ ld, uint64_t n, uint32_t pack, uint64_t n_elems) {
  const uint64_t tid = (uint64_t)blockIdx.x * 256u + threadIdx.x;
  if (tid >= n * pack) return;
  const uint64_t li = tid / pack, ei = tid % pack;
  const uint64_t a = (uint64_t)la[li] * pack + ei, b = (uint64_t)lb[li] * pack + ei, d = (uint64_t)ld[li] * pack + ei;
  if (a < n_elems && b < n_elems && d < n_elems) data[d] = apply_op2(op, data[a], data[b]);
}
// op: 0 mul, 1 div, 2 add, 3 sub; scalar loc is an element index (not scaled by pack)
__global__ void __launch_bounds__(256)
k_broadcast(float* data, uint32_t op, const uint32_t* __restrict__ ls, const uint32_t* __restrict__ lk,
            const uint32_t* __restrict__ ld, uint64_t n, uint32_t pack, uint64_t n_elems) {
  const uint64_t tid = (uint64_t)blockIdx.x * 256u + threadIdx.x;
  if (tid >= n * pack) return;
  const uint64_t li = tid / pack, ei = tid % pack;
  const uint64_t s = (uint64_t)ls[li] * pack + ei, k = lk[li], d = (uint64_t)ld[li] * pack + ei;
  if (s >= n_elems || k >= n_elems || d >= n_elems) return;
  const float v = data[s], c = data[k];
  data[d] = op == 0 ? v * c : op == 1 ? v / c : op == 2 ? v + c : v - c;
}
__global__ void __launch_bounds__(256)
k_fma(float* data, const uint32_t* __restrict__ la, const uint32_t* __restrict__ lb, const uint32_t* __restrict__ lc,
      const uint32_t* __restrict__ ld, uint64_t n, uint32_t pack, uint64_t n_elems) {
  const uint64_t tid = (uint64_t)blockIdx.x * 256u + threadIdx.x;
  if (tid >= n * pack) return;
  const uint64_t li = tid / pack, ei = tid % pack;
  const uint64_t a = (uint64_t)la[li] * pack + ei, b = (uint64_t)lb[li] * pack + ei, c = (uint64_t)lc[li] * pack + ei,
                 d = (uint64_t)ld[li] * pack + ei;
  if (a < n_elems && b < n_elems && c < n_elems && d < n_elems) data[d] = __fadd_rn(__fmul_rn(data[a], data[b]), data[c]);
}

__device__ __forceinline__ float wred(float v, uint32_t op) {
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) {
    const float t = __shfl_xor(v, o, 64);
    v = op == 0 ? v + t : op == 1 ? fmaxf(v, t) : fminf(v, t);
  }
  return v;
}
// per loc: reduce the pack (0 sum, 1 max, 2 min) into locs_dst[li]
__global__ void __launch_bounds__(256)
k_reduce(float* data, uint32_t op, const uint32_t* __restrict__ ls, const uint32_t* __restrict__ ld, uint32_t pack,
         uint64_t n_elems) {
  __shared__ float sh[4];
  const uint32_t li = blockIdx.x, tid = threadIdx.x;
  const uint64_t base = (uint64_t)ls[li] * pack;
  float v = op == 0 ? 0.0f : op == 1 ? -1e38f : 1e38f;
  for (uint32_t i = tid; i < pack; i += 256u)
    if (base + i < n_elems) {
      const float x = data[base + i];
      v = op == 0 ? v + x : op == 1 ? fmaxf(v, x) : fminf(v, x);
    }
  v = wred(v, op);
  if ((tid & 63u) == 0) sh[tid >> 6] = v;
  __syncthreads();
  if (tid == 0) {
    float r = sh[0];
    for (int w = 1; w < 4; w++) r = op == 0 ? r + sh[w] : op == 1 ? fmaxf(r, sh[w]) : fminf(r, sh[w]);
    if (ld[li] < n_elems) data[ld[li]] = r;
  }
}

// src/dst row bases = loc*dim, gamma/beta bases absolute (map_layernorm.comp)
__global__ void __launch_bounds__(256)
k_layernorm(float* data, const uint32_t* __restrict__ ls, const uint32_t* __restrict__ ld, const uint32_t* __restrict__ lg,
            const uint32_t* __restrict__ lb, uint32_t dim, float eps, uint64_t n_elems) {
  __shared__ float sh[4];
  const uint32_t ri = blockIdx.x, tid = threadIdx.x;
  const uint64_t sb = (uint64_t)ls[ri] * dim, db = (uint64_t)ld[ri] * dim, gb = lg[ri], bb = lb[ri];
  if (sb + dim > n_elems || db + dim > n_elems || gb + dim > n_elems || bb + dim > n_elems) return;
  float s = 0.f;
  for (uint32_t i = tid; i < dim; i += 256u) s += data[sb + i];
  s = wred(s, 0);
  if ((tid & 63u) == 0) sh[tid >> 6] = s;
  __syncthreads();
  const float mean = ((sh[0] + sh[1]) + (sh[2] + sh[3])) / (float)dim;
  __syncthreads();
  float v = 0.f;
  for (uint32_t i = tid; i < dim; i += 256u) { const float d = data[sb + i] - mean; v = fmaf(d, d, v); }
  v = wred(v, 0);
  if ((tid & 63u) == 0) sh[tid >> 6] = v;
  __syncthreads();
  const float inv = 1.0f / sqrtf(((sh[0] + sh[1]) + (sh[2] + sh[3])) / (float)dim + eps);
  for (uint32_t i = tid; i < dim; i += 256u)
    data[db + i] = (data[sb + i] - mean) * inv * data[gb + i] + data[bb + i];
}

__device__ __forceinline__ bool better_am(float cv, uint32_t ci, float bv, uint32_t bi) {
  if (bi == 0xffffffffu) return true;
  if (ci == 0xffffffffu) return false;
  return (cv > bv) || ((cv == bv) && (ci < bi));
}
// argmax over n scalar locs; NaN -> -FLT_MAX; ties -> lower index; float(index) to locs_dst[0]
__global__ void __launch_bounds__(1024)
k_argmax(float* data, const uint32_t* __restrict__ ls, const uint32_t* __restrict__ ld, uint32_t n, uint64_t n_elems) {
  __shared__ float sv[1024];
  __shared__ uint32_t si[1024];
  const uint32_t tid = threadIdx.x;
  float bv = NEG_FLT_MAX; uint32_t bi = 0xffffffffu;
  for (uint32_t i = tid; i < n; i += 1024u) {
    float v = ls[i] < n_elems ? data[ls[i]] : NEG_FLT_MAX;
    if (isnan(v)) v = NEG_FLT_MAX;
    if (better_am(v, i, bv, bi)) { bv = v; bi = i; }
  }
  sv[tid] = bv; si[tid] = bi;
  __syncthreads();
  for (uint32_t s = 512; s > 0; s >>= 1) {
    if (tid < s && better_am(sv[tid + s], si[tid + s], sv[tid], si[tid])) { sv[tid] = sv[tid + s]; si[tid] = si[tid + s]; }
    __syncthreads();
  }
  if (tid == 0 && ld[0] < n_elems) data[ld[0]] = (float)(si[0] == 0xffffffffu ? 0u : si[0]);
}

// dst[e] = deq(src_base + row*row_size + e) * scale  (Q8 embedding row fetch)
__global__ void __launch_bounds__(256)
k_row_gather_q8(float* act, const uint8_t* __restrict__ W, const float2* __restrict__ qp, uint64_t src, uint64_t dst,
                uint32_t row_size, uint32_t group, float scale) {
  const uint32_t e = blockIdx.x * 256u + threadIdx.x;
  if (e >= row_size) return;
  const uint64_t i = src + e;
  const float2 p = qp[i / group];
  act[dst + e] = __fmul_rn(__fadd_rn(__fmul_rn((float)W[i], p.x), p.y), scale);
}

struct EwArgs { Map* m; const uint32_t* l[4]; };
static int ew_setup(uint32_t map_id, const uint32_t* handles, int nh, uint64_t n, EwArgs* out) {
  out->m = get_f32_map(map_id);
  if (!out->m) return ADAMAH_ERR_INVALID;
  for (int i = 0; i < nh; i++) {
    out->l[i] = n ? res_u32(handles[i], n) : nullptr;
    if (n && !out->l[i]) return ADAMAH_ERR_INVALID;
  }
  return ADAMAH_OK;
}

}  // namespace adamah

using namespace adamah;

extern "C" {

int map_op1_dev(uint32_t map_id, uint32_t op, uint32_t hs, uint32_t hd, uint32_t n) { ADAMAH_API();
  EwArgs a; uint32_t h[2] = {hs, hd};
  int r = ew_setup(map_id, h, 2, n, &a);
  if (r || n == 0) return r;
  k_op1<<<cdiv((uint64_t)n * a.m->pack_size, 256), 256, 0, g.stream>>>((float*)a.m->buf, op, a.l[0], a.l[1], n,
                                                                       a.m->pack_size, a.m->n_elems);
  count_launch();
  return check_launch();
}
int map_op2_dev(uint32_t map_id, uint32_t op, uint32_t ha, uint32_t hb, uint32_t hd, uint32_t n) {
  if ((op == 0 || op == 34 || op == 35) && n > 0 && can_defer()) {
    // ADD / GEGLU / SWIGLU over three contiguous ranges known on the host: queue it for fusion
    Map* m = get_f32_map(map_id);
    PendOp p;
    if (m && m->pack_size == 1 && res_run(ha, n, &p.a) && res_run(hb, n, &p.b) && res_run(hd, n, &p.c) &&
        in_range(p.a, n, m->n_elems) && in_range(p.b, n, m->n_elems) && in_range(p.c, n, m->n_elems)) {
      p.kind = PK_OP2; p.map_act = map_id; p.n = n; p.op = op;
      g.pend.push_back(p);
      return ADAMAH_OK;
    }
  }
  flush_pending();
  EwArgs a; uint32_t h[3] = {ha, hb, hd};
  int r = ew_setup(map_id, h, 3, n, &a);
  if (r || n == 0) return r;
  k_op2<<<cdiv((uint64_t)n * a.m->pack_size, 256), 256, 0, g.stream>>>((float*)a.m->buf, op, a.l[0], a.l[1], a.l[2], n,
                                                                       a.m->pack_size, a.m->n_elems);
  count_launch();
  return check_launch();
}
int map_broadcast_dev(uint32_t map_id, uint32_t op, uint32_t hs, uint32_t hk, uint32_t hd, uint32_t n) { ADAMAH_API();
  EwArgs a; uint32_t h[3] = {hs, hk, hd};
  int r = ew_setup(map_id, h, 3, n, &a);
  if (r || n == 0) return r;
  k_broadcast<<<cdiv((uint64_t)n * a.m->pack_size, 256), 256, 0, g.stream>>>((float*)a.m->buf, op, a.l[0], a.l[1],
                                                                             a.l[2], n, a.m->pack_size, a.m->n_elems);
  count_launch();
  return check_launch();
}
int map_fma_dev(uint32_t map_id, uint32_t ha, uint32_t hb, uint32_t hc, uint32_t hd, uint32_t n) { ADAMAH_API();
  EwArgs a; uint32_t h[4] = {ha, hb, hc, hd};
  int r = ew_setup(map_id, h, 4, n, &a);
  if (r || n == 0) return r;
  k_fma<<<cdiv((uint64_t)n * a.m->pack_size, 256), 256, 0, g.stream>>>((float*)a.m->buf, a.l[0], a.l[1], a.l[2], a.l[3],
                                                                       n, a.m->pack_size, a.m->n_elems);
  count_launch();
  return check_launch();
}
int map_reduce_dev(uint32_t map_id, uint32_t op, uint32_t hs, uint32_t hd, uint32_t n) { ADAMAH_API();
  EwArgs a; uint32_t h[2] = {hs, hd};
  int r = ew_setup(map_id, h, 2, n, &a);
  if (r || n == 0) return r;
  if (op > 2) return ADAMAH_ERR_INVALID;
  k_reduce<<<n, 256, 0, g.stream>>>((float*)a.m->buf, op, a.l[0], a.l[1], a.m->pack_size, a.m->n_elems);
  count_launch();
  return check_launch();
}
int map_layernorm_dev(uint32_t map_id, uint32_t hs, uint32_t hd, uint32_t hg, uint32_t hb, uint32_t n_rows,
                      uint32_t dim, float eps) { ADAMAH_API();
  EwArgs a; uint32_t h[4] = {hs, hd, hg, hb};
  int r = ew_setup(map_id, h, 4, n_rows, &a);
  if (r || n_rows == 0 || dim == 0) return r;
  k_layernorm<<<n_rows, 256, 0, g.stream>>>((float*)a.m->buf, a.l[0], a.l[1], a.l[2], a.l[3], dim, eps, a.m->n_elems);
  count_launch();
  return check_launch();
}
int map_argmax_dev(uint32_t map_id, uint32_t hs, uint32_t hd, uint32_t n) { ADAMAH_API();
  Map* m = get_f32_map(map_id);
  if (!m) return ADAMAH_ERR_INVALID;
  const uint32_t* ld = res_u32(hd, 1);
  const uint32_t* ls = n ? res_u32(hs, n) : ld;
  if (!ld || !ls) return ADAMAH_ERR_INVALID;
  k_argmax<<<1, 1024, 0, g.stream>>>((float*)m->buf, ls, ld, n, m->n_elems);
  count_launch();
  return check_launch();
}

int map_row_gather_xq8_dev(uint32_t map_act, uint32_t map_wt, uint32_t src_base, uint32_t dst_base, uint32_t row_idx,
                           uint32_t row_size, float scale) { ADAMAH_API();
  Map* ma = get_f32_map(map_act);
  Map* mw = get_map(map_wt);
  if (!ma || !mw || mw->dtype != DTYPE_Q8 || !mw->qp || mw->group_size == 0) return ADAMAH_ERR_INVALID;
  if (row_size == 0) return ADAMAH_OK;
  const uint64_t src = (uint64_t)src_base + (uint64_t)row_idx * row_size;
  if (!in_range(src, row_size, mw->n_elems) || !in_range(dst_base, row_size, ma->n_elems)) return ADAMAH_ERR_INVALID;
  k_row_gather_q8<<<cdiv(row_size, 256), 256, 0, g.stream>>>((float*)ma->buf, mw->buf, mw->qp, src, dst_base, row_size,
                                                             mw->group_size, scale);
  count_launch();
  return check_launch();
}

// ---- host-locs variants: copy the locs into library-owned handles, then run the handle op ----
#define UP(slot, ptr, n) scratch_handle(slot, ptr, (uint32_t)((n) * 4u))
int map_op1(uint32_t map_id, uint32_t op, const uint32_t* ls, const uint32_t* ld, uint32_t n) { ADAMAH_API();
  if (n == 0) return get_map(map_id) ? ADAMAH_OK : ADAMAH_ERR_INVALID;
  uint32_t a = UP(0, ls, n), b = UP(1, ld, n);
  if (!a || !b) return ADAMAH_ERR_INVALID;
  return map_op1_dev(map_id, op, a, b, n);
}
int map_op2(uint32_t map_id, uint32_t op, const uint32_t* la, const uint32_t* lb, const uint32_t* ld, uint32_t n) { ADAMAH_API();
  if (n == 0) return get_map(map_id) ? ADAMAH_OK : ADAMAH_ERR_INVALID;
  uint32_t a = UP(0, la, n), b = UP(1, lb, n), d = UP(2, ld, n);
  if (!a || !b || !d) return ADAMAH_ERR_INVALID;
  return map_op2_dev(map_id, op, a, b, d, n);
}
int map_broadcast(uint32_t map_id, uint32_t op, const uint32_t* ls, const uint32_t* lk, const uint32_t* ld, uint32_t n) { ADAMAH_API();
  if (n == 0) return get_map(map_id) ? ADAMAH_OK : ADAMAH_ERR_INVALID;
  uint32_t a = UP(0, ls, n), b = UP(1, lk, n), d = UP(2, ld, n);
  if (!a || !b || !d) return ADAMAH_ERR_INVALID;
  return map_broadcast_dev(map_id, op, a, b, d, n);
}
int map_reduce(uint32_t map_id, uint32_t op, const uint32_t* ls, const uint32_t* ld, uint32_t n) { ADAMAH_API();
  if (n == 0) return get_map(map_id) ? ADAMAH_OK : ADAMAH_ERR_INVALID;
  uint32_t a = UP(0, ls, n), b = UP(1, ld, n);
  if (!a || !b) return ADAMAH_ERR_INVALID;
  return map_reduce_dev(map_id, op, a, b, n);
}
int map_matmul(uint32_t map_id, const uint32_t* la, const uint32_t* lb, const uint32_t* lc, uint32_t M, uint32_t K,
               uint32_t N, uint32_t n_ops) { ADAMAH_API();
  if (n_ops == 0) return get_map(map_id) ? ADAMAH_OK : ADAMAH_ERR_INVALID;
  uint32_t a = UP(0, la, n_ops), b = UP(1, lb, n_ops), c = UP(2, lc, n_ops);
  if (!a || !b || !c) return ADAMAH_ERR_INVALID;
  return map_matmul_dev(map_id, a, b, c, M, K, N, n_ops);
}
int map_softmax(uint32_t map_id, const uint32_t* ls, const uint32_t* ld, uint32_t n_rows, uint32_t row_size) { ADAMAH_API();
  if (n_rows == 0) return get_map(map_id) ? ADAMAH_OK : ADAMAH_ERR_INVALID;
  uint32_t a = UP(0, ls, n_rows), b = UP(1, ld, n_rows);
  if (!a || !b) return ADAMAH_ERR_INVALID;
  return map_softmax_dev(map_id, a, b, n_rows, row_size);
}
int map_layernorm(uint32_t map_id, const uint32_t* ls, const uint32_t* ld, const uint32_t* lg, const uint32_t* lb,
                  uint32_t n_rows, uint32_t dim, float eps) { ADAMAH_API();
  if (n_rows == 0) return get_map(map_id) ? ADAMAH_OK : ADAMAH_ERR_INVALID;
  uint32_t a = UP(0, ls, n_rows), b = UP(1, ld, n_rows), c = UP(2, lg, n_rows), d = UP(3, lb, n_rows);
  if (!a || !b || !c || !d) return ADAMAH_ERR_INVALID;
  return map_layernorm_dev(map_id, a, b, c, d, n_rows, dim, eps);
}
#undef UP

}  // extern "C"
