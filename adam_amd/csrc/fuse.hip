// Deferred row-wise ops and their fusion.
//
// The reference records the ops of a batch into one command buffer and lets its fusion scheduler
// merge neighbours (adamah.c:1629-1721 batch_begin/batch_end, :4670-4691 and :5653-5714 fusion
// enable/flush).  Here a HIP stream already gives the ordering, so only the ops that can be folded
// into a neighbouring kernel are held back: single-row RMSNorm (+ residual), the M = 1 Q4 GEMV and
// GEMV + argmax, and ADD / GEGLU / SWIGLU over contiguous ranges.  They are queued with their operand
// offsets resolved on the host; when the batch ends, on adamah_fusion_flush, or as soon as any other
// entry point is called, the queue is launched in order with these folds applied:
//
//   RMSNorm(x -> n); GEMV(n -> y)                         -> GEMV that normalises while staging n
//   RMSNorm+residual(o, r -> r); RMSNorm(r -> n); GEMV(n)  -> GEMV that does both norms while staging
//   GEMV(-> y); ADD(r, y -> d)                            -> GEMV that also stores r + y
//   GEMV(-> [g; u]); GEGLU/SWIGLU(g, u -> t)              -> GEMV over paired rows that also stores t
//   GEMV(x, W1 -> y1); GEMV(x, W2 -> y2), W2 after W1, y2 after y1 -> one GEMV over the stacked rows
//   (scores; softmax . V) of tokens t, t+1, ... over one cache      -> one causal launch (attn_prefill.hip)
//   RoPE(q); RoPE(k) | QK-norm+RoPE; row copy (KV append)  -> one launch of row tasks (rowprep.hip), or, directly
//                                                             before one token's decode attention, done by that launch
//
// Every folded op still stores its own result where it would have stored it alone, so the contents
// of the maps after a batch do not depend on whether anything was folded.
#include "gemv_common.h"
#include "attn_common.h"
#include <stdlib.h>

namespace adamah {

bool can_defer() {
  return g.batch_depth > 0 && g.no_defer == 0 && tuning("ADAMAH_NO_FUSE", 0) == 0;
}

bool res_scalar(uint32_t h, uint32_t* out) {
  const uint32_t* p = res_host(h, 1);
  if (!p) return false;
  *out = p[0];
  return true;
}

bool res_run(uint32_t h, uint64_t n, uint32_t* start) {
  Res* r = get_res(h);
  if (!r || !r->host_valid || !r->contig || n * 4 > r->size_bytes || n == 0) return false;
  *start = ((const uint32_t*)r->host.data())[0];
  return true;
}

// ---- stand-alone kernels with operands passed by value -------------------------------------------
__global__ void __launch_bounds__(1024)
k_rmsnorm_v(const float* act, const float* wt, float* out, uint32_t src, uint32_t w, uint32_t res, uint32_t dst,
            uint32_t dim, float eps, int add) {
  __shared__ float sh[16];
  const uint32_t tid = threadIdx.x, lane = tid & 63u, wave = tid >> 6;
  float ss = 0.f;
  for (uint32_t i = tid; i < dim; i += 1024u) { const float x = act[(uint64_t)src + i]; ss = fmaf(x, x, ss); }
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) ss += __shfl_xor(ss, o, 64);
  if (lane == 0) sh[wave] = ss;
  __syncthreads();
  ss = 0.f;
#pragma unroll
  for (int i = 0; i < 16; i++) ss += sh[i];
  const float inv = 1.0f / sqrtf(ss / (float)dim + eps);
  for (uint32_t i = tid; i < dim; i += 1024u) {
    float y = act[(uint64_t)src + i] * inv * wt[(uint64_t)w + i];
    if (add) y += act[(uint64_t)res + i];
    out[(uint64_t)dst + i] = y;
  }
}

__global__ void __launch_bounds__(256)
k_op2_v(float* data, uint32_t op, uint32_t a, uint32_t b, uint32_t d, uint32_t n) {
  const uint32_t i = blockIdx.x * 256u + threadIdx.x;
  if (i >= n) return;
  const float x = data[(uint64_t)a + i], y = data[(uint64_t)b + i];
  float r;
  if (op == 0) r = x + y;
  else if (op == 34) r = gelu_tanh(x) * y;
  else r = (x / (1.0f + expf(-x))) * y;
  data[(uint64_t)d + i] = r;
}

int launch_rmsnorm_v(const PendOp& p) {
  Map* ma = get_f32_map(p.map_act);
  Map* mw = get_f32_map(p.map_wt);
  if (!ma || !mw) return ADAMAH_ERR_INVALID;
  float* a = (float*)ma->buf;
  k_rmsnorm_v<<<1, 1024, 0, g.stream>>>(a, (const float*)mw->buf, a, p.a, p.b, p.d, p.c, p.n, p.eps, (int)p.op);
  count_launch();
  return check_launch();
}

int launch_op2_v(const PendOp& p) {
  Map* ma = get_f32_map(p.map_act);
  if (!ma) return ADAMAH_ERR_INVALID;
  k_op2_v<<<cdiv(p.n, 256), 256, 0, g.stream>>>((float*)ma->buf, p.op, p.a, p.b, p.c, p.n);
  count_launch();
  return check_launch();
}

static bool disjoint(uint64_t a, uint64_t na, uint64_t b, uint64_t nb) { return a + na <= b || b + nb <= a; }

// A prologue fold makes every workgroup of the GEMV read the norm's inputs (and workgroup 0 / the last ticket
// store the norm's own results) while other workgroups already store result rows: whatever the GEMV writes --
// its result rows, or the partial (index, value) lists and the token slot of a GEMV + argmax -- has to lie
// clear of all of them, or the ops are launched one by one.
static bool gemv_writes_clear(const PendOp& gp, const uint64_t (*rg)[2], int n_rg) {
  auto clear_of_all = [&](uint64_t lo, uint64_t len) {
    for (int r = 0; r < n_rg; r++)
      if (!disjoint(lo, len, rg[r][0], rg[r][1])) return false;
    return true;
  };
  if (gp.kind == PK_GEMV) return clear_of_all(gp.c, gp.n);
  const uint32_t n_groups = cdiv(gp.n, gp.rpg);
  const uint32_t *idx = res_host(gp.h[0], n_groups), *val = res_host(gp.h[1], n_groups), *dst = res_host(gp.h[2], 1);
  if (!idx || !val || !dst) return false;   // locations only known on the device: cannot be checked here
  for (uint32_t i = 0; i < n_groups; i++)
    if (!clear_of_all(idx[i], 1) || !clear_of_all(val[i], 1)) return false;
  return clear_of_all(dst[0], 1);
}

// May the queued op read or write elements [lo, lo + n) of activation map `map`?  Conservative: true whenever its
// operands are not known on the host.
static bool op_touches(const PendOp& p, uint32_t map, uint64_t lo, uint64_t n) {
  if (p.map_act != map && p.map_wt != map) return false;
  auto hit = [&](uint64_t a, uint64_t len) { return !disjoint(a, len, lo, n); };
  auto rows = [&](uint32_t handle, uint32_t count, uint64_t len, bool* known) {
    const uint32_t* h = res_host(handle, count);
    if (!h) { *known = false; return true; }
    for (uint32_t i = 0; i < count; i++) if (hit(h[i], len)) return true;
    return false;
  };
  bool known = true;
  switch (p.kind) {
    case PK_RMSNORM:
      return (p.map_act == map && (hit(p.a, p.n) || hit(p.c, p.n) || (p.op == 1 && hit(p.d, p.n)))) || (p.map_wt == map && hit(p.b, p.n));
    case PK_GEMV:
      return p.map_act == map && (hit(p.a, p.k) || hit(p.c, p.n));
    case PK_OP2:
      return p.map_act == map && (hit(p.a, p.n) || hit(p.b, p.n) || hit(p.c, p.n));
    case PK_SCORES:
      return rows(p.h[0], p.rpg, p.k, &known) || rows(p.h[1], p.rpg, (uint64_t)p.n * p.k, &known) || rows(p.h[2], p.rpg, p.n, &known);
    case PK_ATTN:
      return rows(p.h[0], p.rpg, p.n, &known) || rows(p.h[1], p.rpg, (uint64_t)p.n * p.k, &known) || rows(p.h[2], p.rpg, p.k, &known);
    case PK_ROPE: case PK_QKNR: case PK_ROWCOPY: {
      std::vector<std::pair<uint64_t, uint64_t>> rg;
      if (!row_op_ranges(p, &rg)) return true;
      for (const auto& r : rg) if (hit(r.first, r.second)) return true;
      return false;
    }
    default: return true;
  }
}

// In-place t of a folded norm + residual pair (PRO_NORM2): the first later GEMV of the queue, from `from` on, that
// can put the parked row in place, i.e. a plain store GEMV such that neither it, nor the ops that may share its
// launch, nor anything queued before it touches the row.  n: none.
static size_t find_unparker(const std::vector<PendOp>& q, size_t from, uint32_t map, uint64_t lo, uint64_t len) {
  const size_t n = q.size();
  for (size_t j = from; j < n; j++) {
    if (op_touches(q[j], map, lo, len)) return n;
    if (q[j].kind != PK_GEMV || q[j].map_act != map) continue;
    // what may ride on the same launch: GEMVs stacked behind it, one element-wise op after them
    size_t e = j + 1;
    while (e < n && q[e].kind == PK_GEMV) { if (op_touches(q[e], map, lo, len)) return n; e++; }
    if (e < n && q[e].kind == PK_OP2 && op_touches(q[e], map, lo, len)) return n;
    return j;
  }
  return n;
}

__global__ void __launch_bounds__(256) k_copy_f32(float* data, const float* src, uint32_t dst, uint32_t n) {
  const uint32_t i = blockIdx.x * 256u + threadIdx.x;
  if (i < n) data[(uint64_t)dst + i] = src[i];
}

static int launch_gemv(const PendOp& gp, const GemvFuse* fz) {
  Map* ma = get_f32_map(gp.map_act);
  Map* mw = get_map(gp.map_wt);
  if (!ma || !mw) return ADAMAH_ERR_INVALID;
  if (gp.kind == PK_GEMV) return launch_mfma_store((int)gp.op, ma, mw, gp.a, gp.b, gp.c, gp.k, gp.n, fz);
  const uint32_t n_groups = cdiv(gp.n, gp.rpg);
  const uint32_t *lidx = res_u32(gp.h[0], n_groups), *lval = res_u32(gp.h[1], n_groups), *ldst = res_u32(gp.h[2], 1);
  if (!lidx || !lval || !ldst) return ADAMAH_ERR_INVALID;
  int r = launch_mfma_argmax((int)gp.op, ma, mw, gp.a, gp.b, lidx, lval, gp.k, gp.n, gp.rpg, fz);
  if (r) return r;
  return launch_argmax_pairs(ma, lidx, lval, ldst, n_groups);
}

// Prologue folds need the whole activation row in the registers of one workgroup.
static bool row_fits(const PendOp& gp) {
  const uint32_t threads = gp.kind == PK_GEMV ? mfma_store_threads(gp.k, gp.n) : 256u;
  return gp.k <= 8u * PRO_WPT * threads;
}

void flush_pending() {
  if (g.pend.empty()) return;
  std::vector<PendOp> q;
  q.swap(g.pend);   // launches below must not see a non-empty queue
  const size_t n = q.size();
  size_t i = 0;
  // the queued ops have returned ADAMAH_OK already: the first launch that fails is kept for the next call
  auto keep = [](int rc) { if (rc != ADAMAH_OK && !g.deferred_err) g.deferred_err = rc; };
  // a row parked by a PRO_NORM2 launch, and the queue index of the GEMV that will put it in place
  struct { bool active; size_t at; uint32_t map, dst, len; } park = {false, 0, 0, 0, 0};
  auto unpark_now = [&]() {   // not taken by the launch it was meant for: a copy of its own
    if (!park.active) return;
    park.active = false;
    Map* m = get_f32_map(park.map);
    if (!m) { keep(ADAMAH_ERR_INVALID); return; }
    k_copy_f32<<<cdiv(park.len, 256), 256, 0, g.stream>>>((float*)m->buf, g.t_park, park.dst, park.len);
    count_launch();
    keep(check_launch());
  };
  while (i < n) {
    if (park.active && i > park.at) unpark_now();
    if ((q[i].kind == PK_ROPE || q[i].kind == PK_ROWCOPY) && q[i].op == 1u) {   // one token of many sequences
      int rc = 0;
      i += launch_wide_rows(q, i, &rc);
      keep(rc);
      continue;
    }
    RowPrepCtx prep = {&q, i, {}};
    bool have_prep = false;
    if (q[i].kind == PK_ROPE || q[i].kind == PK_QKNR || q[i].kind == PK_ROWCOPY) {
      // Rotation of the new Q / K rows and the KV append.  When the run is followed directly by the decode attention
      // of one token, it is offered to that launch, which does the preparation of its own operands itself;
      // otherwise: one launch for the run.
      bool alone = false;
      const size_t used = build_row_run(q, i, &prep.tasks, &alone);
      const size_t s = i + used;
      if (used && !alone && s + 1 < n && q[s].map_act == q[i].map_act && attn_foldable(q[s], q[s + 1]) &&
          !(s + 2 < n && q[s + 2].kind == PK_SCORES)) {
        have_prep = true;
        i = s;
      } else {
        int rc = 0;
        i += launch_row_run(q, i, &rc);
        keep(rc);
        continue;
      }
    }
    const PendOp& p = q[i];
    auto is_gemv = [&](size_t j) {   // a launch of the int8 matrix-instruction kernel (Q8 argmax ops are not)
      return j < n && (q[j].kind == PK_GEMV || (q[j].kind == PK_ARGMAX && q[j].op != (uint32_t)FMT_Q8_B16));
    };
    size_t gi = n;    // the GEMV this group is built around, if any
    GemvFuse fz = {};
    if (p.kind == PK_GEMM) {
      // Matmuls over the same few rows whose weight matrices lie back to back: one launch over the stacked
      // rows, every result where its own op puts it.  All of them read the rows as they were before the
      // first, so no result may touch the rows (or another result).
      Map* ma = get_f32_map(p.map_act);
      Map* mw = get_map(p.map_wt);
      const uint64_t M = p.rpg, an = M * p.k;
      GemmSegs sg = {};
      sg.count = 1; sg.begin[0] = 0; sg.begin[1] = p.n; sg.n[0] = p.n; sg.c[0] = p.c;
      size_t m = 1;
      uint64_t next_b = (uint64_t)p.b + (uint64_t)p.n * p.k;
      bool clear = disjoint(p.c, M * p.n, p.a, an);
      while (clear && i + m < n && m < 4) {
        const PendOp& x = q[i + m];
        if (x.kind != PK_GEMM || x.map_act != p.map_act || x.map_wt != p.map_wt || x.a != p.a || x.rpg != p.rpg || x.k != p.k ||
            x.op != p.op || (uint64_t)x.b != next_b || (uint64_t)sg.begin[m] + x.n > 0xFFFFFFFFull)
          break;
        bool ok = disjoint(x.c, M * x.n, p.a, an);
        for (size_t j = 0; ok && j < m; j++) ok = disjoint(x.c, M * x.n, sg.c[j], M * sg.n[j]);
        if (!ok) break;
        sg.n[m] = x.n; sg.c[m] = x.c; sg.begin[m + 1] = sg.begin[m] + x.n;
        next_b += (uint64_t)x.n * x.k;
        m++;
      }
      sg.count = (uint32_t)m;
      // one matrix followed by the add that consumes its result (hidden += projection): stored by the matmul.
      // The matmul reads its fp16 copy of the rows, so only the result and the residual have to lie clear.
      size_t used = m;
      // (many rows: only where the matmul runs over shares of K, whose adding launch stores the add as well)
      if (m == 1 && (M <= 32 || (p.op != (uint32_t)FMT_Q8_B16 && gemm_q4_k_shares((uint32_t)M, p.k, p.n) > 1)) && i + 1 < n &&
          q[i + 1].kind == PK_OP2 && q[i + 1].op == 0 && q[i + 1].map_act == p.map_act &&
          q[i + 1].n == M * p.n && tuning("ADAMAH_GEMM_EPI", 1) != 0) {
        const PendOp& e = q[i + 1];
        if ((e.a == p.c) != (e.b == p.c)) {
          const uint32_t r = e.a == p.c ? e.b : e.a;
          if (disjoint(e.c, e.n, p.c, e.n) && (r == e.c || disjoint(r, e.n, e.c, e.n)) && disjoint(r, e.n, p.c, e.n)) {
            sg.count = 0; sg.add = 1; sg.res = r; sg.dst = e.c;
            used = 2;
          }
        }
      }
      // gate and up stacked, followed by the gated activation over their two results: stored by the matmul as well
      // (a workgroup then takes 16 gate rows and their 16 up rows).  The activation must not land on either result.
      if (m == 2 && M <= 32 && sg.n[0] == sg.n[1] && (sg.n[0] & 15u) == 0 && i + 2 < n && q[i + 2].kind == PK_OP2 &&
          (q[i + 2].op == 34u || q[i + 2].op == 35u) && q[i + 2].map_act == p.map_act && tuning("ADAMAH_GEMM_EPI", 1) != 0) {
        const PendOp& e = q[i + 2];
        if (e.a == sg.c[0] && e.b == sg.c[1] && e.n == M * sg.n[0] && disjoint(e.c, e.n, sg.c[0], e.n) &&
            disjoint(e.c, e.n, sg.c[1], e.n)) {
          sg.glu = e.op; sg.dst = e.c;
          used = 3;
        }
      }
      const uint32_t *la = res_u32(p.h[0], 1), *lb = res_u32(p.h[1], 1), *lc = res_u32(p.h[2], 1);
      if (!(ma && mw && la && lb && lc)) keep(ADAMAH_ERR_INVALID);
      else
        keep(launch_gemm_q4_mfma(ma, mw, la, lb, lc, p.rpg, p.k, sg.begin[m], 1, p.op == (uint32_t)FMT_Q8_B16, nullptr, (int64_t)p.a,
                                 (m == 1 && !sg.add) ? (int64_t)p.c : -1, (m == 1 && !sg.add) ? nullptr : &sg, (int64_t)p.b));
      i += used;
      continue;
    }
    if (p.kind == PK_OP2 && (p.op == 34u || p.op == 35u) && i + 1 < n && q[i + 1].kind == PK_GEMM) {
      // gated activation over the rows a batched matmul reads next: the op's launch also leaves the fp16 form of
      // its result, and the matmul skips its conversion launch
      const PendOp& mm = q[i + 1];
      Map* ma = get_f32_map(p.map_act);
      if (ma && mm.map_act == p.map_act && mm.a == p.c && (uint64_t)mm.rpg * mm.k == p.n && disjoint(p.c, p.n, p.a, p.n) &&
          disjoint(p.c, p.n, p.b, p.n) && tuning("ADAMAH_GLU_EMIT", 1) != 0 &&
          launch_glu_act_f16(ma, p.op, p.a, p.b, p.c, mm.rpg, mm.k)) {
        keep(check_launch());
        i++;
        continue;
      }
    }
    if (p.kind == PK_ARGMAX) {
      // the LM head of several sequences in lockstep: one pass over the matrix for all their rows
      int rc = 0;
      const size_t used = launch_argmax_run(q, i, &rc);
      keep(rc);
      if (used) { i += used; continue; }
      if (p.op == (uint32_t)FMT_Q8_B16) { keep(launch_argmax_direct(p)); i++; continue; }
    }
    if (p.kind == PK_SCORES && !have_prep) {
      // a prefill chunk: the attention of consecutive tokens over one growing cache, one launch
      int rc = 0;
      size_t used = launch_attn_chunk(q, i, &rc);
      if (!used) used = launch_attn_batch(q, i, &rc);   // or one token of several sequences in lockstep
      keep(rc);
      if (used) { i += used; continue; }
    }
    if (p.kind == PK_SCORES || p.kind == PK_ATTN) {
      // decode attention: scores computed inside the softmax . V launch; the merge of the sequence
      // splits moves into the GEMV that consumes the heads' outputs when the partials are small
      const PendOp* sc = nullptr;
      size_t ai = i;
      if (p.kind == PK_SCORES) {
        if (i + 1 < n && attn_foldable(p, q[i + 1])) { sc = &p; ai = i + 1; }
        else { keep(launch_scores(p)); i++; continue; }
      }
      const PendOp& at = q[ai];
      bool fold = false;
      if (ai + 1 < n && q[ai + 1].kind == PK_GEMV && q[ai + 1].map_act == at.map_act) {
        const PendOp& gp = q[ai + 1];
        const uint32_t* oh = res_host(at.h[2], at.rpg);
        fold = oh && gp.a == oh[0] && gp.k == at.rpg * at.k && (at.k & 7u) == 0 && at.k <= 8184u && disjoint(gp.c, gp.n, gp.a, gp.k);
        for (uint32_t h = 1; fold && h < at.rpg; h++) fold = oh[h] == oh[0] + h * at.k;
        // a merging GEMV may also have to put the token's prepared queries in place (workgroup 0, while others
        // already store result rows): its results must lie clear of those rows
        if (fold && have_prep && !prep.tasks.empty()) fold = disjoint(gp.c, gp.n, prep.tasks[0].dst, (uint64_t)at.rpg * at.k);
      }
      AttnPartials ap = {nullptr, 1, 0, 0, 0, nullptr, 0, 0};
      keep(launch_attn(sc, at, fold, &ap, have_prep ? &prep : nullptr));
      if (fold && ap.n_splits > 1) {   // partials left for the GEMV to merge
        fz.pro = PRO_COMBINE; fz.c_partial = ap.base; fz.c_splits = ap.n_splits; fz.c_vd = at.k;
        fz.c_qsrc = ap.q_src; fz.c_qdst = ap.q_dst; fz.c_qn = ap.q_n;
        fz.p_dst = q[ai + 1].a;
        gi = ai + 1;
      }
      if (gi == n) { i = ai + 1; continue; }
    } else if (is_gemv(i)) gi = i;
    else if (p.kind == PK_RMSNORM && p.op == 1 && i + 2 < n && q[i + 1].kind == PK_RMSNORM && q[i + 1].op == 0 &&
             is_gemv(i + 2)) {
      // RMSNorm + residual (t), RMSNorm of t (x), GEMV of x
      const PendOp &m = q[i + 1], &gp = q[i + 2];
      Map *mw1 = get_f32_map(p.map_wt), *mw2 = get_f32_map(m.map_wt);
      const bool chain = m.map_act == p.map_act && gp.map_act == p.map_act && m.a == p.c && m.n == p.n &&
                         gp.a == m.c && gp.k == m.n;
      // t may overwrite the residual (ticket-protected) but nothing else that is read; x must not
      // overwrite any input
      bool safe = disjoint(p.c, p.n, p.a, p.n) && (p.c == p.d || disjoint(p.c, p.n, p.d, p.n)) &&
                  disjoint(m.c, m.n, p.a, p.n) && disjoint(m.c, m.n, p.d, p.n) && disjoint(m.c, m.n, p.c, p.n);
      // norm weights that live in the activation map: neither t nor x may land on them
      if (p.map_wt == p.map_act) safe = safe && disjoint(p.c, p.n, p.b, p.n) && disjoint(m.c, m.n, p.b, p.n);
      if (m.map_wt == p.map_act) safe = safe && disjoint(p.c, p.n, m.b, m.n) && disjoint(m.c, m.n, m.b, m.n);
      const uint64_t rd[4][2] = {{p.a, p.n}, {p.d, p.n}, {p.c, p.n}, {m.c, m.n}};   // src, residual, t, x
      if (chain && safe && mw1 && mw2 && (p.n & 31u) == 0 && row_fits(gp) && g.sync_ctr && gemv_writes_clear(gp, rd, 4)) {
        fz.pro = PRO_NORM2; fz.p_src = p.a; fz.p_src2 = p.b; fz.p_eps = p.eps; fz.p_wt = (const float*)mw1->buf;
        fz.p_res = p.d; fz.p_tdst = p.c; fz.p_w2 = m.b; fz.p_eps2 = m.eps; fz.p_wt2 = (const float*)mw2->buf;
        fz.p_dst = m.c; fz.counter = g.sync_ctr;
        fz.t_mode = p.c == p.d ? 0u : 1u;   // t clear of the residual (and, `safe`, of the source): stored at once
        gi = i + 2;
      }
    } else if (p.kind == PK_RMSNORM && p.op == 0 && is_gemv(i + 1)) {
      const PendOp& gp = q[i + 1];
      Map* mw = get_f32_map(p.map_wt);
      // the prologue reads its source in every workgroup while workgroup 0 stores its result
      const uint64_t rd[2][2] = {{p.a, p.n}, {p.c, p.n}};   // src, x
      if (gp.map_act == p.map_act && gp.a == p.c && gp.k == p.n && disjoint(p.a, p.n, p.c, p.n) && (p.n & 31u) == 0 &&
          mw && row_fits(gp) && gemv_writes_clear(gp, rd, 2)) {
        fz.pro = PRO_RMSNORM; fz.p_src = p.a; fz.p_src2 = p.b; fz.p_dst = p.c; fz.p_eps = p.eps;
        fz.p_wt = (const float*)mw->buf;
        gi = i + 1;
      }
    }
    if (gi == n) {   // nothing to fold: launch the op alone
      keep(p.kind == PK_RMSNORM ? launch_rmsnorm_v(p) : launch_op2_v(p));
      i++;
      continue;
    }
    // GEMVs over the same activation vector whose matrices and results lie back to back (Q, K, V or
    // gate, up issued one after the other): one launch over the stacked rows.  All of them read the
    // activations as they were before the first, so no result may overlap what the launch reads.
    PendOp gp = q[gi];
    const size_t gi0 = gi;   // queue index of the group's first GEMV
    if (gp.kind == PK_GEMV) {
      while (gi + 1 < n && q[gi + 1].kind == PK_GEMV) {
        const PendOp& nx = q[gi + 1];
        if (nx.map_act != gp.map_act || nx.map_wt != gp.map_wt || nx.a != gp.a || nx.k != gp.k || nx.op != gp.op ||
            (uint64_t)nx.b != (uint64_t)gp.b + (uint64_t)gp.n * gp.k || (uint64_t)nx.c != (uint64_t)gp.c + gp.n)
          break;
        const uint64_t nn = (uint64_t)gp.n + nx.n;
        bool clear = nn <= 0xFFFFFFFFull && disjoint(gp.c, nn, gp.a, gp.k);
        if (fz.pro == PRO_RMSNORM || fz.pro == PRO_NORM2) clear = clear && disjoint(gp.c, nn, fz.p_src, gp.k);
        if (fz.pro == PRO_NORM2) clear = clear && disjoint(gp.c, nn, fz.p_res, gp.k) && disjoint(gp.c, nn, fz.p_tdst, gp.k);
        if (fz.pro == PRO_COMBINE && fz.c_qn) clear = clear && disjoint(gp.c, nn, fz.c_qdst, fz.c_qn);
        if (!clear) break;
        gp.n = (uint32_t)nn;
        gi++;
      }
    }
    size_t last = gi;
    if (gp.kind == PK_GEMV && gi + 1 < n && q[gi + 1].kind == PK_OP2 && q[gi + 1].map_act == gp.map_act) {
      const PendOp& e = q[gi + 1];
      // Result rows are stored while other workgroups still read the kernel's inputs: the epilogue's
      // destination must not touch any of them, nor the GEMV result.
      bool clear = disjoint(e.c, e.n, gp.c, gp.n) && disjoint(e.c, e.n, gp.a, gp.k);
      if (fz.pro) clear = clear && disjoint(e.c, e.n, fz.p_src, gp.k);
      if (fz.pro == PRO_NORM2) clear = clear && disjoint(e.c, e.n, fz.p_res, gp.k) && disjoint(e.c, e.n, fz.p_tdst, gp.k);
      // the prepared queries workgroup 0 puts in place: neither written nor read (a residual) by the epilogue
      if (fz.pro == PRO_COMBINE && fz.c_qn)
        clear = clear && disjoint(e.c, e.n, fz.c_qdst, fz.c_qn) && disjoint(e.a, e.n, fz.c_qdst, fz.c_qn) && disjoint(e.b, e.n, fz.c_qdst, fz.c_qn);
      if (e.op == 0 && e.n == gp.n && (e.a == gp.c) != (e.b == gp.c)) {
        const uint32_t r = e.a == gp.c ? e.b : e.a;   // the residual may be updated in place
        bool ok = clear && (r == e.c || disjoint(r, e.n, e.c, e.n));
        if (fz.pro == PRO_NORM2) ok = ok && disjoint(r, e.n, fz.p_tdst, gp.k);
        if (ok) { fz.e_mode = EPIX_ADD; fz.e_res = r; fz.e_dst = e.c; last = gi + 1; }
      } else if ((e.op == 34 || e.op == 35) && gp.n == 2u * e.n && (e.n & 1u) == 0 && e.a == gp.c && e.b == gp.c + e.n &&
                 clear) {
        // gate rows then up rows in one matrix, activation over the two halves of its result
        fz.e_mode = e.op == 34 ? EPIX_GEGLU : EPIX_SWIGLU; fz.e_dst = e.c;
        last = gi + 1;
      }
    }
    if (park.active && park.at <= last) {
      if (park.at == gi0 && gp.kind == PK_GEMV) { fz.d_src = g.t_park; fz.d_dst = park.dst; fz.d_n = park.len; park.active = false; }
      else unpark_now();
    }
    if (fz.pro == PRO_NORM2 && fz.t_mode == 0u && !park.active && g.t_park && gp.k <= T_PARK_FLOATS &&
        tuning("ADAMAH_NORM2_PARK", 1) != 0) {
      const size_t at = find_unparker(q, last + 1, gp.map_act, fz.p_tdst, gp.k);
      if (at < n) { fz.t_mode = 2u; fz.t_park = g.t_park; park = {true, at, gp.map_act, fz.p_tdst, gp.k}; }
    }
    keep(launch_gemv(gp, (fz.pro || fz.e_mode || fz.d_n) ? &fz : nullptr));
    i = last + 1;
  }
  unpark_now();
}

}  // namespace adamah
