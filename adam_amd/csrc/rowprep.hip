// Row preparation before decode attention in one launch: RoPE of the new Q and K rows (with the
// per-head RMSNorm of map_qk_norm_rope_x when asked for) and the append of the new K and V rows to
// the KV cache.
//
// Reference kernels: shaders/src/f32/map_rope.comp:11-37, map_qk_norm_rope_x.comp:32-84,
// map_row_copy.comp:13-24 (dispatch adamah.c:7610-7878, 8061-8085).  The decode loop issues them back
// to back per layer (adam/models/engine.py: rope q, rope k or qk_norm_rope, then row_copy_offset of
// the K and V rows).  Inside a batch these ops are queued like the other row-wise ops; a run of them
// becomes a list of row tasks (source row, optional norm weights, optional rotation, destination
// row, optional cache row), passed to one kernel by value.  A copy whose source is exactly the
// destination of an earlier task of the run rides on that task, which then stores the row twice; any
// other overlap between a task and an earlier one ends the run, so tasks of one launch are
// independent.  The arithmetic and its order are those of the stand-alone kernels, so results do not
// depend on whether a run was merged.
#include "attn_common.h"
#include "../../include/adamah_hip.h"
#include <algorithm>

namespace adamah {

struct RowTasks { RowTask t[ROWT_MAX]; };

__device__ __forceinline__ void store_row_elem(float* act, __half* kv16, uint64_t kv_start, uint64_t kv_count,
                                               uint32_t dst, uint32_t cache, uint32_t i, float v) {
  if (dst != ROWT_NONE) act[(uint64_t)dst + i] = v;
  if (cache != ROWT_NONE) {
    const uint64_t dof = (uint64_t)cache + i;
    if (kv16 && dof >= kv_start && dof - kv_start < kv_count) {
      const __half h = __float2half(v);
      kv16[dof - kv_start] = h;
      v = __half2float(h);
    }
    act[dof] = v;
  }
}

// One 256-thread workgroup per task, as the stand-alone kernels have per row.
__global__ void __launch_bounds__(256)
k_row_tasks(float* act, const RowTasks ts, __half* kv16, uint64_t kv_start, uint64_t kv_count) {
  __shared__ float sh[4];
  const RowTask t = ts.t[blockIdx.x];
  const uint32_t tid = threadIdx.x, dim = t.dim, half = dim >> 1;
  float inv = 1.f;
  if (t.flags & 1u) {
    float ss = 0.f;
    for (uint32_t i = tid; i < dim; i += 256u) { const float x = act[(uint64_t)t.src + i]; ss = fmaf(x, x, ss); }
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) ss += __shfl_xor(ss, o, 64);
    if ((tid & 63u) == 0) sh[tid >> 6] = ss;
    __syncthreads();
    ss = (sh[0] + sh[1]) + (sh[2] + sh[3]);
    inv = 1.0f / sqrtf(ss / (float)dim + 1e-6f);
  }
  if (t.flags & 2u) {
    for (uint32_t i = tid; i < half; i += 256u) {
      float y0 = act[(uint64_t)t.src + i], y1 = act[(uint64_t)t.src + i + half];
      if (t.flags & 1u) {
        y0 = y0 * inv * act[(uint64_t)t.w + i];
        y1 = y1 * inv * act[(uint64_t)t.w + i + half];
      }
      float c, s;
      rope_cs2(i, dim, t.pos, t.base, &c, &s);
      store_row_elem(act, kv16, kv_start, kv_count, t.dst, t.cache, i, y0 * c - y1 * s);
      store_row_elem(act, kv16, kv_start, kv_count, t.dst, t.cache, i + half, y0 * s + y1 * c);
    }
  } else {
    for (uint32_t i = tid; i < dim; i += 256u) {
      float y = act[(uint64_t)t.src + i];
      if (t.flags & 1u) y = y * inv * act[(uint64_t)t.w + i];
      store_row_elem(act, kv16, kv_start, kv_count, t.dst, t.cache, i, y);
    }
  }
}

static bool overlap(uint32_t a, uint32_t na, uint32_t b, uint32_t nb) {
  if (a == ROWT_NONE || b == ROWT_NONE) return false;
  return !((uint64_t)a + na <= b || (uint64_t)b + nb <= a);
}

// Tasks of one queued op; false: operands not usable from the host (the caller launches it alone).
static bool expand(const PendOp& p, const Map* m, std::vector<RowTask>* out) {
  out->clear();
  if (p.kind == PK_ROPE) {
    for (uint32_t h = 0; h < p.rpg; h++)
      out->push_back({p.a + h * p.k, p.c + h * p.k, ROWT_NONE, ROWT_NONE, p.k, p.n, 2u, p.eps});
  } else if (p.kind == PK_QKNR) {
    const uint32_t q_rows = p.rpg, q_dim = p.k, k_rows = p.op, k_dim = p.d;
    const uint32_t *lqs = res_host(p.h[0], q_rows), *lqw = res_host(p.h[1], q_rows);
    const uint32_t *lks = res_host(p.h[2], k_rows), *lkw = res_host(p.h[3], k_rows), *ld = res_host(p.h[4], 1);
    if (!ld || (q_rows && (!lqs || !lqw)) || (k_rows && (!lks || !lkw))) return false;
    for (uint32_t r = 0; r < q_rows; r++)
      out->push_back({lqs[r], ld[0] + r * q_dim, ROWT_NONE, lqw[r], q_dim, p.n, 3u, p.eps});
    for (uint32_t r = 0; r < k_rows; r++)
      out->push_back({lks[r], ld[0] + q_rows * q_dim + r * k_dim, ROWT_NONE, lkw[r], k_dim, p.n, 3u, p.eps});
  } else if (p.kind == PK_ROWCOPY) {
    const uint32_t *spec = res_host(p.h[0], 2ull * p.rpg), *base = res_host(p.h[1], 1);
    if (!spec || !base) return false;
    for (uint32_t ci = 0; ci < p.rpg; ci++) {
      const uint64_t so = (uint64_t)base[0] + (uint64_t)spec[2 * ci] * p.k;
      const uint64_t dof = ((uint64_t)spec[2 * ci + 1] + p.n) * p.k;
      if (so > 0xFFFFFFF0ull || dof > 0xFFFFFFF0ull) return false;
      out->push_back({(uint32_t)so, ROWT_NONE, (uint32_t)dof, ROWT_NONE, p.k, 0u, 0u, 0.f});
    }
  } else {
    return false;
  }
  for (const RowTask& t : *out) {
    if (t.dim == 0 || ((t.flags & 2u) && (t.dim & 1u))) return false;
    if (!in_range(t.src, t.dim, m->n_elems)) return false;
    if (t.dst != ROWT_NONE && !in_range(t.dst, t.dim, m->n_elems)) return false;
    if (t.cache != ROWT_NONE && !in_range(t.cache, t.dim, m->n_elems)) return false;
    if (t.w != ROWT_NONE && !in_range(t.w, t.dim, m->n_elems)) return false;
  }
  return true;
}

bool row_op_deferrable(const PendOp& p) {
  Map* m = get_f32_map(p.map_act);
  std::vector<RowTask> ts;
  return m && expand(p, m, &ts) && !ts.empty() && ts.size() <= ROWT_MAX;
}

bool row_op_ranges(const PendOp& p, std::vector<std::pair<uint64_t, uint64_t>>* out) {
  Map* m = get_f32_map(p.map_act);
  std::vector<RowTask> ts;
  if (!m || !expand(p, m, &ts)) return false;
  for (const RowTask& t : ts) {
    out->push_back({t.src, t.dim});
    if (t.dst != ROWT_NONE) out->push_back({t.dst, t.dim});
    if (t.cache != ROWT_NONE) out->push_back({t.cache, t.dim});
    if (t.w != ROWT_NONE) out->push_back({t.w, t.dim});
  }
  return true;
}

static int launch_tasks(Map* m, const std::vector<RowTask>& run) {
  if (run.empty()) return ADAMAH_OK;
  RowTasks ts;
  for (size_t i = 0; i < run.size(); i++) ts.t[i] = run[i];
  k_row_tasks<<<(uint32_t)run.size(), 256, 0, g.stream>>>((float*)m->buf, ts, m->kv16, m->kv_start, m->kv_count);
  count_launch();
  return check_launch();
}

// The merged tasks of the run of row ops that starts at q[i]; returns how many queue entries the run covers.  0:
// the first op cannot be expanded on the host.  *alone: q[i] by itself does not fit one launch (run holds its tasks,
// which are independent of each other).
size_t build_row_run(const std::vector<PendOp>& q, size_t i, std::vector<RowTask>* out, bool* alone) {
  *alone = false;
  out->clear();
  Map* m = get_f32_map(q[i].map_act);
  if (!m) return 0;
  std::vector<RowTask> run, add;
  size_t j = i;
  for (; j < q.size(); j++) {
    const PendOp& p = q[j];
    if ((p.kind != PK_ROPE && p.kind != PK_QKNR && p.kind != PK_ROWCOPY) || p.map_act != q[i].map_act) break;
    if (p.kind != PK_QKNR && p.op == 1u) break;   // more rows than a run holds: launched by itself
    if (!expand(p, m, &add)) { if (j == i) return 0; break; }
    // every new task against every task already in the run
    std::vector<RowTask> next = run;
    bool ok = run.size() + add.size() <= ROWT_MAX || p.kind == PK_ROWCOPY;
    for (size_t a = 0; ok && a < add.size(); a++) {
      RowTask nt = add[a];
      bool merged = false;
      for (size_t e = 0; ok && e < run.size(); e++) {
        const RowTask& et = run[e];
        if (nt.flags == 0u && nt.dst == ROWT_NONE && et.dst == nt.src && et.dim == nt.dim && next[e].cache == ROWT_NONE &&
            !overlap(nt.cache, nt.dim, et.src, et.dim) && !overlap(nt.cache, nt.dim, et.w, et.dim) &&
            !overlap(nt.cache, nt.dim, et.dst, et.dim)) {
          // copy of a row an earlier task of the run produces
          bool clash = false;
          for (size_t f = 0; f < next.size(); f++)
            if (f != e && (overlap(nt.cache, nt.dim, next[f].src, next[f].dim) || overlap(nt.cache, nt.dim, next[f].dst, next[f].dim) ||
                           overlap(nt.cache, nt.dim, next[f].cache, next[f].dim) || overlap(nt.cache, nt.dim, next[f].w, next[f].dim)))
              clash = true;
          if (clash) { ok = false; break; }
          next[e].cache = nt.cache;
          merged = true;
          break;
        }
        const bool reads_written = overlap(nt.src, nt.dim, et.dst, et.dim) || overlap(nt.src, nt.dim, et.cache, et.dim) ||
                                   overlap(nt.w, nt.dim, et.dst, et.dim) || overlap(nt.w, nt.dim, et.cache, et.dim);
        const bool writes_used = overlap(nt.dst, nt.dim, et.src, et.dim) || overlap(nt.dst, nt.dim, et.w, et.dim) ||
                                 overlap(nt.dst, nt.dim, et.dst, et.dim) || overlap(nt.dst, nt.dim, et.cache, et.dim) ||
                                 overlap(nt.cache, nt.dim, et.src, et.dim) || overlap(nt.cache, nt.dim, et.w, et.dim) ||
                                 overlap(nt.cache, nt.dim, et.dst, et.dim) || overlap(nt.cache, nt.dim, et.cache, et.dim);
        if (reads_written || writes_used) ok = false;
      }
      if (ok && !merged) next.push_back(nt);
    }
    if (!ok || next.size() > ROWT_MAX) {
      if (j == i) { *alone = true; *out = add; return 1; }
      break;
    }
    run.swap(next);
  }
  *out = run;
  return j - i;
}

// Launches the run of row ops that starts at q[i]; returns how many queue entries it consumed.
size_t launch_row_run(const std::vector<PendOp>& q, size_t i, int* rc) {
  *rc = ADAMAH_OK;
  Map* m = get_f32_map(q[i].map_act);
  std::vector<RowTask> run;
  bool alone = false;
  const size_t used = build_row_run(q, i, &run, &alone);
  if (!m || used == 0) { *rc = ADAMAH_ERR_INVALID; return 1; }
  if (alone) {   // a single op that does not fit one launch: task by task in chunks (tasks of one op are independent)
    for (size_t a = 0; a < run.size() && *rc == ADAMAH_OK; a += ROWT_MAX)
      *rc = launch_tasks(m, std::vector<RowTask>(run.begin() + a, run.begin() + std::min(run.size(), a + (size_t)ROWT_MAX)));
    return 1;
  }
  *rc = launch_tasks(m, run);
  return used;
}

}  // namespace adamah
