// Shared by the attention kernels: score preparation and the launch interface of the grouped
// decode kernel.
#pragma once
#include "common.h"
#include <vector>

namespace adamah {

// map_attn_softmax_value.comp:52-60: scale, then the optional tanh soft cap.
__device__ __forceinline__ float prep(float v, float scale, float cap) {
  v *= scale;
  if (cap > 0.0f) v = tanhf(v / cap) * cap;
  return v;
}

// Same arithmetic as rope_cs in norm_rope.hip.
__device__ __forceinline__ void rope_cs2(uint32_t i, uint32_t dim, uint32_t pos, float base, float* c, float* s) {
  const float e = (float)(2u * i) / (float)dim;
  const float p = (float)pow((double)base, (double)e);
  const float angle = (float)pos * (1.0f / p);
  *c = cosf(angle);
  *s = sinf(angle);
}

// A row task of the preparation before decode attention (rowprep.hip): source row, optional norm weights,
// optional rotation, destination row, optional cache row.
#define ROWT_MAX ROW_RUN_MAX
#define ROWT_NONE 0xFFFFFFFFu
struct RowTask {
  uint32_t src, dst, cache, w;   // element offsets; dst / cache / w may be ROWT_NONE
  uint32_t dim, pos, flags;      // flags: 1 = RMSNorm (eps 1e-6), 2 = RoPE
  float base;
};
size_t build_row_run(const std::vector<PendOp>& q, size_t i, std::vector<RowTask>* out, bool* alone);
// The run of row ops q[i0 ...] that directly precedes a (scores, softmax . V) pair, as merged tasks.  The decode
// attention launch does them itself when they are exactly the preparation of its own operands; otherwise
// launch_attn launches the run on its own first.
struct RowPrepCtx { const std::vector<PendOp>* q; size_t i0; std::vector<RowTask> tasks; };

// Grouped decode attention (attn_decode.hip).  Returns false when the shape is not one it covers and
// nothing was launched; otherwise *rc carries the launch status, *ap the partials still to be merged
// (n_splits == 1: the outputs are final) and *left whether they are few enough for the consumer.
struct AttnDecodeArgs {
  float* data;                  // the float32 map (queries, score rows, outputs)
  const __half* kv;             // fp16 copy of the KV range
  uint64_t kv_shift;            // first element of that range
  const uint32_t *la, *lb, *lc, *lv, *lo;        // device handles: q rows, K bases, score rows, V bases, out rows
  const uint32_t *ha, *hb, *hc, *hv, *ho;        // their host copies
  uint32_t n_ops, head_dim, row_size;
  float scale, cap;
  bool leave_partials;          // stop before the merge of the sequence splits when there are few partials
  uint32_t fold_floats;         // "few": at most this many partial floats
  const std::vector<RowTask>* prep;   // optional: the row tasks queued just before the pair (rotation of the new
                                      // Q / K rows, KV append); done inside the launch when they fit its pattern
  bool* prep_done;              // set by launch_attn_decode when it took them
};
bool launch_attn_decode(const AttnDecodeArgs& a, AttnPartials* ap, bool* left, int* rc);
int tuning(const char* name, int dflt);   // behaviour switch from the environment (gemv_q.hip)
int knob(const char* name, int dflt);     // launch-shape number, fixed unless built with -DADAMAH_TUNING

}  // namespace adamah
