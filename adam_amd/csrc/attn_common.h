// Shared by the attention kernels: score preparation and the launch interface of the grouped
// decode kernel.
#pragma once
#include "common.h"

namespace adamah {

// map_attn_softmax_value.comp:52-60: scale, then the optional tanh soft cap.
__device__ __forceinline__ float prep(float v, float scale, float cap) {
  v *= scale;
  if (cap > 0.0f) v = tanhf(v / cap) * cap;
  return v;
}

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
};
bool launch_attn_decode(const AttnDecodeArgs& a, AttnPartials* ap, bool* left, int* rc);
int tuning(const char* name, int dflt);   // behaviour switch from the environment (gemv_q.hip)
int knob(const char* name, int dflt);     // launch-shape number, fixed unless built with -DADAMAH_TUNING

}  // namespace adamah
