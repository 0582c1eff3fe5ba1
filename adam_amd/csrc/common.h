// Shared state of libadamah_hip: maps, loc handles, the stream, staging and launch helpers.
//
// The library re-implements the native side of the ADAMAH op surface (reference:
// adamah-MAIN/adamah/adamah.c) for one MI355X.  Everything is ordered on one HIP stream,
// which replaces the reference's command-buffer batching and per-dispatch barriers.
#pragma once
#include <hip/hip_runtime.h>
#include <hip/hip_fp16.h>
#include <stdint.h>
#include <stddef.h>
#include <vector>
#include <utility>

// Error codes of the reference C ABI (adamah.c:24-28).
#define ADAMAH_OK 0
#define ADAMAH_ERR_BACKEND -1
#define ADAMAH_ERR_MEMORY -2
#define ADAMAH_ERR_INVALID -3
#define ADAMAH_ERR_NOT_FOUND -4

#define MAX_MAPS 16
#define MAX_RES 65536          // reference: 2048; ids stay 32-bit so a larger table is invisible to callers
#define MAX_PLANS 8
#define MAX_PLAN_OPS 4096
#define T_PARK_FLOATS 65536

#define DTYPE_F32 0
#define DTYPE_BF16 1
#define DTYPE_Q8 2
#define DTYPE_Q4 3
#define DTYPE_Q6 4
#define DTYPE_COUNT 5

#define WAVE 64

namespace adamah {

// How a quantised map's per-group parameters are held on the device.
enum QLayout : int {
  QL_AFFINE = 0,   // float2 (scale, zp) per group -- any qparams
  QL_BLOCK16 = 1,  // additionally an fp16 scale plane: every group has zp == -off*scale with an
                   // fp16-exact scale (off = 8 for Q4, 128 for Q8), i.e. GGUF Q4_0 / Q8_0 blocks
};

struct Map {
  bool active = false;
  uint32_t dtype = 0, word_size = 0, pack_size = 0, n_packs = 0, group_size = 0;
  uint64_t n_elems = 0, total_bytes = 0, n_groups = 0;
  uint8_t* buf = nullptr;   // f32 values, or packed codes (Q4: 2 per byte, Q8: 1 per byte)
  float2* qp = nullptr;     // (scale, zp) per group
  __half* d16 = nullptr;    // fp16 scale per group, valid for groups [0, block16_groups)
  uint64_t block16_groups = 0;
  // fp16 KV region of an f32 map: elements [kv_start, kv_start+kv_count) are mirrored in kv16
  uint64_t kv_start = 0, kv_count = 0;
  __half* kv16 = nullptr;
};

struct Res {
  bool active = false;
  uint32_t size_bytes = 0, cap_bytes = 0;
  uint8_t* dptr = nullptr;
  std::vector<uint8_t> host;  // last uploaded contents; empty when the device wrote the resource
  bool host_valid = false;
  bool contig = false;        // host copy is the uint32 sequence host[0], host[0]+1, host[0]+2, ...
};

// A row-wise op recorded inside a batch instead of being launched at once, so that neighbours can be
// folded into one kernel when the batch is flushed.  All offsets are element offsets resolved from
// the host copies of the handles at record time (any later handle upload flushes the queue first).
enum PendKind : uint32_t { PK_RMSNORM = 1, PK_GEMV = 2, PK_OP2 = 3, PK_ARGMAX = 4, PK_SCORES = 5, PK_ATTN = 6,
                           PK_ROPE = 7, PK_QKNR = 8, PK_ROWCOPY = 9, PK_GEMM = 10 };
struct PendOp {
  uint32_t kind = 0;
  uint32_t map_act = 0, map_wt = 0;
  uint32_t a = 0, b = 0, c = 0, d = 0;   // RMSNORM: src, weight, dst, residual.  GEMV: x, W, y.  OP2: a, b, dst.
  uint32_t n = 0, k = 0;                 // RMSNORM: n = dim.  GEMV/ARGMAX: k = K, n = N.  OP2: n elements.
  uint32_t op = 0;                       // RMSNORM: 1 = with residual.  GEMV/ARGMAX: weight format.  OP2: op code.
  uint32_t h[5] = {0, 0, 0, 0, 0};       // ARGMAX: idx, val, dst, x, W handles.  SCORES: q, K, score rows.  ATTN: scores, V, out
  uint32_t rpg = 0;                      // ARGMAX: rows per group.  SCORES / ATTN: number of heads (ops)
  float eps = 0.f;                       // RMSNORM: eps.  ATTN: score scale
  float f2 = 0.f;                        // ATTN: soft cap
  // SCORES: k = head dim, n = sequence length.  ATTN: n = sequence length, k = value dim.
  // ROPE (one token): a = src, c = dst, rpg = heads, k = head dim, n = position, eps = frequency base; op = 1: more
  //   heads than a row run holds (h = src, dst handles).
  // QKNR: h = q rows, q weights, k rows, k weights, dst; rpg/k = q rows/dim, op/d = k rows/dim, n, eps as ROPE.
  // ROWCOPY: h = spec, source base; rpg = copies, k = row size, n = destination row offset; op = 1: more copies than
  //   a row run holds.
  // GEMM (two or more activation rows, block16 weights): a, b, c = X, W, Y; rpg = M; k, n = K, N; op = weight format;
  //   h = X, W, Y handles.
};

struct Stats {
  uint64_t dispatch = 0, submit = 0, barrier = 0, fusion_flush = 0;
  uint32_t last_batch_dispatch = 0;
};

enum : uint32_t { ZERO_WORD = 64 };   // index into Ctx::sync_ctr

struct PlanOp {  // mirrors DecodePlanOp (adamah.c:175-194)
  uint32_t kind, map_id, map_id2, op_code, h0, h1, h2, h3, h4, h5, u0, u1, u2, u3, u4, u5;
  float f0, f1;
};

struct Ctx {
  bool initialized = false;
  int device = 0;
  hipStream_t stream = nullptr;
  hipDeviceProp_t prop;
  int n_cu = 256;
  Map maps[MAX_MAPS];
  std::vector<Res> res;      // index = handle id (0 unused)
  uint32_t res_next = 1;
  // device arena for handles
  std::vector<uint8_t*> arena_chunks;
  uint8_t* arena_cur = nullptr;
  size_t arena_left = 0;
  // pinned staging, double buffered
  uint8_t* stage[2] = {nullptr, nullptr};
  size_t stage_cap = 0, stage_off = 0;
  int stage_cur = 0;
  bool stage_used[2] = {false, false};
  // attention split-KV partials
  float* attn_scratch = nullptr;
  size_t attn_scratch_floats = 0;
  int batch_depth = 0;
  int fusion_enabled = 0;
  int scheduler_mode = 0;
  uint32_t active_dtype = 0;
  Stats stats;
  hipEvent_t timer_ev[2] = {nullptr, nullptr};
  std::vector<PlanOp> plans[MAX_PLANS];
  bool plan_active[MAX_PLANS] = {false};
  // deferred row-wise ops of the open batch
  std::vector<PendOp> pend;
  int no_defer = 0;              // > 0 while an entry point runs on library-owned scratch handles
  uint64_t mem_gen = 0;          // counts host-to-device copies (with stats.dispatch: "has device memory changed?")
  uint32_t* sync_ctr = nullptr;  // device counters for last-workgroup epilogues, zero between launches (word 0 in use);
                                 // word ZERO_WORD is cleared at init and never written: a constant zero for kernels
  float* t_park = nullptr;       // T_PARK_FLOATS floats: a row on its way to a place that is still being read
  int deferred_err = 0;          // first failure of a queued op's launch; returned (once) by the next call that can
  uint64_t layout_gen = 0;       // counts events after which device pointers or offsets seen earlier may be stale:
                                 // a map created, destroyed or given new qparams / an fp16 KV range, a library
                                 // scratch buffer re-allocated (recorded HIP graphs are dropped when it moves)
};

extern Ctx g;

// ---- runtime helpers (runtime.hip) -------------------------------------------------------
Map* get_map(uint32_t id);                       // nullptr unless active
Map* get_f32_map(uint32_t id);                   // nullptr unless active and DTYPE_F32
Res* get_res(uint32_t h);                        // nullptr unless active
// Device pointer to a handle's words, or nullptr if the handle is missing or shorter than n words.
const uint32_t* res_u32(uint32_t h, uint64_t n_words);
// Host copy of a handle's words (nullptr when the device produced it or it is too short).
const uint32_t* res_host(uint32_t h, uint64_t n_words);
uint32_t res_alloc(uint32_t n_bytes);            // 0 on failure
// Library-owned handle `slot` (0..7) holding a copy of host data; reused across calls.
uint32_t scratch_handle(int slot, const void* data, uint32_t n_bytes);
void* stage_alloc(size_t n);                     // pinned region; enqueue its copy before allocating much more
int h2d(void* dst, const void* src, size_t n);   // stream-ordered, source consumed before return
int d2h(void* dst, const void* src, size_t n);   // stream-ordered copy + wait
// Deferral of row-wise ops (fuse.hip).  Every extern "C" entry point that is not itself deferred
// starts with ADAMAH_API(), which launches whatever is pending, so stream order equals call order.
bool can_defer();                // inside a batch, fusion not disabled, no scratch handles involved
void flush_pending();
#define ADAMAH_API() do { if (!adamah::g.pend.empty()) adamah::flush_pending(); } while (0)
// Element offset held by a single-entry handle whose host copy is known; false otherwise.
bool res_scalar(uint32_t h, uint32_t* out);
// First element of a handle whose host copy is a run of n consecutive indices; false otherwise.
bool res_run(uint32_t h, uint64_t n, uint32_t* start);
void gemm_q4_mfma_release();   // frees the GEMM's scratch (shutdown)
void sampling_release();       // frees the scratch lists of the chunked top-k (shutdown)
void topk_fused_release();     // frees the scratch logits of the GEMV + top-k ops (shutdown)
int topk_noalloc_setup(int device);   // topk_fused.hip: address of this device's fixed logit scratch (init)
size_t launch_argmax_run(const std::vector<PendOp>& q, size_t i, int* rc);   // topk_fused.hip
int launch_argmax_direct(const PendOp& p);   // gemv_q.hip: one queued Q8 GEMV + argmax
int launch_rmsnorm_v(const PendOp& p);
bool row_op_deferrable(const PendOp& p);                                  // rowprep.hip
// Element ranges (start, length) of the activation map a queued row op reads or writes; false: not known on the host.
bool row_op_ranges(const PendOp& p, std::vector<std::pair<uint64_t, uint64_t>>* out);   // rowprep.hip
size_t launch_row_run(const std::vector<PendOp>& q, size_t i, int* rc);   // rowprep.hip
// a rotation / row copy with more rows than a row run holds (PendOp.op == 1): alone, or rotation + rotation + KV append
// of one position in one launch; returns the queue entries used
#define ROW_RUN_MAX 64u
size_t launch_wide_rows(const std::vector<PendOp>& q, size_t i, int* rc);   // norm_rope.hip
int launch_op2_v(const PendOp& p);
// Attention (attention.hip): stand-alone launches of queued ops, and the fused form.  launch_attn
// runs scores (when sc != nullptr) and softmax . V; with leave_partials it stops before the merge
// of the sequence splits and reports their layout so that the consumer can merge them itself.
// q_n > 0: the launch also prepared the token's queries and left them in scratch memory; whoever merges the
// partials copies q_n floats from q_src to element q_dst of the map (the rows the rotation writes).
struct AttnPartials { const float* base; uint32_t n_splits, value_dim, n_ops, out0; const float* q_src; uint32_t q_dst, q_n; };
int launch_scores(const PendOp& sc);
struct RowPrepCtx;   // attn_common.h: the row ops queued just before the pair, offered to the attention launch
int launch_attn(const PendOp* sc, const PendOp& at, bool leave_partials, AttnPartials* ap, const RowPrepCtx* prep = nullptr);
int launch_attn_combine(const PendOp& at, const AttnPartials& ap);
bool attn_foldable(const PendOp& sc, const PendOp& at);
size_t launch_attn_chunk(const std::vector<PendOp>& q, size_t i, int* rc);   // attn_prefill.hip
size_t launch_attn_batch(const std::vector<PendOp>& q, size_t i, int* rc);   // attn_decode.hip
int launch_attn_combine_dev(Map* m, const float* partial, const uint32_t* lo_dev, uint32_t n_ops, uint32_t value_dim,
                            uint32_t n_splits);
void attn_decode_release();
void attn_prefill_release();   // attn_prefill.hip: the transposed V tiles (shutdown)
void token_feed_release();      // frees the pinned ring tokens reach the host through (shutdown)

inline void layout_changed() { g.layout_gen++; }
inline void count_launch(int n = 1) { g.stats.dispatch += n; g.stats.barrier += n; g.stats.last_batch_dispatch += n; }
int check_launch();                              // hipGetLastError -> ADAMAH code

inline uint32_t cdiv(uint64_t a, uint64_t b) { return (uint32_t)((a + b - 1) / b); }

// True when [lo, lo+n) lies inside a map of n_elems elements.
inline bool in_range(uint64_t lo, uint64_t n, uint64_t n_elems) { return lo <= n_elems && n <= n_elems - lo; }

// ---- internal op entry points shared between translation units -----------------------------
int op_matmul_t_xq(uint32_t dtype, uint32_t map_act, uint32_t map_wt, uint32_t ha, uint32_t hb, uint32_t hc,
                   uint32_t M, uint32_t K, uint32_t N, uint32_t n_ops, bool transposed);
int op_matvec_argmax(uint32_t dtype, uint32_t map_act, uint32_t map_wt, uint32_t ha, uint32_t hb, uint32_t hidx,
                     uint32_t hval, uint32_t hdst, uint32_t K, uint32_t N, uint32_t rows_per_group);

}  // namespace adamah
