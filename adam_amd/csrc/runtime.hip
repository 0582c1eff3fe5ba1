// Context, maps, handles, host<->device traffic, batching and bookkeeping entry points.
#include "common.h"
#include "../../include/adamah_hip.h"
#include <string.h>
#include <stdio.h>
#include <stdlib.h>
#include <algorithm>
#include <deque>
#include "gemv_common.h"

namespace adamah {

Ctx g;

#define HIPCHK(expr)                                                        \
  do {                                                                      \
    hipError_t _e = (expr);                                                 \
    if (_e != hipSuccess) {                                                 \
      if (getenv("ADAMAH_DEBUG"))                                           \
        fprintf(stderr, "adamah_hip: %s -> %s\n", #expr, hipGetErrorString(_e)); \
      return (_e == hipErrorOutOfMemory) ? ADAMAH_ERR_MEMORY : ADAMAH_ERR_BACKEND; \
    }                                                                       \
  } while (0)

int check_launch() {
  hipError_t e = hipGetLastError();
  if (e != hipSuccess) {
    if (getenv("ADAMAH_DEBUG")) fprintf(stderr, "adamah_hip: launch -> %s\n", hipGetErrorString(e));
    return ADAMAH_ERR_BACKEND;
  }
  // An op queued earlier has already returned ADAMAH_OK to its caller; if its launch failed when the queue was
  // flushed, the first entry point that launches afterwards reports it.
  if (g.deferred_err && g.pend.empty()) { const int d = g.deferred_err; g.deferred_err = 0; return d; }
  return ADAMAH_OK;
}

Map* get_map(uint32_t id) {
  if (!g.initialized || id >= MAX_MAPS || !g.maps[id].active) return nullptr;
  return &g.maps[id];
}
Map* get_f32_map(uint32_t id) {
  Map* m = get_map(id);
  return (m && m->dtype == DTYPE_F32) ? m : nullptr;
}
Res* get_res(uint32_t h) {
  if (h == 0 || h >= g.res.size() || !g.res[h].active) return nullptr;
  return &g.res[h];
}
const uint32_t* res_u32(uint32_t h, uint64_t n_words) {
  Res* r = get_res(h);
  if (!r || n_words * 4 > r->size_bytes) return nullptr;
  return (const uint32_t*)r->dptr;
}
const uint32_t* res_host(uint32_t h, uint64_t n_words) {
  Res* r = get_res(h);
  if (!r || !r->host_valid || n_words * 4 > r->size_bytes) return nullptr;
  return (const uint32_t*)r->host.data();
}

// ---- device arena for handles: bump allocation out of 64 MiB chunks, released at shutdown ----
static uint8_t* arena_alloc(size_t n) {
  n = (n + 255) & ~(size_t)255;
  if (n > g.arena_left) {
    size_t chunk = std::max<size_t>(n, (size_t)64 << 20);
    uint8_t* p = nullptr;
    if (hipMalloc((void**)&p, chunk) != hipSuccess) return nullptr;
    g.arena_chunks.push_back(p);
    g.arena_cur = p;
    g.arena_left = chunk;
  }
  uint8_t* out = g.arena_cur;
  g.arena_cur += n;
  g.arena_left -= n;
  return out;
}

uint32_t res_alloc(uint32_t n_bytes) {
  if (n_bytes == 0 || g.res_next >= MAX_RES) return 0;
  uint8_t* p = arena_alloc(n_bytes);
  if (!p) return 0;
  uint32_t id = g.res_next++;
  if (g.res.size() <= id) g.res.resize(std::max<size_t>(id + 1, g.res.size() * 2));
  Res& r = g.res[id];
  r.active = true;
  r.size_bytes = n_bytes;
  r.cap_bytes = (n_bytes + 255u) & ~255u;
  r.dptr = p;
  r.host.clear();
  r.host_valid = false;
  r.contig = false;
  return id;
}

// map_gather_dev results, one ring per size class (storage rounded up to a power of two, 256 B at least), each in
// the order the results were made.  Once a class holds gather_class_limit() results its oldest is handed out again
// (same id, same storage), so ids and arena bytes stay bounded whatever sizes a caller alternates between: a class
// keeps at most 64 MiB (two results for the classes above 32 MiB) and at most 4096 results.
enum : uint32_t { GATHER_CLASSES = 33, GATHER_MIN_LOG2 = 8 };
static std::deque<uint32_t> g_gather_ring[GATHER_CLASSES];
static inline uint32_t gather_class(uint32_t need) {
  uint32_t c = GATHER_MIN_LOG2;
  while (c < 32 && ((uint64_t)1 << c) < need) ++c;
  return c;
}
static inline size_t gather_class_limit(uint32_t c) {
  const uint64_t n = ((uint64_t)64 << 20) >> c;
  return (size_t)(n < 2 ? 2 : n > 4096 ? 4096 : n);
}
static void gather_ring_reset() { for (auto& r : g_gather_ring) r.clear(); }

// Remember what was uploaded into a handle, and whether it is a run of consecutive indices.
static void note_host(Res* r, const void* data, uint32_t n_bytes) {
  r->host.assign((const uint8_t*)data, (const uint8_t*)data + n_bytes);
  r->host_valid = true;
  r->contig = false;
  if (n_bytes >= 4 && (n_bytes & 3u) == 0) {
    const uint32_t* v = (const uint32_t*)r->host.data();
    const uint32_t n = n_bytes >> 2;
    bool run = true;
    for (uint32_t i = 1; run && i < n; i++) run = v[i] == v[0] + i;
    r->contig = run;
  }
}

static uint32_t g_scratch_h[8] = {0, 0, 0, 0, 0, 0, 0, 0};
uint32_t scratch_handle(int slot, const void* data, uint32_t n_bytes) {
  if (slot < 0 || slot >= 8 || n_bytes == 0 || !data) return 0;
  Res* r = get_res(g_scratch_h[slot]);
  if (!r || r->cap_bytes < n_bytes) {
    g_scratch_h[slot] = res_alloc(std::max<uint32_t>(n_bytes, 4096u));
    r = get_res(g_scratch_h[slot]);
    if (!r) return 0;
  }
  r->size_bytes = n_bytes;
  note_host(r, data, n_bytes);
  if (h2d(r->dptr, data, n_bytes) != ADAMAH_OK) return 0;
  return g_scratch_h[slot];
}

// ---- pinned staging: two buffers used alternately.  Before a buffer is handed out again the
// stream is drained, so every async copy issued from it has consumed its source.  Callers must
// enqueue the copy of a region before allocating more than one further buffer's worth. ----------
void* stage_alloc(size_t n) {
  n = (n + 255) & ~(size_t)255;
  if (n > g.stage_cap) return nullptr;
  if (g.stage_off + n > g.stage_cap) {
    g.stage_cur ^= 1;
    if (g.stage_used[g.stage_cur]) hipStreamSynchronize(g.stream);
    g.stage_off = 0;
  }
  g.stage_used[g.stage_cur] = true;
  void* p = g.stage[g.stage_cur] + g.stage_off;
  g.stage_off += n;
  return p;
}

int h2d(void* dst, const void* src, size_t n) {
  g.mem_gen++;
  const uint8_t* s = (const uint8_t*)src;
  uint8_t* d = (uint8_t*)dst;
  while (n) {
    size_t c = std::min(n, g.stage_cap);
    void* p = stage_alloc(c);
    if (!p) return ADAMAH_ERR_MEMORY;
    memcpy(p, s, c);
    HIPCHK(hipMemcpyAsync(d, p, c, hipMemcpyHostToDevice, g.stream));
    s += c; d += c; n -= c;
  }
  return ADAMAH_OK;
}

int d2h(void* dst, const void* src, size_t n) {
  uint8_t* d = (uint8_t*)dst;
  const uint8_t* s = (const uint8_t*)src;
  while (n) {
    size_t c = std::min(n, g.stage_cap);
    void* p = stage_alloc(c);
    if (!p) return ADAMAH_ERR_MEMORY;
    HIPCHK(hipMemcpyAsync(p, s, c, hipMemcpyDeviceToHost, g.stream));
    HIPCHK(hipStreamSynchronize(g.stream));
    memcpy(d, p, c);
    s += c; d += c; n -= c;
  }
  return ADAMAH_OK;
}

// ---- fp16 bit conversion on the host (round to nearest even) ---------------------------------
static uint16_t f32_to_f16_bits(float f) {
  uint32_t x;
  memcpy(&x, &f, 4);
  uint32_t sign = (x >> 16) & 0x8000u;
  uint32_t mant = x & 0x7FFFFFu;
  int32_t exp = (int32_t)((x >> 23) & 0xFF);
  if (exp == 0xFF) return (uint16_t)(sign | 0x7C00u | (mant ? 0x200u : 0));
  int32_t e = exp - 127 + 15;
  if (e >= 31) return (uint16_t)(sign | 0x7C00u);
  if (e <= 0) {
    if (e < -10) return (uint16_t)sign;
    mant |= 0x800000u;
    uint32_t shift = (uint32_t)(14 - e);
    uint32_t half = mant >> shift;
    uint32_t rem = mant & ((1u << shift) - 1), mid = 1u << (shift - 1);
    if (rem > mid || (rem == mid && (half & 1))) half++;
    return (uint16_t)(sign | half);
  }
  uint32_t half = ((uint32_t)e << 10) | (mant >> 13);
  uint32_t rem = mant & 0x1FFFu;
  if (rem > 0x1000u || (rem == 0x1000u && (half & 1))) half++;
  return (uint16_t)(sign | half);
}
static float f16_bits_to_f32(uint16_t h) {
  uint32_t sign = (uint32_t)(h & 0x8000u) << 16, exp = (h >> 10) & 0x1F, mant = h & 0x3FFu, x;
  if (exp == 0) {
    if (mant == 0) x = sign;
    else {
      int e = -1;
      do { mant <<= 1; e++; } while (!(mant & 0x400u));
      x = sign | ((uint32_t)(127 - 15 - e) << 23) | ((mant & 0x3FFu) << 13);
    }
  } else if (exp == 31) x = sign | 0x7F800000u | (mant << 13);
  else x = sign | ((exp - 15 + 127) << 23) | (mant << 13);
  float f;
  memcpy(&f, &x, 4);
  return f;
}

// ---- small kernels -----------------------------------------------------------------------------
__global__ void k_fill_u32(uint32_t* p, uint32_t v, uint64_t n) {
  uint64_t i = (uint64_t)blockIdx.x * blockDim.x + threadIdx.x, st = (uint64_t)gridDim.x * blockDim.x;
  for (; i < n; i += st) p[i] = v;
}
__global__ void k_fill_qp(float2* p, uint64_t n) {
  uint64_t i = (uint64_t)blockIdx.x * blockDim.x + threadIdx.x, st = (uint64_t)gridDim.x * blockDim.x;
  for (; i < n; i += st) p[i] = make_float2(1.0f, 0.0f);
}
// f32 scatter by pack index (shaders/src/f32/map_scatter.comp); mirrors into the fp16 KV copy.
__global__ void k_scatter_f32(float* map, const float* src, const uint32_t* locs, uint64_t n_locs, uint32_t pack,
                              uint64_t n_elems, __half* kv16, uint64_t kv_start, uint64_t kv_count) {
  uint64_t tid = (uint64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (tid >= n_locs * pack) return;
  uint64_t idx = (uint64_t)locs[tid / pack] * pack + tid % pack;
  if (idx >= n_elems) return;
  float v = src[tid];
  if (kv16 && idx >= kv_start && idx - kv_start < kv_count) {
    __half h = __float2half(v);
    kv16[idx - kv_start] = h;
    v = __half2float(h);
  }
  map[idx] = v;
}
__global__ void k_scatter_u8(uint8_t* map, const uint8_t* src, const uint32_t* locs, uint64_t n_locs, uint32_t pack,
                             uint64_t n_elems) {
  uint64_t tid = (uint64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (tid >= n_locs * pack) return;
  uint64_t idx = (uint64_t)locs[tid / pack] * pack + tid % pack;
  if (idx < n_elems) map[idx] = src[tid];
}
// Device quantiser for f32 -> Q4 scatter (shaders/src/q4/map_scatter.comp:13-34).
__global__ void k_scatter_q4(uint32_t* map, const float* src, const uint32_t* locs, uint64_t n_locs, uint32_t pack,
                             uint32_t group, uint64_t base_pack, int use_locs, const float2* qp, uint64_t n_elems) {
  uint64_t tid = (uint64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (tid >= n_locs * pack) return;
  uint64_t li = tid / pack, ei = tid % pack;
  uint64_t idx = (use_locs ? (uint64_t)locs[li] : base_pack + li) * pack + ei;
  if (idx >= n_elems) return;
  float2 p = qp[idx / group];
  float qf = (src[tid] - p.y) / fmaxf(p.x, 1e-10f);
  uint32_t q = (uint32_t)fminf(fmaxf(rintf(qf), 0.0f), 15.0f);
  uint32_t shift = (uint32_t)(idx & 7) * 4;
  atomicAnd(&map[idx >> 3], ~(0xFu << shift));
  atomicOr(&map[idx >> 3], (q & 0xFu) << shift);
}
__global__ void k_gather_f32(const float* map, float* dst, const uint32_t* locs, uint64_t n_locs, uint32_t pack,
                             uint64_t n_elems) {
  uint64_t tid = (uint64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (tid >= n_locs * pack) return;
  uint64_t idx = (uint64_t)locs[tid / pack] * pack + tid % pack;
  dst[tid] = idx < n_elems ? map[idx] : 0.0f;
}
__global__ void k_gather_u8(const uint8_t* map, uint8_t* dst, const uint32_t* locs, uint64_t n_locs, uint64_t n_bytes) {
  uint64_t tid = (uint64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (tid >= n_locs) return;
  uint64_t idx = locs[tid];
  dst[tid] = idx < n_bytes ? map[idx] : 0;
}
// Dequantising gather (shaders/src/q4/map_gather.comp, q8 analogue): float(code)*scale + zp.
__global__ void k_gather_q(const uint8_t* map, float* dst, const uint32_t* locs, uint64_t n_locs, uint32_t pack,
                           uint32_t group, const float2* qp, uint64_t n_elems, int is_q4) {
  uint64_t tid = (uint64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (tid >= n_locs * pack) return;
  uint64_t idx = (uint64_t)locs[tid / pack] * pack + tid % pack;
  if (idx >= n_elems) { dst[tid] = 0.0f; return; }
  uint32_t code = is_q4 ? ((map[idx >> 1] >> ((idx & 1) * 4)) & 0xFu) : map[idx];
  float2 p = qp[idx / group];
  dst[tid] = __fadd_rn(__fmul_rn((float)code, p.x), p.y);
}
// Round a float32 range to fp16 in place and refresh its fp16 mirror.
__global__ void k_f32_to_kv16(float* src, __half* dst, uint64_t n) {
  uint64_t i = (uint64_t)blockIdx.x * blockDim.x + threadIdx.x, st = (uint64_t)gridDim.x * blockDim.x;
  for (; i < n; i += st) {
    __half h = __float2half(src[i]);
    dst[i] = h;
    src[i] = __half2float(h);
  }
}

static uint32_t fill_grid(uint64_t n) { return (uint32_t)std::min<uint64_t>(cdiv(n, 256), 65535u * 4); }

// Temporary device buffer that lives until the stream has passed the work using it: allocated
// from the handle arena's allocator would leak, so a growable scratch pair is kept instead.
static uint8_t* g_tmp[3] = {nullptr, nullptr, nullptr};
static size_t g_tmp_cap[3] = {0, 0, 0};
static void* tmp_dev(int slot, size_t n) {
  if (n <= g_tmp_cap[slot]) return g_tmp[slot];
  hipStreamSynchronize(g.stream);
  layout_changed();
  if (g_tmp[slot]) hipFree(g_tmp[slot]);
  g_tmp[slot] = nullptr;
  g_tmp_cap[slot] = 0;
  size_t cap = std::max<size_t>(n, (size_t)1 << 20);
  if (hipMalloc((void**)&g_tmp[slot], cap) != hipSuccess) return nullptr;
  g_tmp_cap[slot] = cap;
  return g_tmp[slot];
}

static void destroy_map(Map* m) {
  hipStreamSynchronize(g.stream);
  layout_changed();
  if (m->buf) hipFree(m->buf);
  if (m->qp) hipFree(m->qp);
  if (m->d16) hipFree(m->d16);
  if (m->kv16) hipFree(m->kv16);
  *m = Map();
}

}  // namespace adamah

using namespace adamah;

static void plan_graph_reset(uint32_t plan_id);   // drops the recorded graphs of a decode plan (defined with them)
static void plan_graph_handle_rewritten(uint32_t handle);   // a recorded graph holds the old contents of a handle by value

// =================================================================================================
extern "C" {

int adamah_init_ex(uint64_t hot_bytes, uint64_t cold_bytes) {
  (void)hot_bytes; (void)cold_bytes;
  if (g.initialized) return ADAMAH_OK;
  int n = 0;
  if (hipGetDeviceCount(&n) != hipSuccess || n <= 0) return ADAMAH_ERR_BACKEND;
  HIPCHK(hipSetDevice(0));
  g.device = 0;
  HIPCHK(hipGetDeviceProperties(&g.prop, 0));
  g.n_cu = g.prop.multiProcessorCount > 0 ? g.prop.multiProcessorCount : 256;
  HIPCHK(hipStreamCreateWithFlags(&g.stream, hipStreamNonBlocking));
  g.stage_cap = (size_t)32 << 20;
  for (int i = 0; i < 2; i++) {
    HIPCHK(hipHostMalloc((void**)&g.stage[i], g.stage_cap, hipHostMallocDefault));
    g.stage_used[i] = false;
    HIPCHK(hipEventCreate(&g.timer_ev[i]));
  }
  g.stage_off = 0; g.stage_cur = 0;
  g.res.assign(4096, Res());
  g.res_next = 1;
  g.attn_scratch_floats = (size_t)4 << 20;   // 16 MiB of split-KV partials
  HIPCHK(hipMalloc((void**)&g.attn_scratch, g.attn_scratch_floats * sizeof(float)));
  // counters of the GEMV prologues (1 KiB), then the row a folded norm + residual parks until a later launch puts
  // it in place (T_PARK_FLOATS floats)
  HIPCHK(hipMalloc((void**)&g.sync_ctr, 1024 + (size_t)T_PARK_FLOATS * 4));
  HIPCHK(hipMemsetAsync(g.sync_ctr, 0, 1024, g.stream));
  g.t_park = (float*)((uint8_t*)g.sync_ctr + 1024);
  if (int r = topk_noalloc_setup(g.device)) return r;
  g.pend.clear();
  g.batch_depth = 0; g.fusion_enabled = 0; g.scheduler_mode = 0; g.active_dtype = 0;
  g.stats = Stats();
  g.initialized = true;
  return ADAMAH_OK;
}

int adamah_init(void) { return adamah_init_ex(0, 0); }

void adamah_shutdown(void) { ADAMAH_API();
  if (!g.initialized) return;
  hipStreamSynchronize(g.stream);
  for (int i = 0; i < MAX_MAPS; i++)
    if (g.maps[i].active) destroy_map(&g.maps[i]);
  for (uint8_t* p : g.arena_chunks) hipFree(p);
  g.arena_chunks.clear(); g.arena_cur = nullptr; g.arena_left = 0;
  g.res.clear();
  gather_ring_reset();
  for (int i = 0; i < 8; i++) g_scratch_h[i] = 0;
  for (int i = 0; i < 3; i++) { if (g_tmp[i]) hipFree(g_tmp[i]); g_tmp[i] = nullptr; g_tmp_cap[i] = 0; }
  for (int i = 0; i < 2; i++) {
    if (g.stage[i]) hipHostFree(g.stage[i]);
    g.stage[i] = nullptr;
    if (g.timer_ev[i]) hipEventDestroy(g.timer_ev[i]);
    g.timer_ev[i] = nullptr;
  }
  if (g.attn_scratch) hipFree(g.attn_scratch);
  g.attn_scratch = nullptr;
  if (g.sync_ctr) hipFree(g.sync_ctr);
  g.sync_ctr = nullptr;
  g.t_park = nullptr;
  gemm_q4_mfma_release();
  topk_fused_release();
  sampling_release();
  attn_decode_release();
  attn_prefill_release();
  token_feed_release();
  g.pend.clear();
  for (int i = 0; i < MAX_PLANS; i++) { g.plans[i].clear(); g.plan_active[i] = false; plan_graph_reset(i); }
  hipStreamDestroy(g.stream);
  g.stream = nullptr;
  g.initialized = false;
}

void adamah_sync(void) { ADAMAH_API(); if (g.initialized) hipStreamSynchronize(g.stream); }
void adamah_synchronize(uint64_t ticket) { (void)ticket; adamah_sync(); }
void adamah_synchronize_all(void) { adamah_sync(); }

int adamah_probe_device(uint64_t* heap_bytes, uint64_t* budget_bytes, uint64_t* usage_bytes, uint32_t* device_type) {
  size_t free_b = 0, total_b = 0;
  int n = 0;
  if (hipGetDeviceCount(&n) != hipSuccess || n <= 0) return ADAMAH_ERR_BACKEND;
  if (hipMemGetInfo(&free_b, &total_b) != hipSuccess) return ADAMAH_ERR_BACKEND;
  if (heap_bytes) *heap_bytes = total_b;
  if (budget_bytes) *budget_bytes = total_b;
  if (usage_bytes) *usage_bytes = total_b - free_b;
  if (device_type) *device_type = 2;  // discrete
  return ADAMAH_OK;
}
int adamah_is_integrated_gpu(void) { return 0; }
void adamah_set_xq_matmul_wg(uint32_t, uint32_t) {}
void adamah_get_gpu_caps(uint32_t* wg, uint32_t* sub, uint64_t* vram) {
  if (wg) *wg = 1024;
  if (sub) *sub = WAVE;
  if (vram) *vram = g.initialized ? (uint64_t)g.prop.totalGlobalMem : 0;
}

// ---- batching / fusion: a HIP stream is already ordered, so these only keep the books ---------
void batch_begin(void) {
  if (!g.initialized) return;
  if (g.batch_depth++ == 0) g.stats.last_batch_dispatch = 0;
}
void batch_end(void) { ADAMAH_API();
  if (!g.initialized || g.batch_depth == 0) return;
  if (--g.batch_depth == 0) g.stats.submit++;
}
void adamah_fusion_enable(int enable) { g.fusion_enabled = enable ? 1 : 0; }
int adamah_fusion_is_enabled(void) { return g.fusion_enabled; }
// A scheduling hint in the reference (submit what has been fused so far); results only become
// observable at a sync or a read-back, so the pending queue is left alone.
int adamah_fusion_flush(void) { g.stats.fusion_flush++; return ADAMAH_OK; }
// First failure among launches of queued ops since the last call, then cleared (0 when none).
static int take_deferred_err() { const int d = g.deferred_err; g.deferred_err = 0; return d; }
void adamah_fusion_set_scheduler_mode(int mode) { if (mode >= 0 && mode <= 2) g.scheduler_mode = mode; }
int adamah_fusion_get_scheduler_mode(void) { return g.scheduler_mode; }
int adamah_register_loc_span(uint32_t h, uint32_t map_id, uint32_t, uint32_t) { ADAMAH_API();
  return (get_res(h) && map_id < MAX_MAPS) ? ADAMAH_OK : ADAMAH_ERR_INVALID;
}
int adamah_register_row_base_span(uint32_t h, uint32_t map_id, uint32_t, uint32_t, uint32_t, uint32_t) { ADAMAH_API();
  return (get_res(h) && map_id < MAX_MAPS) ? ADAMAH_OK : ADAMAH_ERR_INVALID;
}
void adamah_clear_loc_alias_meta(uint32_t) { ADAMAH_API();}
void adamah_stats_reset(void) { ADAMAH_API(); g.stats = Stats(); }
void adamah_stats_get(uint64_t* dispatch, uint64_t* submit, uint64_t* barrier, uint64_t* flush, uint64_t* dsu,
                      uint64_t* hit, uint64_t* miss, uint64_t* alias, uint64_t* mode) { ADAMAH_API();
  if (dispatch) *dispatch = g.stats.dispatch;   // kernel launches
  if (submit) *submit = g.stats.submit;
  if (barrier) *barrier = g.stats.barrier;      // in-order stream: one implicit dependency per launch
  if (flush) *flush = g.stats.fusion_flush;
  if (dsu) *dsu = 0;
  if (hit) *hit = 0;
  if (miss) *miss = 0;
  if (alias) *alias = 0;
  if (mode) *mode = (uint64_t)g.scheduler_mode;
}
uint32_t adamah_get_last_barrier_count(void) { ADAMAH_API(); return g.stats.last_batch_dispatch; }

// ---- maps ------------------------------------------------------------------------------------------
int adamah_set_dtype(uint32_t dtype) {
  if (!g.initialized || dtype >= DTYPE_COUNT) return ADAMAH_ERR_INVALID;
  if (dtype == DTYPE_BF16 || dtype == DTYPE_Q6) return ADAMAH_ERR_INVALID;  // storage types not built
  g.active_dtype = dtype;
  return ADAMAH_OK;
}
uint32_t adamah_get_dtype(void) { return g.active_dtype; }

int map_init_dtype(uint32_t id, uint32_t dtype, uint32_t pack_size, uint32_t n_packs, uint32_t group_size) { ADAMAH_API();
  if (!g.initialized || id >= MAX_MAPS || dtype >= DTYPE_COUNT) return ADAMAH_ERR_INVALID;
  if (dtype == DTYPE_BF16 || dtype == DTYPE_Q6) return ADAMAH_ERR_INVALID;
  Map* m = &g.maps[id];
  g.mem_gen++;   // the fills below rewrite device memory without counting as launches
  layout_changed();
  if (m->active) destroy_map(m);
  bool quant = dtype == DTYPE_Q8 || dtype == DTYPE_Q4;
  m->dtype = dtype; m->pack_size = pack_size; m->n_packs = n_packs;
  m->group_size = quant ? group_size : 0;
  m->word_size = dtype == DTYPE_F32 ? 4 : 1;
  m->n_elems = (uint64_t)pack_size * n_packs;
  if (dtype == DTYPE_F32) m->total_bytes = m->n_elems * 4;
  else if (dtype == DTYPE_Q8) m->total_bytes = ((m->n_elems + 3) / 4) * 4;
  else m->total_bytes = ((m->n_elems + 7) / 8) * 4;
  size_t alloc = std::max<uint64_t>(m->total_bytes, 4) + 256;   // tail pad keeps 16-byte row loads in bounds
  if (hipMalloc((void**)&m->buf, alloc) != hipSuccess) { *m = Map(); return ADAMAH_ERR_MEMORY; }
  k_fill_u32<<<fill_grid(alloc / 4), 256, 0, g.stream>>>((uint32_t*)m->buf, 0u, alloc / 4);
  if (quant && group_size > 0) {
    m->n_groups = (m->n_elems + group_size - 1) / group_size;
    size_t ng = std::max<uint64_t>(m->n_groups, 1) + 64;
    if (hipMalloc((void**)&m->qp, ng * sizeof(float2)) != hipSuccess ||
        hipMalloc((void**)&m->d16, ng * sizeof(__half)) != hipSuccess) {
      destroy_map(m);
      return ADAMAH_ERR_MEMORY;
    }
    k_fill_qp<<<fill_grid(ng), 256, 0, g.stream>>>(m->qp, ng);   // default (scale 1, zp 0)
    k_fill_u32<<<fill_grid(ng / 2 + 1), 256, 0, g.stream>>>((uint32_t*)m->d16, 0u, ng / 2);
  }
  m->block16_groups = 0;
  m->active = true;
  return check_launch();
}

int map_init(uint32_t id, uint32_t word_size, uint32_t pack_size, uint32_t n_packs) { ADAMAH_API();
  uint32_t dtype = word_size == 2 ? DTYPE_BF16 : word_size == 1 ? DTYPE_Q8 : DTYPE_F32;
  return map_init_dtype(id, dtype, pack_size, n_packs, 128);
}

int map_destroy(uint32_t id) { ADAMAH_API();
  Map* m = get_map(id);
  if (!m) return ADAMAH_ERR_INVALID;
  g.mem_gen++;
  destroy_map(m);
  return ADAMAH_OK;
}
uint64_t map_size(uint32_t id) { ADAMAH_API(); Map* m = get_map(id); return m ? m->n_packs : 0; }
uint32_t map_get_dtype(uint32_t id) { ADAMAH_API(); Map* m = get_map(id); return m ? m->dtype : 0; }

int map_set_qparams(uint32_t map_id, const float* scales, const float* zps, uint32_t n_groups) { ADAMAH_API();
  Map* m = get_map(map_id);
  if (!m || !m->qp || !scales || !zps) return ADAMAH_ERR_INVALID;
  if ((uint64_t)n_groups > m->n_groups) return ADAMAH_ERR_INVALID;
  layout_changed();   // the storage format of the map's groups (and with it the kernel chosen) may change
  const float off = m->dtype == DTYPE_Q4 ? -8.0f : -128.0f;
  uint64_t prefix = 0;
  bool conform = m->group_size == 32;
  const size_t CH = 1 << 20;
  for (uint64_t g0 = 0; g0 < n_groups; g0 += CH) {
    uint64_t c = std::min<uint64_t>(CH, n_groups - g0);
    float2* sp = (float2*)stage_alloc(c * sizeof(float2));
    uint16_t* hp = (uint16_t*)stage_alloc(c * sizeof(uint16_t));
    if (!sp || !hp) return ADAMAH_ERR_MEMORY;
    for (uint64_t i = 0; i < c; i++) {
      float s = scales[g0 + i], z = zps[g0 + i];
      sp[i] = make_float2(s, z);
      uint16_t hb = f32_to_f16_bits(s);
      hp[i] = hb;
      if (conform) {
        bool ok = ((hb & 0x7C00u) != 0x7C00u) && f16_bits_to_f32(hb) == s && z == off * s;
        if (ok) prefix = g0 + i + 1; else conform = false;
      }
    }
    HIPCHK(hipMemcpyAsync(m->qp + g0, sp, c * sizeof(float2), hipMemcpyHostToDevice, g.stream));
    HIPCHK(hipMemcpyAsync(m->d16 + g0, hp, c * sizeof(uint16_t), hipMemcpyHostToDevice, g.stream));
  }
  // groups beyond n_groups keep their earlier parameters
  if (prefix == n_groups && m->block16_groups > prefix) prefix = m->block16_groups;
  m->block16_groups = prefix;
  return ADAMAH_OK;
}

int adamah_hip_map_layout(uint32_t map_id) { ADAMAH_API();
  Map* m = get_map(map_id);
  if (!m) return ADAMAH_ERR_INVALID;
  return (m->qp && m->n_groups > 0 && m->block16_groups == m->n_groups) ? QL_BLOCK16 : QL_AFFINE;
}

int adamah_kv_cache_fp16(uint32_t map_id, uint32_t start, uint32_t count) { ADAMAH_API();
  Map* m = get_f32_map(map_id);
  if (!m || count == 0 || !in_range(start, count, m->n_elems)) return ADAMAH_ERR_INVALID;
  hipStreamSynchronize(g.stream);
  layout_changed();
  if (m->kv16) hipFree(m->kv16);
  m->kv16 = nullptr;
  if (hipMalloc((void**)&m->kv16, (size_t)count * sizeof(__half) + 256) != hipSuccess) return ADAMAH_ERR_MEMORY;
  m->kv_start = start; m->kv_count = count;
  k_f32_to_kv16<<<fill_grid(count), 256, 0, g.stream>>>((float*)m->buf + start, m->kv16, count);
  return check_launch();
}

// ---- host -> map ---------------------------------------------------------------------------------
static int scatter_impl(Map* m, const uint32_t* locs, uint64_t start_pack, bool contiguous, const void* data,
                        uint32_t n_locs) { ADAMAH_API();
  uint64_t n_vals = (uint64_t)n_locs * m->pack_size;
  if (m->dtype == DTYPE_Q4) {
    if (!m->qp) return ADAMAH_ERR_INVALID;
    float* src = (float*)tmp_dev(0, n_vals * 4);
    uint32_t* dl = nullptr;
    if (!src) return ADAMAH_ERR_MEMORY;
    int r = h2d(src, data, n_vals * 4);
    if (r) return r;
    if (!contiguous) {
      dl = (uint32_t*)tmp_dev(1, (size_t)n_locs * 4);
      if (!dl) return ADAMAH_ERR_MEMORY;
      if ((r = h2d(dl, locs, (size_t)n_locs * 4))) return r;
    }
    k_scatter_q4<<<cdiv(n_vals, 256), 256, 0, g.stream>>>((uint32_t*)m->buf, src, dl, n_locs, m->pack_size,
                                                          m->group_size, start_pack, contiguous ? 0 : 1, m->qp,
                                                          m->n_elems);
    count_launch();
    return check_launch();
  }
  size_t es = m->word_size;
  if (contiguous) {
    int r = h2d(m->buf + start_pack * m->pack_size * es, data, n_vals * es);
    if (r) return r;
    if (m->kv16) {
      uint64_t lo = std::max<uint64_t>(start_pack * m->pack_size, m->kv_start);
      uint64_t hi = std::min<uint64_t>(start_pack * m->pack_size + n_vals, m->kv_start + m->kv_count);
      if (lo < hi) {
        k_f32_to_kv16<<<fill_grid(hi - lo), 256, 0, g.stream>>>((float*)m->buf + lo, m->kv16 + (lo - m->kv_start),
                                                                hi - lo);
        count_launch();
      }
    }
    return check_launch();
  }
  uint8_t* src = (uint8_t*)tmp_dev(0, n_vals * es);
  uint32_t* dl = (uint32_t*)tmp_dev(1, (size_t)n_locs * 4);
  if (!src || !dl) return ADAMAH_ERR_MEMORY;
  int r = h2d(src, data, n_vals * es);
  if (r) return r;
  if ((r = h2d(dl, locs, (size_t)n_locs * 4))) return r;
  if (m->dtype == DTYPE_F32)
    k_scatter_f32<<<cdiv(n_vals, 256), 256, 0, g.stream>>>((float*)m->buf, (const float*)src, dl, n_locs, m->pack_size,
                                                           m->n_elems, m->kv16, m->kv_start, m->kv_count);
  else
    k_scatter_u8<<<cdiv(n_vals, 256), 256, 0, g.stream>>>(m->buf, src, dl, n_locs, m->pack_size, m->n_elems);
  count_launch();
  return check_launch();
}

static bool locs_contiguous(const uint32_t* locs, uint32_t n, uint32_t n_packs, uint32_t* start) {
  if (n == 0 || locs[0] >= n_packs || (uint64_t)locs[0] + n > n_packs) return false;
  for (uint32_t i = 1; i < n; i++)
    if (locs[i] != locs[0] + i) return false;
  *start = locs[0];
  return true;
}

uint64_t map_scatter(uint32_t map_id, const uint32_t* locs, const void* data, uint32_t n_locs) { ADAMAH_API();
  Map* m = get_map(map_id);
  if (!m) return (uint64_t)(int64_t)ADAMAH_ERR_INVALID;
  if (n_locs == 0) return ADAMAH_OK;
  if (!locs || !data) return (uint64_t)(int64_t)ADAMAH_ERR_INVALID;
  uint32_t start = 0;
  bool cont = locs_contiguous(locs, n_locs, m->n_packs, &start);
  return (uint64_t)(int64_t)scatter_impl(m, locs, start, cont, data, n_locs);
}

uint64_t map_scatter_contiguous(uint32_t map_id, uint32_t start_pack, const void* data, uint32_t n_locs) { ADAMAH_API();
  Map* m = get_map(map_id);
  if (!m) return (uint64_t)(int64_t)ADAMAH_ERR_INVALID;
  if (n_locs == 0) return ADAMAH_OK;
  if (!data || start_pack >= m->n_packs || (uint64_t)start_pack + n_locs > m->n_packs)
    return (uint64_t)(int64_t)ADAMAH_ERR_INVALID;
  return (uint64_t)(int64_t)scatter_impl(m, nullptr, start_pack, true, data, n_locs);
}

uint64_t map_scatter_q4_packed_contiguous(uint32_t map_id, uint32_t start_pack, const void* packed, uint32_t n_locs) { ADAMAH_API();
  Map* m = get_map(map_id);
  if (!m) return (uint64_t)(int64_t)ADAMAH_ERR_INVALID;
  if (!packed || n_locs == 0) return ADAMAH_OK;
  if (m->dtype != DTYPE_Q4 || m->pack_size != 1 || start_pack >= m->n_packs ||
      (uint64_t)start_pack + n_locs > m->n_packs || (start_pack & 1u) || (n_locs & 1u))
    return (uint64_t)(int64_t)ADAMAH_ERR_INVALID;
  return (uint64_t)(int64_t)h2d(m->buf + start_pack / 2, packed, n_locs / 2);
}

uint64_t map_gather(uint32_t map_id, const uint32_t* locs, void* data, uint32_t n_locs) { ADAMAH_API();
  Map* m = get_map(map_id);
  if (!m) return (uint64_t)(int64_t)ADAMAH_ERR_INVALID;
  if (n_locs == 0) return ADAMAH_OK;
  if (!locs || !data) return (uint64_t)(int64_t)ADAMAH_ERR_INVALID;
  size_t pack_bytes = (size_t)m->word_size * m->pack_size;
  uint32_t start = 0;
  if (locs_contiguous(locs, n_locs, m->n_packs, &start) && (start + (uint64_t)n_locs) * pack_bytes <= m->total_bytes)
    return (uint64_t)(int64_t)d2h(data, m->buf + (size_t)start * pack_bytes, (size_t)n_locs * pack_bytes);
  uint32_t* dl = (uint32_t*)tmp_dev(1, (size_t)n_locs * 4);
  uint8_t* dst = (uint8_t*)tmp_dev(0, (size_t)n_locs * pack_bytes);
  if (!dl || !dst) return (uint64_t)(int64_t)ADAMAH_ERR_MEMORY;
  int r = h2d(dl, locs, (size_t)n_locs * 4);
  if (r) return (uint64_t)(int64_t)r;
  if (m->dtype == DTYPE_F32)
    k_gather_f32<<<cdiv((uint64_t)n_locs * m->pack_size, 256), 256, 0, g.stream>>>(
        (const float*)m->buf, (float*)dst, dl, n_locs, m->pack_size, m->n_elems);
  else {
    if (m->pack_size != 1) return (uint64_t)(int64_t)ADAMAH_ERR_INVALID;
    k_gather_u8<<<cdiv(n_locs, 256), 256, 0, g.stream>>>(m->buf, dst, dl, n_locs, m->total_bytes);
  }
  count_launch();
  if ((r = check_launch())) return (uint64_t)(int64_t)r;
  return (uint64_t)(int64_t)d2h(data, dst, (size_t)n_locs * pack_bytes);
}

// ---- handles ---------------------------------------------------------------------------------------
uint64_t map_upload_dev(uint32_t handle, const void* data, uint32_t n_bytes) {
  // a new handle cannot be an operand of anything queued; rewriting an existing one can
  if (handle != 0) { ADAMAH_API(); plan_graph_handle_rewritten(handle); }
  if (!g.initialized || !data || n_bytes == 0) return 0;
  uint32_t id = handle;
  if (id == 0) {
    id = res_alloc(n_bytes);
    if (id == 0) return 0;
  }
  Res* r = get_res(id);
  if (!r || r->size_bytes != n_bytes) return 0;   // re-upload must keep the byte size (adamah.c:3601-3608)
  note_host(r, data, n_bytes);
  if (h2d(r->dptr, data, n_bytes) != ADAMAH_OK) return 0;
  return (uint64_t)id;
}

int map_download_dev(uint32_t handle, void* data, uint32_t n_bytes) { ADAMAH_API();
  if (!g.initialized || !data || n_bytes == 0) return ADAMAH_ERR_INVALID;
  Res* r = get_res(handle);
  if (!r || n_bytes > r->size_bytes) return ADAMAH_ERR_INVALID;
  return d2h(data, r->dptr, n_bytes);
}

uint64_t map_gather_dev(uint32_t map_id, uint32_t locs_handle, uint32_t n_locs) { ADAMAH_API();
  Map* m = get_map(map_id);
  if (!m || n_locs == 0) return 0;
  const uint32_t* locs = res_u32(locs_handle, n_locs);
  if (!locs) return 0;
  if (m->dtype != DTYPE_F32 && !m->qp) return 0;
  uint64_t n_vals = (uint64_t)n_locs * m->pack_size;
  if (n_vals * 4 > 0xFFFFFFFFull) return 0;
  // Results are never released individually (as in the reference, whose table ends after 2048).  A decode loop
  // gathers one embedding row per token and a chunked prefill a block of rows per chunk, so only the latest results
  // of a size class are kept: the storage and id of the class's oldest is handed out again, and handles and arena
  // stop growing.  A caller that still holds the id of a result older than the class limit sees the newer contents.
  const uint32_t need = (uint32_t)(n_vals * 4);
  const uint32_t cls = gather_class(need);
  std::deque<uint32_t>& ring = g_gather_ring[cls];
  uint32_t id = 0;
  if (ring.size() >= gather_class_limit(cls)) {
    Res* old = get_res(ring.front());
    if (old && old->cap_bytes >= need) {
      id = ring.front();
      old->size_bytes = need; old->host.clear(); old->host_valid = false; old->contig = false;
    }
    ring.pop_front();
  }
  if (id == 0) {
    const uint64_t cap = (uint64_t)1 << cls;
    id = res_alloc(cap > 0xFFFFFFFFull ? need : (uint32_t)cap);
    if (id == 0) return 0;
    g.res[id].size_bytes = need;
  }
  ring.push_back(id);
  float* dst = (float*)g.res[id].dptr;
  if (m->dtype == DTYPE_F32)
    k_gather_f32<<<cdiv(n_vals, 256), 256, 0, g.stream>>>((const float*)m->buf, dst, locs, n_locs, m->pack_size,
                                                          m->n_elems);
  else
    k_gather_q<<<cdiv(n_vals, 256), 256, 0, g.stream>>>(m->buf, dst, locs, n_locs, m->pack_size, m->group_size, m->qp,
                                                        m->n_elems, m->dtype == DTYPE_Q4);
  count_launch();
  if (check_launch()) return 0;
  return (uint64_t)id;
}

uint64_t map_scatter_dev(uint32_t map_id, uint32_t locs_handle, uint32_t n_locs, uint32_t src_handle) { ADAMAH_API();
  Map* m = get_f32_map(map_id);
  if (!m || n_locs == 0) return 0;
  const uint32_t* locs = res_u32(locs_handle, n_locs);
  const uint32_t* src = res_u32(src_handle, (uint64_t)n_locs * m->pack_size);
  if (!locs || !src) return 0;
  uint64_t n_vals = (uint64_t)n_locs * m->pack_size;
  k_scatter_f32<<<cdiv(n_vals, 256), 256, 0, g.stream>>>((float*)m->buf, (const float*)src, locs, n_locs, m->pack_size,
                                                         m->n_elems, m->kv16, m->kv_start, m->kv_count);
  count_launch();
  check_launch();
  return 0;
}

// ---- stopwatch -------------------------------------------------------------------------------------
int adamah_hip_timer_begin(void) { ADAMAH_API();
  if (!g.initialized) return ADAMAH_ERR_INVALID;
  return hipEventRecord(g.timer_ev[0], g.stream) == hipSuccess ? ADAMAH_OK : ADAMAH_ERR_BACKEND;
}
float adamah_hip_timer_end(void) { ADAMAH_API();
  if (!g.initialized) return -1.0f;
  float ms = -1.0f;
  if (hipEventRecord(g.timer_ev[1], g.stream) != hipSuccess) return -1.0f;
  if (hipEventSynchronize(g.timer_ev[1]) != hipSuccess) return -1.0f;
  if (hipEventElapsedTime(&ms, g.timer_ev[0], g.timer_ev[1]) != hipSuccess) return -1.0f;
  return ms;
}

// ---- decode plan (adamah.c:10244-10398): a recorded op list replayed with runtime pos / seq_len ---
#define RT_POS 0xFFFFFFFEu
#define RT_SEQ 0xFFFFFFFDu
int adamah_register_decode_plan(uint32_t plan_id, const AdamahDecodePlanOp* ops, uint32_t n_ops) { ADAMAH_API();
  if (plan_id >= MAX_PLANS || n_ops > MAX_PLAN_OPS || (n_ops > 0 && !ops)) return ADAMAH_ERR_INVALID;
  g.plans[plan_id].resize(n_ops);
  if (n_ops) memcpy(g.plans[plan_id].data(), ops, sizeof(PlanOp) * n_ops);
  g.plan_active[plan_id] = true;
  plan_graph_reset(plan_id);
  return ADAMAH_OK;
}
void adamah_clear_decode_plan(uint32_t plan_id) { ADAMAH_API();
  if (plan_id >= MAX_PLANS) return;
  g.plans[plan_id].clear();
  g.plan_active[plan_id] = false;
  plan_graph_reset(plan_id);
}
// The op list of a plan with pos / seq_len substituted, through the ordinary entry points.
static int replay_plan(uint32_t plan_id, uint32_t pos, uint32_t seq_len) {
  int ret = ADAMAH_OK;
  for (const PlanOp& op : g.plans[plan_id]) {
    auto rs = [&](uint32_t v) { return v == RT_POS ? pos : v == RT_SEQ ? seq_len : v; };
    uint32_t u0 = rs(op.u0), u1 = rs(op.u1), u2 = rs(op.u2), u3 = rs(op.u3), u4 = rs(op.u4);
    switch (op.kind) {
      case 0: ret = ADAMAH_OK; break;
      case 1: ret = adamah_fusion_flush(); break;
      case 2: adamah_fusion_enable((int)u0); ret = ADAMAH_OK; break;
      case 10: ret = map_op1_dev(op.map_id, op.op_code, op.h0, op.h1, u0); break;
      case 11: ret = map_op2_dev(op.map_id, op.op_code, op.h0, op.h1, op.h2, u0); break;
      case 12: ret = map_rmsnorm_dev(op.map_id, op.h0, op.h1, op.h2, u0, u1, op.f0); break;
      case 13: ret = map_rmsnorm_x_dev(op.map_id, op.map_id2, op.h0, op.h1, op.h2, u0, u1, op.f0); break;
      case 14: ret = map_rmsnorm_add_dev(op.map_id, op.h0, op.h1, op.h2, op.h3, u0, u1, op.f0); break;
      case 15: ret = map_rope_dev(op.map_id, op.h0, op.h1, u0, u1, u2, u3, op.f0); break;
      case 16: ret = map_matmul_t_dev(op.map_id, op.h0, op.h1, op.h2, u0, u1, u2, u3); break;
      case 17: ret = map_matmul_t_x_dev(op.map_id, op.map_id2, op.h0, op.h1, op.h2, u0, u1, u2, u3); break;
      case 18: ret = map_matmul_x_dev(op.map_id, op.map_id2, op.h0, op.h1, op.h2, u0, u1, u2, u3); break;
      case 19: ret = map_matmul_t_xq4_dev(op.map_id, op.map_id2, op.h0, op.h1, op.h2, u0, u1, u2, u3); break;
      case 20: ret = map_matmul_xq4_dev(op.map_id, op.map_id2, op.h0, op.h1, op.h2, u0, u1, u2, u3); break;
      case 21: ret = map_matmul_t_xq8_dev(op.map_id, op.map_id2, op.h0, op.h1, op.h2, u0, u1, u2, u3); break;
      case 22: ret = map_matmul_xq8_dev(op.map_id, op.map_id2, op.h0, op.h1, op.h2, u0, u1, u2, u3); break;
      case 23: ret = map_qk_norm_rope_x_dev(op.map_id, op.map_id2, op.h0, op.h1, op.h2, op.h3, op.h4, u0, u1, u2, u3,
                                            u4, op.f0); break;
      case 24: ret = map_row_copy_offset_dev(op.map_id, op.h0, op.h1, u0, u1, u2); break;
      case 25: ret = map_attn_softmax_value_dev(op.map_id, op.h0, op.h1, op.h2, u0, u1, u2, op.f0, op.f1); break;
      // fused projections (adamah.c:10318-10334): the seventh handle of the Q/K/V form travels in u0
      case 26: ret = map_fused_qkv_t_xq4_dev(op.map_id, op.map_id2, op.h0, op.h1, op.h2, op.h3, op.h4, op.h5, u0, u1, u2, u3, u4); break;
      case 27: ret = map_fused_gateup_t_xq4_dev(op.map_id, op.map_id2, op.h0, op.h1, op.h2, op.h3, op.h4, u0, u1, u2); break;
      case 28: ret = map_fused_qkv_t_xq8_dev(op.map_id, op.map_id2, op.h0, op.h1, op.h2, op.h3, op.h4, op.h5, u0, u1, u2, u3, u4); break;
      case 29: ret = map_fused_gateup_t_xq8_dev(op.map_id, op.map_id2, op.h0, op.h1, op.h2, op.h3, op.h4, u0, u1, u2); break;
      case 30: ret = map_fused_gateup_act_t_xq8_dev(op.map_id, op.map_id2, op.h0, op.h1, op.h2, op.h3, u0, u1); break;
      default: ret = ADAMAH_ERR_INVALID; break;
    }
    if (ret != ADAMAH_OK) break;
  }
  return ret;
}

// Graph replay of a plan (on unless ADAMAH_PLAN_GRAPH=0).  A decode loop calls the plan with pos, pos + 1, ...: after
// serving step (pos, seq_len) the library records the launches of step (pos + 1, seq_len + 1) into a HIP graph
// -- stream capture of the same entry points, nothing executes -- while the device is still busy with the
// current step, and the next call launches that graph if it asks for exactly that step (anything else is
// replayed the ordinary way).  Kernels of a graph start ~0.7 us sooner after their predecessor than
// stream launches do.  Three executable graphs take turns and each launch is followed by an event: before a graph is
// updated (its kernels' arguments are rewritten in place) the host waits for that graph's last launch to have
// finished.  With three, a caller that issues step n + 1 before it has seen the result of step n (one step of
// lookahead) never waits: the graph being rewritten last ran step n - 1.
// A plan whose ops copy from the host (tables of operand bases) or fail to capture is left to the
// ordinary replay for good.
#define PLAN_EXECS 3
struct PlanGraph {
  hipGraphExec_t exec[PLAN_EXECS] = {nullptr, nullptr, nullptr};
  hipEvent_t done[PLAN_EXECS] = {nullptr, nullptr, nullptr};   // recorded behind the last launch of exec[i]
  bool launched[PLAN_EXECS] = {false, false, false};
  int cur = 0;               // exec[cur] holds the recorded step when ready
  bool ready = false, disabled = false;
  uint32_t pos = 0, seq = 0, n_nodes = 0;
  uint32_t last_pos = 0xFFFFFFFFu, last_seq = 0xFFFFFFFFu;   // the previous call's step
  int eager_steps = 0;
  uint32_t n_graph = 0, n_update = 0, n_inst = 0;   // steps served by a graph, in-place updates, instantiations
  uint64_t gen = 0;          // g.layout_gen when the graph was recorded: it holds device pointers and offsets by value
  std::vector<uint32_t> handles;   // sorted ids of the handles the plan's ops name (their contents are baked in too)
  std::vector<PendOp> tail;        // the recorded step's last queued norms: not in the graph, queued again behind it
};
static PlanGraph g_pg[MAX_PLANS];

static bool plan_graphs_on() {
  const char* e = getenv("ADAMAH_PLAN_GRAPH");
  return !(e && e[0] == '0');
}

static void plan_graph_drop(PlanGraph& pg, bool for_good) {
  for (int i = 0; i < PLAN_EXECS; i++) {
    if (pg.launched[i] && pg.done[i]) hipEventSynchronize(pg.done[i]);
    pg.launched[i] = false;
    if (pg.exec[i]) hipGraphExecDestroy(pg.exec[i]);
    pg.exec[i] = nullptr;
  }
  pg.ready = false;
  if (for_good) pg.disabled = true;
}

// A plan usually ends in the norms that the caller's next op (the LM head) folds into its own launch.  They stay in
// the queue when the rest of the step is launched (or recorded), so that a step from a graph leaves the queue as an
// ordinary replay does.
static std::vector<PendOp> take_trailing_norms() {
  size_t n = g.pend.size(), k = 0;
  while (k < 2 && k < n && g.pend[n - 1 - k].kind == PK_RMSNORM) k++;
  std::vector<PendOp> tail(g.pend.end() - (long)k, g.pend.end());
  g.pend.resize(n - k);
  return tail;
}

static void plan_graph_record(uint32_t plan_id, uint32_t pos, uint32_t seq_len) {
  PlanGraph& pg = g_pg[plan_id];
  pg.ready = false;
  const uint64_t gen0 = g.mem_gen, lay0 = g.layout_gen;
  const Stats saved = g.stats;
  if (hipStreamBeginCapture(g.stream, hipStreamCaptureModeThreadLocal) != hipSuccess) { (void)hipGetLastError(); plan_graph_drop(pg, true); return; }
  int r = replay_plan(plan_id, pos, seq_len);
  pg.tail = take_trailing_norms();
  flush_pending();
  hipGraph_t graph = nullptr;
  const hipError_t e = hipStreamEndCapture(g.stream, &graph);
  const uint32_t n_nodes = (uint32_t)(g.stats.dispatch - saved.dispatch);
  g.stats = saved;                                   // nothing ran: the launches are counted when the graph does
  if (r != ADAMAH_OK || e != hipSuccess || !graph || g.mem_gen != gen0 || g.layout_gen != lay0 || n_nodes == 0) {
    if (graph) hipGraphDestroy(graph);
    (void)hipGetLastError();
    plan_graph_drop(pg, true);
    return;
  }
  gemm_act_forget();   // the note "these rows are converted" was taken while nothing ran
  const int slot = (pg.cur + 1) % PLAN_EXECS;
  if (pg.launched[slot]) {                           // its kernels read their arguments from the graph's own memory
    hipEventSynchronize(pg.done[slot]);
    pg.launched[slot] = false;
  }
  if (pg.exec[slot]) {
    hipGraphNode_t bad = nullptr;
    hipGraphExecUpdateResult res;
    if (hipGraphExecUpdate(pg.exec[slot], graph, &bad, &res) != hipSuccess) {   // another launch shape (e.g. one more slice)
      (void)hipGetLastError();
      hipGraphExecDestroy(pg.exec[slot]);
      pg.exec[slot] = nullptr;
    } else pg.n_update++;
  }
  const bool fresh = !pg.exec[slot];
  if (fresh) pg.n_inst++;
  if (!pg.exec[slot] && hipGraphInstantiate(&pg.exec[slot], graph, nullptr, nullptr, 0) != hipSuccess) {
    (void)hipGetLastError();
    pg.exec[slot] = nullptr;
    hipGraphDestroy(graph);
    plan_graph_drop(pg, true);
    return;
  }
  hipGraphDestroy(graph);
  pg.cur = slot; pg.ready = true; pg.pos = pos; pg.seq = seq_len; pg.n_nodes = n_nodes; pg.gen = g.layout_gen;
}

// The graph of a plan was recorded from the host copies of its handles: rewriting one of them makes it stale.
static void plan_graph_handle_rewritten(uint32_t handle) {
  for (int i = 0; i < MAX_PLANS; i++) {
    PlanGraph& pg = g_pg[i];
    if (pg.ready && std::binary_search(pg.handles.begin(), pg.handles.end(), handle)) pg.ready = false;
  }
}

static void plan_graph_reset(uint32_t plan_id) {
  const PlanGraph& o = g_pg[plan_id];
  if (getenv("ADAMAH_DEBUG") && (o.n_graph || o.eager_steps))
    fprintf(stderr, "[adamah] plan %u: %u steps from graphs, %d replayed, %u updates, %u instantiations, %u nodes%s\n", plan_id,
            o.n_graph, o.eager_steps, o.n_update, o.n_inst, o.n_nodes, o.disabled ? ", graphs given up" : "");
  hipStreamSynchronize(g.stream);
  plan_graph_drop(g_pg[plan_id], false);
  for (int i = 0; i < PLAN_EXECS; i++) if (g_pg[plan_id].done[i]) hipEventDestroy(g_pg[plan_id].done[i]);
  g_pg[plan_id] = PlanGraph();
}

int adamah_decode_step(uint32_t plan_id, uint32_t pos, uint32_t seq_len) {
  if (plan_id >= MAX_PLANS) return ADAMAH_ERR_INVALID;
  if (!g.plan_active[plan_id]) return ADAMAH_ERR_NOT_FOUND;
  bool opened = g.batch_depth == 0;
  if (opened) batch_begin();
  int ret;
  PlanGraph& pg = g_pg[plan_id];
  if (!plan_graphs_on() || pg.disabled) ret = replay_plan(plan_id, pos, seq_len);
  else {
    flush_pending();                                 // what was queued before the plan runs ahead of it
    if (pg.ready && pg.gen != g.layout_gen) pg.ready = false;   // a map or scratch buffer moved since the recording
    if (pg.handles.empty()) {
      for (const PlanOp& op : g.plans[plan_id]) {
        for (uint32_t h : {op.h0, op.h1, op.h2, op.h3, op.h4, op.h5}) if (h) pg.handles.push_back(h);
        if ((op.kind == 26 || op.kind == 28) && op.u0) pg.handles.push_back(op.u0);   // their seventh handle
      }
      std::sort(pg.handles.begin(), pg.handles.end());
      pg.handles.erase(std::unique(pg.handles.begin(), pg.handles.end()), pg.handles.end());
    }
    if (pg.ready && pg.pos == pos && pg.seq == seq_len) {
      ret = hipGraphLaunch(pg.exec[pg.cur], g.stream) == hipSuccess ? ADAMAH_OK : ADAMAH_ERR_BACKEND;
      if (!pg.done[pg.cur] && hipEventCreateWithFlags(&pg.done[pg.cur], hipEventDisableTiming) != hipSuccess) ret = ADAMAH_ERR_BACKEND;
      if (ret == ADAMAH_OK && hipEventRecord(pg.done[pg.cur], g.stream) != hipSuccess) ret = ADAMAH_ERR_BACKEND;
      pg.launched[pg.cur] = ret == ADAMAH_OK;
      count_launch((int)pg.n_nodes);
      pg.n_graph++;
      g.pend.insert(g.pend.end(), pg.tail.begin(), pg.tail.end());
    } else {
      ret = replay_plan(plan_id, pos, seq_len);
      pg.eager_steps++;
    }
    // the step's launches are out (but for its last norms, which wait for the caller's next op as they would without
    // graphs); the recording below must find the queue without them
    const std::vector<PendOp> tail = take_trailing_norms();
    flush_pending();
    // The first steps run the ordinary way (scratch buffers reach their sizes).  Then the next step is recorded, but
    // only for a caller that is walking through positions (this call continued the previous one): a plan that is
    // called with the same step again and again (a benchmark loop) would pay for a recording it never uses.
    const bool walking = pg.last_pos != 0xFFFFFFFFu && pos == pg.last_pos + 1u && seq_len == pg.last_seq + 1u;
    pg.last_pos = pos; pg.last_seq = seq_len;
    if (ret == ADAMAH_OK && pg.eager_steps >= 2 && walking && pos != 0xFFFFFFFFu && seq_len != 0xFFFFFFFFu)
      plan_graph_record(plan_id, pos + 1, seq_len + 1);
    else pg.ready = false;
    g.pend.insert(g.pend.end(), tail.begin(), tail.end());
  }
  if (opened) batch_end();
  if (ret == ADAMAH_OK && g.pend.empty()) ret = take_deferred_err();
  return ret;
}

}  // extern "C"
