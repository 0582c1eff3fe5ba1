// Sampling tail on logits resident in a float32 map: top-k selection, temperature / top-p
// renormalisation of a short candidate list, index resolution, categorical draw, repetition penalty.
//
// Reference: shaders/src/f32/map_topk.comp, map_topp.comp, map_resolve_idx.comp,
// map_sample_categorical.comp, map_repeat_penalty.comp; dispatchers adamah.c:6787-6873 (repeat
// penalty), 6978-7093 (top-k), 7095-7208 (top-p), 7210-7284 (resolve), 7286-7370 (categorical).
// Limits as there: k, n <= 64 for top-p / categorical / repeat penalty ids, k <= 64 for top-k.
// These are tiny latency-bound kernels; the serial parts run in one lane in the order the shaders
// use, so the float32 results match a sequential evaluation.  Every location read from a handle is
// checked against the map size before it is used.
#include "common.h"
#include "gemv_common.h"
#include <algorithm>
#include "../../include/adamah_hip.h"

namespace adamah {

#define SMP_MAX 64u
#define SMP_INVALID 0xffffffffu
#define SMP_NEG_INF (-3.402823466e+38f)

__device__ __forceinline__ bool smp_better(float cv, uint32_t ci, float bv, uint32_t bi) {
  if (bi == SMP_INVALID) return true;
  if (ci == SMP_INVALID) return false;
  return cv > bv || (cv == bv && ci < bi);
}

// Top-k over n candidates: the k best in the order (value descending, candidate index ascending); NaN
// counts as the lowest value; rounds past n store index 0 and the lowest value.  The order is strict,
// so round t takes the best candidate that ranks after the pick of round t - 1 and no list of taken
// candidates is needed.  A workgroup keeps a chunk of 4096 candidates in registers (16 per thread,
// one coalesced pass over the handle and the map); one chunk writes the result itself, several chunks
// leave their own k best in a scratch list that a second launch merges the same way.
#define TOPK_CHUNK 4096u
#define TOPK_PER_THREAD 16u

struct TopkPick { float v; uint32_t i; };

// best (value, index) over the workgroup, the same in every thread
__device__ __forceinline__ TopkPick topk_block_best(float bv, uint32_t bi, float* sv, uint32_t* si) {
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) {
    const float ov = __shfl_xor(bv, o, 64);
    const uint32_t oi = __shfl_xor(bi, o, 64);
    if (smp_better(ov, oi, bv, bi)) { bv = ov; bi = oi; }
  }
  const uint32_t lane = threadIdx.x & 63u, wave = threadIdx.x >> 6;
  __syncthreads();                       // sv / si may still be read from the previous round
  if (lane == 0) { sv[wave] = bv; si[wave] = bi; }
  __syncthreads();
  bv = sv[0]; bi = si[0];
#pragma unroll
  for (int w = 1; w < 4; w++)
    if (smp_better(sv[w], si[w], bv, bi)) { bv = sv[w]; bi = si[w]; }
  return {bv, bi};
}

__device__ __forceinline__ bool topk_after(float pv, uint32_t pi, float v, uint32_t i) {
  return pv > v || (pv == v && pi < i);
}

__global__ void __launch_bounds__(256)
k_topk_chunk(float* data, const uint32_t* __restrict__ ls, const uint32_t* __restrict__ li, const uint32_t* __restrict__ lv,
             uint32_t n, uint32_t k, uint64_t n_elems, float* part_v, uint32_t* part_i) {
  __shared__ float sv[4];
  __shared__ uint32_t si[4];
  const uint32_t tid = threadIdx.x, c0 = blockIdx.x * TOPK_CHUNK;
  const bool single = gridDim.x == 1u;
  float v[TOPK_PER_THREAD];
#pragma unroll
  for (uint32_t u = 0; u < TOPK_PER_THREAD; u++) {
    const uint32_t i = c0 + u * 256u + tid;
    float x = SMP_NEG_INF;
    if (i < n) { const uint32_t l = ls[i]; if (l < n_elems) x = data[l]; }
    v[u] = x != x ? SMP_NEG_INF : x;
  }
  float pv = 0.f;
  uint32_t pi = SMP_INVALID;
  for (uint32_t t = 0; t < k; t++) {
    float bv = SMP_NEG_INF;
    uint32_t bi = SMP_INVALID;
    if (t == 0u || pi != SMP_INVALID) {
#pragma unroll
      for (uint32_t u = 0; u < TOPK_PER_THREAD; u++) {
        const uint32_t i = c0 + u * 256u + tid;
        if (i < n && (t == 0u || topk_after(pv, pi, v[u], i)) && smp_better(v[u], i, bv, bi)) { bv = v[u]; bi = i; }
      }
    }
    const TopkPick b = topk_block_best(bv, bi, sv, si);
    pv = b.v; pi = b.i;
    if (tid == 0) {
      if (single) {
        if (li[t] < n_elems) data[li[t]] = (float)(b.i == SMP_INVALID ? 0u : b.i);
        if (lv[t] < n_elems) data[lv[t]] = b.i == SMP_INVALID ? SMP_NEG_INF : b.v;
      } else {
        part_v[blockIdx.x * k + t] = b.v;
        part_i[blockIdx.x * k + t] = b.i;
      }
    }
  }
}

// merge of the chunks' lists: n2 = chunks * k (value, candidate index) pairs, invalid entries skipped
__global__ void __launch_bounds__(256)
k_topk_merge(float* data, const float* __restrict__ part_v, const uint32_t* __restrict__ part_i,
             const uint32_t* __restrict__ li, const uint32_t* __restrict__ lv, uint32_t n2, uint32_t k, uint64_t n_elems) {
  __shared__ float sv[4];
  __shared__ uint32_t si[4];
  const uint32_t tid = threadIdx.x;
  float pv = 0.f;
  uint32_t pi = SMP_INVALID;
  for (uint32_t t = 0; t < k; t++) {
    float bv = SMP_NEG_INF;
    uint32_t bi = SMP_INVALID;
    if (t == 0u || pi != SMP_INVALID) {
      for (uint32_t j = tid; j < n2; j += 256u) {
        const uint32_t i = part_i[j];
        const float x = part_v[j];
        if (i != SMP_INVALID && (t == 0u || topk_after(pv, pi, x, i)) && smp_better(x, i, bv, bi)) { bv = x; bi = i; }
      }
    }
    const TopkPick b = topk_block_best(bv, bi, sv, si);
    pv = b.v; pi = b.i;
    if (tid == 0) {
      if (li[t] < n_elems) data[li[t]] = (float)(b.i == SMP_INVALID ? 0u : b.i);
      if (lv[t] < n_elems) data[lv[t]] = b.i == SMP_INVALID ? SMP_NEG_INF : b.v;
    }
  }
}


// Top-k of 4096 < n <= 40960 candidates in one launch: radix selection instead of k rounds.  A candidate's place in
// the strict order (value descending, index ascending) is the 48-bit key (orderable value bits, 0xFFFF - index); five
// histogram passes over its digits (11, 11, 10 bits of the value, then 8, 8 of the index, top down) find the key of the k-th best -- each pass counts
// the candidates that agree with the digits fixed so far, a suffix scan over the bins finds the bin the k-th falls in --
// and everything at or above that key is gathered and put in order by counting.  One workgroup of 1024 threads, the
// values in registers (at most 40 per thread).  Same results as the rounds (tests/test_gpu_sampling.py); the partial
// lists of the sampled LM head (40960 candidates, k = 40): 145 -> 20 us.
#define TSEL_THREADS 1024u
#define TSEL_PER 40u
__global__ void __launch_bounds__(1024)
k_topk_select(float* data, const uint32_t* __restrict__ ls, const uint32_t* __restrict__ li, const uint32_t* __restrict__ lv,
              uint32_t n, uint32_t k, uint64_t n_elems) {
  __shared__ uint32_t hist[2048];
  __shared__ uint32_t wtot[16];
  __shared__ uint32_t sel_bin, sel_rem, n_win;
  __shared__ float win_v[SMP_MAX];
  __shared__ uint32_t win_i[SMP_MAX];
  const uint32_t tid = threadIdx.x, lane = tid & 63u, wave = tid >> 6;
  const uint32_t per = (n + TSEL_THREADS - 1u) / TSEL_THREADS;
  uint32_t vk[TSEL_PER];   // orderable value bits of candidate u * 1024 + tid
#pragma unroll
  for (uint32_t u0 = 0; u0 < TSEL_PER; u0 += 8u) {   // eight at a time: the loads' temporaries stay within the budget
#pragma unroll
    for (uint32_t u = u0; u < u0 + 8u; u++) {
      const uint32_t i = u * TSEL_THREADS + tid;
      float x = SMP_NEG_INF;
      if (u < per && i < n) { const uint32_t l = ls[i]; if (l < n_elems) x = data[l]; }
      x = x != x ? SMP_NEG_INF : x;
      const uint32_t b = __float_as_uint(x);
      vk[u] = (b & 0x80000000u) ? ~b : (b | 0x80000000u);
    }
    __builtin_amdgcn_sched_barrier(0);
  }
  const uint32_t kk = min(k, n);
  const uint32_t inv0 = 0xFFFFu - tid;          // index digits of candidate u: inv0 - u * 1024 (lower index = larger)
  uint32_t prefix = 0, mask = 0, iprefix = 0, imask = 0;
  uint32_t remaining = kk;
#pragma unroll 1
  for (uint32_t pass = 0; pass < 5u; pass++) {
    const bool on_idx = pass >= 3u;             // passes 0..2: value bits 31..21, 20..10, 9..0; 3, 4: index bits 15..8, 7..0
    const uint32_t sh = pass == 0u ? 21u : pass == 1u ? 10u : pass == 3u ? 8u : 0u;
    const uint32_t bm = pass < 2u ? 2047u : pass == 2u ? 1023u : 255u;
    hist[2u * tid] = 0u; hist[2u * tid + 1u] = 0u;
    __syncthreads();
    uint32_t inv = inv0, idx = tid;
    asm volatile("" : "+v"(inv), "+v"(idx));   // per pass, so that the 40 index digits are not all kept in registers
#pragma unroll
    for (uint32_t u = 0; u < TSEL_PER; u++) {
      if (u < per && idx + u * TSEL_THREADS < n) {
        const uint32_t iv = inv - u * TSEL_THREADS;
        const bool in = on_idx ? (vk[u] == prefix && (iv & imask) == iprefix) : ((vk[u] & mask) == prefix);
        if (in) atomicAdd(&hist[((on_idx ? iv : vk[u]) >> sh) & bm], 1u);
      }
    }
    __syncthreads();
    // suffix sums over the bins (two per thread), top down: the bin in which the count reaches `remaining`
    const uint32_t h0 = hist[2u * tid], h1 = hist[2u * tid + 1u], own = h0 + h1;
    uint32_t suf = own;   // inclusive suffix sum within the wave
#pragma unroll
    for (int o = 1; o < 64; o <<= 1) {
      const uint32_t t = __shfl_down(suf, o, 64);
      if (lane + (uint32_t)o < 64u) suf += t;
    }
    if (lane == 0u) wtot[wave] = suf;
    __syncthreads();
    for (uint32_t w = wave + 1u; w < 16u; w++) suf += wtot[w];
    const uint32_t above = suf - own;
    if (above < remaining && remaining <= suf) {
      if (above + h1 >= remaining) { sel_bin = 2u * tid + 1u; sel_rem = remaining - above; }
      else { sel_bin = 2u * tid; sel_rem = remaining - above - h1; }
    }
    __syncthreads();
    if (on_idx) { iprefix |= sel_bin << sh; imask |= bm << sh; }
    else { prefix |= sel_bin << sh; mask |= bm << sh; }
    remaining = sel_rem;
  }
  // (prefix, iprefix) is now the key of the kk-th best: everything at or above it wins
  if (tid == 0) n_win = 0u;
  __syncthreads();
#pragma unroll
  for (uint32_t u = 0; u < TSEL_PER; u++) {
    const uint32_t i = u * TSEL_THREADS + tid;
    if (u < per && i < n && (vk[u] > prefix || (vk[u] == prefix && inv0 - u * TSEL_THREADS >= iprefix))) {
      const uint32_t slot = atomicAdd(&n_win, 1u);
      if (slot < SMP_MAX) {
        const uint32_t b = (vk[u] & 0x80000000u) ? (vk[u] & 0x7FFFFFFFu) : ~vk[u];
        win_v[slot] = __uint_as_float(b); win_i[slot] = i;
      }
    }
  }
  __syncthreads();
  const uint32_t cnt = min(n_win, kk);
  if (tid < k) {
    if (tid < cnt) {
      const float v = win_v[tid];
      const uint32_t i = win_i[tid];
      uint32_t rank = 0;
      for (uint32_t j = 0; j < cnt; j++) rank += (win_v[j] > v || (win_v[j] == v && win_i[j] < i)) ? 1u : 0u;
      if (li[rank] < n_elems) data[li[rank]] = (float)i;
      if (lv[rank] < n_elems) data[lv[rank]] = v;
    } else {   // fewer candidates than k: the rounds past the last one
      if (li[tid] < n_elems) data[li[tid]] = 0.0f;
      if (lv[tid] < n_elems) data[lv[tid]] = SMP_NEG_INF;
    }
  }
}

static float* g_topk_part = nullptr;   // chunks * k values, then chunks * k candidate indices
static size_t g_topk_part_cap = 0;     // entries

void sampling_release() {
  if (g_topk_part) hipFree(g_topk_part);
  g_topk_part = nullptr;
  g_topk_part_cap = 0;
}

// softmax(logits / temperature) over n <= 64 candidates in list order, cut after the first prefix
// whose mass reaches top_p, renormalised over the kept prefix.
__global__ void __launch_bounds__(64)
k_topp(float* data, const uint32_t* __restrict__ ls, const uint32_t* __restrict__ ld, uint32_t n, float temperature,
       float top_p, uint64_t n_elems) {
  __shared__ float lg[SMP_MAX], pr[SMP_MAX];
  const uint32_t tid = threadIdx.x;
  lg[tid] = SMP_NEG_INF;
  pr[tid] = 0.f;
  if (tid < n) {
    float v = ls[tid] < n_elems ? data[ls[tid]] : SMP_NEG_INF;
    if (isnan(v) || isinf(v)) v = SMP_NEG_INF;
    lg[tid] = v;
  }
  __syncthreads();
  // One lane per candidate for the exponentials, the divisions and the stores; the sums run over the candidates in
  // order in lane 0, as the reference's single invocation adds them up (same values, same order, same bits).
  __shared__ float s_sum, s_ks;
  __shared__ uint32_t s_keep;
  auto put = [&](uint32_t i, float v) { if (ld[i] < n_elems) data[ld[i]] = v; };
  const float temp = fmaxf(temperature, 1e-6f);
  const float keep_p = fminf(fmaxf(top_p, 0.f), 1.f);
  float mx = lg[tid];
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) mx = fmaxf(mx, __shfl_xor(mx, o, 64));
  if (mx == SMP_NEG_INF) { if (tid < n) put(tid, 0.f); return; }
  if (tid < n) pr[tid] = lg[tid] == SMP_NEG_INF ? 0.f : expf((lg[tid] - mx) / temp);
  __syncthreads();
  if (tid == 0) {
    float sum = 0.f;
    for (uint32_t i = 0; i < n; i++) if (lg[i] != SMP_NEG_INF) sum += pr[i];
    s_sum = sum;
  }
  __syncthreads();
  const float sum = s_sum;
  if (sum <= 0.f) { if (tid < n) put(tid, tid == 0 ? 1.f : 0.f); return; }
  if (tid < n) pr[tid] /= sum;
  __syncthreads();
  if (tid == 0) {
    uint32_t keep = 0;
    float csum = 0.f;
    for (uint32_t i = 0; i < n; i++) {
      csum += pr[i];
      keep = i + 1;
      if (keep_p >= 0.999999f || csum >= keep_p) break;
    }
    if (keep == 0 && n > 0) keep = 1;
    float ks = 0.f;
    for (uint32_t i = 0; i < keep; i++) ks += pr[i];
    if (ks <= 0.f) ks = 1.f;
    s_keep = keep; s_ks = ks;
  }
  __syncthreads();
  if (tid < n) put(tid, tid < s_keep ? pr[tid] / s_ks : 0.f);
}

// dst[i] = data[base + uint(data[sel[i]])]  (candidate position -> token id), negatives / non-finite -> 0
__global__ void __launch_bounds__(64)
k_resolve_idx(float* data, const uint32_t* __restrict__ lbase, const uint32_t* __restrict__ lsel,
              const uint32_t* __restrict__ ldst, uint32_t n, uint64_t n_elems) {
  const uint32_t i = blockIdx.x * 64u + threadIdx.x;
  if (i >= n) return;
  float s = lsel[i] < n_elems ? data[lsel[i]] : 0.f;
  if (isnan(s) || isinf(s) || s < 0.f) s = 0.f;
  const uint64_t src = (uint64_t)lbase[0] + (uint32_t)fminf(s, 4294967040.f);
  float t = src < n_elems ? data[src] : 0.f;
  if (isnan(t) || isinf(t) || t < 0.f) t = 0.f;
  if (ldst[i] < n_elems) data[ldst[i]] = t;
}

// Inverse-CDF draw over n <= 64 probabilities with the uniform number stored in the map.
__global__ void __launch_bounds__(64)
k_sample_categorical(float* data, const uint32_t* __restrict__ lidx, const uint32_t* __restrict__ lprob,
                     const uint32_t* __restrict__ lrand, const uint32_t* __restrict__ ldst, uint32_t n, uint64_t n_elems) {
  // the probabilities come in with one load per lane; the sums run over them in order in lane 0 (same bits as a
  // single invocation that reads them one after the other)
  __shared__ float ps[SMP_MAX];
  const uint32_t tid = threadIdx.x;
  if (n == 0) return;
  if (tid < n) {
    float p = lprob[tid] < n_elems ? data[lprob[tid]] : 0.f;
    if (isnan(p) || isinf(p) || p < 0.f) p = 0.f;
    ps[tid] = p;
  }
  __syncthreads();
  if (tid != 0) return;
  auto idx = [&](uint32_t i) { return lidx[i] < n_elems ? data[lidx[i]] : 0.f; };
  if (ldst[0] >= n_elems) return;
  float total = 0.f;
  for (uint32_t i = 0; i < n; i++) total += ps[i];
  if (!(total > 0.f)) { data[ldst[0]] = idx(0); return; }
  float r = lrand[0] < n_elems ? data[lrand[0]] : 0.f;
  if (isnan(r) || isinf(r)) r = 0.f;
  r = fminf(fmaxf(r, 0.f), 0.99999994f);
  const float target = r * total;
  float acc = 0.f;
  uint32_t chosen = n - 1;
  for (uint32_t i = 0; i < n; i++) {
    acc += ps[i];
    if (target < acc) { chosen = i; break; }
  }
  data[ldst[0]] = idx(chosen);
}

// logits[locs[tok]] /= penalty when positive, *= penalty otherwise, once per listed token id
__global__ void __launch_bounds__(64)
k_repeat_penalty(float* data, const uint32_t* __restrict__ llog, uint64_t n_logit_locs, const uint32_t* __restrict__ toks,
                 uint32_t n_ids, float penalty, uint64_t n_elems) {
  const uint32_t i = blockIdx.x * 64u + threadIdx.x;
  if (i >= n_ids) return;
  const uint32_t tok = toks[i];
  if (tok >= n_logit_locs) return;
  // The reference's callers pass distinct ids (adam/models/engine.py:2052); with a repeated id the
  // shader's invocations race.  Here every distinct id is penalised exactly once.
  for (uint32_t j = 0; j < i; j++) if (toks[j] == tok) return;
  const uint32_t loc = llog[tok];
  if (loc >= n_elems) return;
  const float v = data[loc];
  data[loc] = v > 0.f ? v / penalty : v * penalty;
}

}  // namespace adamah

using namespace adamah;

extern "C" {

int map_topk_dev(uint32_t map_id, uint32_t hs, uint32_t hi, uint32_t hv, uint32_t n, uint32_t k) { ADAMAH_API();
  Map* m = get_f32_map(map_id);
  if (!m) return ADAMAH_ERR_INVALID;
  if (n == 0 || k == 0) return ADAMAH_OK;
  if (k > SMP_MAX) return ADAMAH_ERR_INVALID;
  const uint32_t *ls = res_u32(hs, n), *li = res_u32(hi, k), *lv = res_u32(hv, k);
  if (!ls || !li || !lv) return ADAMAH_ERR_INVALID;
  const uint32_t chunks = cdiv(n, TOPK_CHUNK);
  if (chunks > 1 && n <= TSEL_THREADS * TSEL_PER && tuning("ADAMAH_TOPK_SELECT", 1) != 0) {
    k_topk_select<<<1, TSEL_THREADS, 0, g.stream>>>((float*)m->buf, ls, li, lv, n, k, m->n_elems);
    count_launch();
    return check_launch();
  }
  float* pv = nullptr;
  uint32_t* pi = nullptr;
  if (chunks > 1) {
    const size_t need = (size_t)chunks * k;
    if (need > g_topk_part_cap) {
      layout_changed();
      if (g_topk_part) { hipStreamSynchronize(g.stream); hipFree(g_topk_part); }
      g_topk_part_cap = std::max<size_t>(need, 4096);
      if (hipMalloc((void**)&g_topk_part, g_topk_part_cap * 8) != hipSuccess) {
        g_topk_part = nullptr; g_topk_part_cap = 0;
        return ADAMAH_ERR_MEMORY;
      }
    }
    pv = g_topk_part;
    pi = (uint32_t*)(g_topk_part + g_topk_part_cap);
  }
  k_topk_chunk<<<chunks, 256, 0, g.stream>>>((float*)m->buf, ls, li, lv, n, k, m->n_elems, pv, pi);
  count_launch();
  if (chunks > 1) {
    k_topk_merge<<<1, 256, 0, g.stream>>>((float*)m->buf, pv, pi, li, lv, chunks * k, k, m->n_elems);
    count_launch();
  }
  return check_launch();
}

int map_topp_dev(uint32_t map_id, uint32_t hs, uint32_t hd, uint32_t n, float temperature, float top_p) { ADAMAH_API();
  Map* m = get_f32_map(map_id);
  if (!m) return ADAMAH_ERR_INVALID;
  if (n == 0) return ADAMAH_OK;
  if (n > SMP_MAX) return ADAMAH_ERR_INVALID;
  const uint32_t *ls = res_u32(hs, n), *ld = res_u32(hd, n);
  if (!ls || !ld) return ADAMAH_ERR_INVALID;
  k_topp<<<1, 64, 0, g.stream>>>((float*)m->buf, ls, ld, n, temperature, top_p, m->n_elems);
  count_launch();
  return check_launch();
}

int map_resolve_idx_dev(uint32_t map_id, uint32_t hbase, uint32_t hsel, uint32_t hdst, uint32_t n) { ADAMAH_API();
  Map* m = get_f32_map(map_id);
  if (!m) return ADAMAH_ERR_INVALID;
  if (n == 0) return ADAMAH_OK;
  const uint32_t *lb = res_u32(hbase, 1), *lsel = res_u32(hsel, n), *ld = res_u32(hdst, n);
  if (!lb || !lsel || !ld) return ADAMAH_ERR_INVALID;
  k_resolve_idx<<<cdiv(n, 64), 64, 0, g.stream>>>((float*)m->buf, lb, lsel, ld, n, m->n_elems);
  count_launch();
  return check_launch();
}

int map_sample_categorical_dev(uint32_t map_id, uint32_t hidx, uint32_t hprob, uint32_t hrand, uint32_t hdst, uint32_t n) {
  ADAMAH_API();
  Map* m = get_f32_map(map_id);
  if (!m) return ADAMAH_ERR_INVALID;
  if (n == 0) return ADAMAH_OK;
  if (n > SMP_MAX) return ADAMAH_ERR_INVALID;
  const uint32_t *li = res_u32(hidx, n), *lp = res_u32(hprob, n), *lr = res_u32(hrand, 1), *ld = res_u32(hdst, 1);
  if (!li || !lp || !lr || !ld) return ADAMAH_ERR_INVALID;
  k_sample_categorical<<<1, 64, 0, g.stream>>>((float*)m->buf, li, lp, lr, ld, n, m->n_elems);
  count_launch();
  return check_launch();
}

int map_repeat_penalty_dev(uint32_t map_id, uint32_t hlog, uint32_t htok, uint32_t n_ids, float penalty) { ADAMAH_API();
  Map* m = get_f32_map(map_id);
  if (!m) return ADAMAH_ERR_INVALID;
  if (n_ids == 0) return ADAMAH_OK;
  if (n_ids > SMP_MAX) return ADAMAH_ERR_INVALID;
  Res* rl = get_res(hlog);
  const uint32_t* toks = res_u32(htok, n_ids);
  if (!rl || !toks || rl->size_bytes < 4) return ADAMAH_ERR_INVALID;
  const uint32_t* llog = res_u32(hlog, 1);
  if (!llog) return ADAMAH_ERR_INVALID;
  k_repeat_penalty<<<cdiv(n_ids, 64), 64, 0, g.stream>>>((float*)m->buf, llog, rl->size_bytes / 4, toks, n_ids, penalty,
                                                         m->n_elems);
  count_launch();
  return check_launch();
}

}  // extern "C"
