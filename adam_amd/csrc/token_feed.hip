// Feeding a decode step's token to the next step without a host round trip.
//
// The reference's loop reads the chosen token id back, looks its embedding row up (on the host for untied
// embeddings, adam/models/engine.py:2986-2992; with a gather of host-made locations for tied ones,
// engine.py:2993-3010) and only then issues the next step, so the device idles for a host round trip per token.
// Two pieces remove that wait while the host still sees every token, in order:
//   * adamah_hip_embed_tokens_dev gathers the embedding rows of tokens that are still on the device (the slots the
//     LM head's arg-max wrote), so step n + 1 can be issued before token n has reached the host;
//   * adamah_hip_token_post / adamah_hip_token_wait hand token n to the host through a small ring in pinned host
//     memory: a one-wave kernel in stream order writes the values and then the post's ticket (a number the
//     library hands out, never twice), the host polls the ticket.
//     No copy engine and no stream synchronisation is involved, so the wait ends when step n does even though
//     step n + 1 is already queued behind it.
#include "common.h"
#include "../../include/adamah_hip.h"
#include <immintrin.h>

namespace adamah {

#define MAIL_SLOTS 8u
#define MAIL_MAX 62u
struct TokenMail { uint32_t ticket, n; float val[MAIL_MAX]; };   // 256 bytes
static TokenMail* g_mail = nullptr;       // host address of the ring
static TokenMail* g_mail_dev = nullptr;   // the same memory as the device sees it
static uint32_t g_ticket = 0;             // last ticket handed out: 1, 2, ... (a ticket is never reused, so a slot
                                          // can only ever show the ticket that was waited for or a later one)

// out[dst0 + r * E + e] = table[row0 + tok_r * E + e] * scale for the m tokens tok_r = act[token slot r].  Quantised
// tables are decoded as the dequantising gather does (float(code) * scale_g + zp_g, shaders/src/q4/map_gather.comp).
// A token outside [0, V) gives a row of zeros, as a gather outside the map does.  tok_by_val: slot r is tok0 + r.
template <int FMT>   // 0 = float32, 1 = Q4 (two codes a byte), 2 = Q8
__global__ void __launch_bounds__(256)
k_embed_tokens(float* act, uint64_t act_elems, const uint8_t* __restrict__ src, uint64_t src_elems, uint64_t row0,
               uint32_t E, uint32_t V, uint32_t total, uint32_t dst0, uint32_t tok0, uint32_t tok_by_val, float scale,
               const uint32_t* __restrict__ tok_locs, const float2* __restrict__ qp, uint32_t group, uint32_t m,
               TokenMail* mail, uint32_t ticket) {
  const uint32_t i = blockIdx.x * 256u + threadIdx.x;
  // mail: the launch also hands the m token values to the host, as k_token_post would (wave 0 of workgroup 0)
  if (mail && blockIdx.x == 0 && threadIdx.x < 64u) {
    if (threadIdx.x < m) {
      const uint32_t ml = tok_by_val ? tok0 + threadIdx.x : tok_locs[threadIdx.x];
      mail->val[threadIdx.x] = ml < act_elems ? act[ml] : 0.0f;
    }
    __threadfence_system();
    if (threadIdx.x == 0) {
      mail->n = m;
      __hip_atomic_store(&mail->ticket, ticket, __ATOMIC_RELEASE, __HIP_MEMORY_SCOPE_SYSTEM);
    }
  }
  if (i >= total) return;
  const uint32_t r = i / E, e = i - r * E;
  const uint32_t tl = tok_by_val ? tok0 + r : tok_locs[r];
  const float tf = tl < act_elems ? act[tl] : -1.0f;
  bool ok = tf >= 0.0f && tf < (float)V;
  const uint64_t idx = row0 + (uint64_t)(ok ? (uint32_t)tf : 0u) * E + e;
  ok = ok && idx < src_elems;
  float v = 0.0f;
  if (ok) {
    if (FMT == 0) v = ((const float*)src)[idx];
    else {
      const uint32_t code = FMT == 1 ? ((src[idx >> 1] >> ((idx & 1) * 4)) & 0xFu) : src[idx];
      const float2 p = qp[idx / group];
      v = __fadd_rn(__fmul_rn((float)code, p.x), p.y);
    }
    v = __fmul_rn(v, scale);
  }
  act[dst0 + i] = v;
}

// One wave: values first, then the ticket, both for the host (system scope).
__global__ void __launch_bounds__(64)
k_token_post(const float* __restrict__ act, uint64_t act_elems, const uint32_t* __restrict__ locs, uint32_t n,
             uint32_t ticket, TokenMail* mail) {
  const uint32_t lane = threadIdx.x;
  if (lane < n) {
    const uint32_t l = locs[lane];
    mail->val[lane] = l < act_elems ? act[l] : 0.0f;
  }
  __threadfence_system();
  if (lane == 0) {
    mail->n = n;
    __hip_atomic_store(&mail->ticket, ticket, __ATOMIC_RELEASE, __HIP_MEMORY_SCOPE_SYSTEM);
  }
}

static int mail_setup() {
  if (g_mail) return ADAMAH_OK;
  if (hipHostMalloc((void**)&g_mail, MAIL_SLOTS * sizeof(TokenMail), hipHostMallocCoherent | hipHostMallocMapped) != hipSuccess) {
    (void)hipGetLastError();
    g_mail = nullptr;
    return ADAMAH_ERR_MEMORY;
  }
  if (hipHostGetDevicePointer((void**)&g_mail_dev, g_mail, 0) != hipSuccess) {
    (void)hipGetLastError();
    hipHostFree(g_mail);
    g_mail = nullptr;
    return ADAMAH_ERR_BACKEND;
  }
  for (uint32_t s = 0; s < MAIL_SLOTS; s++) { g_mail[s].ticket = 0xFFFFFFFFu; g_mail[s].n = 0; }
  return ADAMAH_OK;
}

void token_feed_release() {
  if (g_mail) hipHostFree(g_mail);
  g_mail = nullptr; g_mail_dev = nullptr;
}

}  // namespace adamah

using namespace adamah;

// ticket_out: the launch also posts the tokens it reads (adamah_hip_embed_post_tokens_dev)
static int embed_tokens(uint32_t map_act, uint32_t map_src, uint32_t locs_tokens, uint32_t src_row0, uint32_t dst_start,
                        uint32_t m, uint32_t E, uint32_t V, float scale, uint32_t* ticket_out) {
  Map* ma = get_f32_map(map_act);
  Map* ms = get_map(map_src);
  if (!ma || !ms || m == 0 || E == 0 || V == 0 || ms->pack_size != 1 || ma->pack_size != 1) return ADAMAH_ERR_INVALID;
  if ((uint64_t)m * E > 0x7FFFFFFFull) return ADAMAH_ERR_INVALID;
  const uint32_t total = m * E;
  if (!in_range(dst_start, total, ma->n_elems)) return ADAMAH_ERR_INVALID;
  // rows stored as float32 only: the fp16 mirror of a KV range would go stale
  if (ma->kv16 && dst_start < ma->kv_start + ma->kv_count && ma->kv_start < (uint64_t)dst_start + total) return ADAMAH_ERR_INVALID;
  if (!in_range(src_row0, (uint64_t)V * E, ms->n_elems)) return ADAMAH_ERR_INVALID;
  const int fmt = ms->dtype == DTYPE_F32 ? 0 : ms->dtype == DTYPE_Q4 ? 1 : ms->dtype == DTYPE_Q8 ? 2 : -1;
  if (fmt < 0 || (fmt != 0 && (!ms->qp || ms->group_size == 0))) return ADAMAH_ERR_INVALID;
  const uint32_t* tl = res_u32(locs_tokens, m);
  if (!tl) return ADAMAH_ERR_INVALID;
  uint32_t tok0 = 0;
  const uint32_t by_val = res_run(locs_tokens, m, &tok0) && in_range(tok0, m, ma->n_elems) ? 1u : 0u;
  TokenMail* mail = nullptr;
  uint32_t ticket = 0;
  if (ticket_out) {
    if (m > MAIL_MAX) return ADAMAH_ERR_INVALID;
    if (int r = mail_setup()) return r;
    ticket = g_ticket = g_ticket >= 0x7FFFFFFFu ? 1u : g_ticket + 1u;
    *ticket_out = ticket;
    mail = g_mail_dev + ticket % MAIL_SLOTS;
  }
  const dim3 grid(cdiv(total, 256));
#define EMBED(F) k_embed_tokens<F><<<grid, 256, 0, g.stream>>>((float*)ma->buf, ma->n_elems, ms->buf, ms->n_elems, src_row0, E, V, \
                                                          total, dst_start, tok0, by_val, scale, tl, ms->qp, ms->group_size, m, mail, ticket)
  if (fmt == 0) EMBED(0); else if (fmt == 1) EMBED(1); else EMBED(2);
#undef EMBED
  count_launch();
  return check_launch();
}

extern "C" {


int adamah_hip_embed_tokens_dev(uint32_t map_act, uint32_t map_src, uint32_t locs_tokens, uint32_t src_row0,
                                uint32_t dst_start, uint32_t m, uint32_t E, uint32_t V, float scale) { ADAMAH_API();
  return embed_tokens(map_act, map_src, locs_tokens, src_row0, dst_start, m, E, V, scale, nullptr);
}

int adamah_hip_embed_post_tokens_dev(uint32_t map_act, uint32_t map_src, uint32_t locs_tokens, uint32_t src_row0,
                                     uint32_t dst_start, uint32_t m, uint32_t E, uint32_t V, float scale,
                                     uint32_t* ticket) { ADAMAH_API();
  if (!ticket) return ADAMAH_ERR_INVALID;
  return embed_tokens(map_act, map_src, locs_tokens, src_row0, dst_start, m, E, V, scale, ticket);
}

int adamah_hip_token_post(uint32_t map_id, uint32_t locs_handle, uint32_t n, uint32_t* ticket_out) { ADAMAH_API();
  Map* m = get_f32_map(map_id);
  if (!m || n == 0 || n > MAIL_MAX || !ticket_out) return ADAMAH_ERR_INVALID;
  const uint32_t* locs = res_u32(locs_handle, n);
  if (!locs) return ADAMAH_ERR_INVALID;
  if (int r = mail_setup()) return r;
  const uint32_t ticket = g_ticket = g_ticket >= 0x7FFFFFFFu ? 1u : g_ticket + 1u;
  *ticket_out = ticket;
  k_token_post<<<1, 64, 0, g.stream>>>((const float*)m->buf, m->n_elems, locs, n, ticket, g_mail_dev + ticket % MAIL_SLOTS);
  count_launch();
  return check_launch();
}

// (no launch of queued ops here: a post is launched by its own call, so the ticket never depends on the queue, and a
// caller may wait in the middle of a batch without breaking up the folds of the ops it has queued so far)
int adamah_hip_token_wait(uint32_t ticket, float* out, uint32_t n) {
  if (!g_mail || !out || n == 0 || n > MAIL_MAX || ticket == 0 || ticket > 0x7FFFFFFFu) return ADAMAH_ERR_INVALID;
  TokenMail* s = g_mail + ticket % MAIL_SLOTS;
  for (uint32_t spins = 1;; spins++) {
    if (__atomic_load_n(&s->ticket, __ATOMIC_ACQUIRE) == ticket) break;
    if ((spins & 1023u) == 0) {
      // the stream has drained without the ticket: it was never posted, or a later post took its slot
      const hipError_t q = hipStreamQuery(g.stream);
      if (q == hipSuccess) {
        if (__atomic_load_n(&s->ticket, __ATOMIC_ACQUIRE) == ticket) break;
        return ADAMAH_ERR_NOT_FOUND;
      }
      if (q != hipErrorNotReady) { (void)hipGetLastError(); return ADAMAH_ERR_BACKEND; }
    }
    _mm_pause();
  }
  if (s->n < n) return ADAMAH_ERR_INVALID;
  for (uint32_t i = 0; i < n; i++) out[i] = s->val[i];
  return ADAMAH_OK;
}

}  // extern "C"
