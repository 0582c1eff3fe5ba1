/* C ABI of libadamah_hip.so -- the MI355X implementation of the ADAMAH native op surface.
 *
 * Each declaration names the reference function it replaces (file:line under
 * adamah-MAIN/adamah/ of the reference tree).  Signatures are identical to the reference's, so
 * its ctypes binding (adamah/__init__.py:527-1131) binds this library unchanged through
 * ADAMAH_LIB_PATH.  Conventions (adamah.c:24-28, __init__.py:150-153):
 *   - int returns: 0 OK, -1 backend error, -2 out of memory, -3 invalid argument/handle/map,
 *     -4 not found;
 *   - uint64_t returns of map_upload_dev / map_gather_dev: handle in the low 32 bits
 *     (ticket bits are always 0), 0 = failure;
 *   - host pointers are borrowed for the duration of the call; one context per process, calls
 *     from one thread; work is ordered on one HIP stream and host-visible reads wait for it.
 * Maps are flat device buffers addressed by map id 0..15; a "handle" names a small device
 * array of uint32 element offsets ("locs") or float data.  Quantised maps hold 4-bit (element i =
 * nibble i%8 of little-endian word i/8) or 8-bit codes with per-group (scale, zero_point):
 * value = float(code) * scale + zero_point, group = flat element index / group_size.
 */
#ifndef ADAMAH_HIP_H
#define ADAMAH_HIP_H
#include <stdint.h>
#ifdef __cplusplus
extern "C" {
#endif

/* ---- lifecycle ------------------------------------------------------------------------- */
int adamah_init(void);                                        /* adamah.c:2503 */
int adamah_init_ex(uint64_t hot_bytes, uint64_t cold_bytes);  /* adamah.c:1975 (pool sizes accepted, unused) */
void adamah_shutdown(void);                                   /* adamah.c:2596 */
void adamah_sync(void);                                       /* adamah.c:1820 */
void adamah_synchronize(uint64_t ticket);                     /* adamah.c:1866 */
void adamah_synchronize_all(void);                            /* adamah.c:1914 */
int adamah_probe_device(uint64_t* heap_bytes, uint64_t* budget_bytes, uint64_t* usage_bytes,
                        uint32_t* device_type);               /* adamah.c:2379 */
int adamah_is_integrated_gpu(void);                           /* adamah.c:11066 (always 0) */
void adamah_set_xq_matmul_wg(uint32_t wg_x, uint32_t wg_y);   /* adamah.c:11071 (no effect) */
void adamah_get_gpu_caps(uint32_t* max_workgroup_size, uint32_t* subgroup_size,
                         uint64_t* vram_bytes);               /* adamah.c:11079 */

/* ---- batching, fusion queue, statistics -------------------------------------------------- */
void batch_begin(void);                                       /* adamah.c:1629 */
void batch_end(void);                                         /* adamah.c:1647 */
void adamah_fusion_enable(int enable);                        /* adamah.c:4670 */
int adamah_fusion_is_enabled(void);                           /* adamah.c:4677 */
int adamah_fusion_flush(void);                                /* adamah.c:5653 */
void adamah_fusion_set_scheduler_mode(int mode);              /* adamah.c:708 */
int adamah_fusion_get_scheduler_mode(void);                   /* adamah.c:718 */
int adamah_register_loc_span(uint32_t handle, uint32_t map_id, uint32_t start,
                             uint32_t count);                 /* adamah.c:675 */
int adamah_register_row_base_span(uint32_t handle, uint32_t map_id, uint32_t start, uint32_t count,
                                  uint32_t stride, uint32_t row_size); /* adamah.c:691 */
void adamah_clear_loc_alias_meta(uint32_t handle);            /* adamah.c:668 */
void adamah_stats_reset(void);                                /* adamah.c:316 */
void adamah_stats_get(uint64_t* dispatch_count, uint64_t* submit_count, uint64_t* barrier_count,
                      uint64_t* fusion_flush_count, uint64_t* descriptor_set_update_count,
                      uint64_t* descriptor_cache_hit_count, uint64_t* descriptor_cache_miss_count,
                      uint64_t* alias_conflict_count, uint64_t* scheduler_mode); /* adamah.c:321 */
uint32_t adamah_get_last_barrier_count(void);                 /* adamah.c:11061 */

/* ---- maps --------------------------------------------------------------------------------- */
int adamah_set_dtype(uint32_t dtype);                         /* adamah.c:4585 */
uint32_t adamah_get_dtype(void);                              /* adamah.c:4614 */
int map_init(uint32_t id, uint32_t word_size, uint32_t pack_size, uint32_t n_packs); /* adamah.c:2686 */
int map_init_dtype(uint32_t id, uint32_t dtype, uint32_t pack_size, uint32_t n_packs,
                   uint32_t group_size);                      /* adamah.c:2698 */
int map_destroy(uint32_t id);                                 /* adamah.c:2826 */
uint64_t map_size(uint32_t id);                               /* adamah.c:2855 */
uint32_t map_get_dtype(uint32_t map_id);                      /* adamah.c:4659 */
int map_set_qparams(uint32_t map_id, const float* scales, const float* zero_points,
                    uint32_t n_groups);                       /* adamah.c:4621 */

/* ---- host <-> map ------------------------------------------------------------------------- */
/* The three scatters and map_gather are `int` in adamah.c; the reference's binding reads them as 64-bit
 * tickets (adamah/__init__.py:578, :586, :597, :608 set restype c_uint64), which is what is declared here:
 * 0 on success. */
uint64_t map_scatter(uint32_t map_id, const uint32_t* locs, const void* data, uint32_t n_locs); /* adamah.c:3087 */
uint64_t map_scatter_contiguous(uint32_t map_id, uint32_t start_pack, const void* data,
                                uint32_t n_locs);             /* adamah.c:2896 */
uint64_t map_scatter_q4_packed_contiguous(uint32_t map_id, uint32_t start_pack, const void* packed_u8,
                                          uint32_t n_locs);   /* adamah.c:3035 */
uint64_t map_gather(uint32_t map_id, const uint32_t* locs, void* data, uint32_t n_locs); /* adamah.c:3374 */

/* ---- device-resident handles --------------------------------------------------------------- */
uint64_t map_upload_dev(uint32_t handle, const void* data, uint32_t n_bytes);  /* adamah.c:3570 */
int map_download_dev(uint32_t handle, void* data, uint32_t n_bytes);           /* adamah.c:3665 */
uint64_t map_gather_dev(uint32_t map_id, uint32_t locs_handle, uint32_t n_locs); /* adamah.c:3788 */
uint64_t map_scatter_dev(uint32_t map_id, uint32_t locs_handle, uint32_t n_locs,
                         uint32_t src_handle);                /* adamah.c:3703 */

/* ---- element-wise / reductions (host-locs and handle variants) ----------------------------- */
int map_op1(uint32_t map_id, uint32_t op, const uint32_t* locs_src, const uint32_t* locs_dst, uint32_t n); /* adamah.c:5837 */
int map_op2(uint32_t map_id, uint32_t op, const uint32_t* locs_a, const uint32_t* locs_b,
            const uint32_t* locs_dst, uint32_t n);            /* adamah.c:5931 */
int map_broadcast(uint32_t map_id, uint32_t op, const uint32_t* locs_src, const uint32_t* locs_scalar,
                  const uint32_t* locs_dst, uint32_t n);      /* adamah.c:6296 */
int map_reduce(uint32_t map_id, uint32_t op, const uint32_t* locs_src, const uint32_t* locs_dst, uint32_t n); /* adamah.c:6184 */
int map_matmul(uint32_t map_id, const uint32_t* locs_a, const uint32_t* locs_b, const uint32_t* locs_c,
               uint32_t M, uint32_t K, uint32_t N, uint32_t n_ops); /* adamah.c:6043 */
int map_softmax(uint32_t map_id, const uint32_t* locs_src, const uint32_t* locs_dst, uint32_t n_rows,
                uint32_t row_size);                           /* adamah.c:6412 */
int map_layernorm(uint32_t map_id, const uint32_t* locs_src, const uint32_t* locs_dst,
                  const uint32_t* locs_gamma, const uint32_t* locs_beta, uint32_t n_rows, uint32_t dim,
                  float eps);                                 /* adamah.c:7384 */
int map_op1_dev(uint32_t map_id, uint32_t op, uint32_t locs_src, uint32_t locs_dst, uint32_t n); /* adamah.c:5923 */
int map_op2_dev(uint32_t map_id, uint32_t op, uint32_t locs_a, uint32_t locs_b, uint32_t locs_dst,
                uint32_t n);                                  /* adamah.c:6029 */
int map_broadcast_dev(uint32_t map_id, uint32_t op, uint32_t locs_src, uint32_t locs_scalar,
                      uint32_t locs_dst, uint32_t n);         /* adamah.c:6398 */
int map_reduce_dev(uint32_t map_id, uint32_t op, uint32_t locs_src, uint32_t locs_dst, uint32_t n); /* adamah.c:6279 */
int map_fma_dev(uint32_t map_id, uint32_t locs_a, uint32_t locs_b, uint32_t locs_c, uint32_t locs_dst,
                uint32_t n_locs);                             /* adamah.c:8086 */
int map_matmul_dev(uint32_t map_id, uint32_t locs_a, uint32_t locs_b, uint32_t locs_c, uint32_t M,
                   uint32_t K, uint32_t N, uint32_t n_ops);   /* adamah.c:6058 */
int map_softmax_dev(uint32_t map_id, uint32_t locs_src, uint32_t locs_dst, uint32_t n_rows,
                    uint32_t row_size);                       /* adamah.c:6573 */
int map_softmax_abs_dev(uint32_t map_id, uint32_t locs_src, uint32_t locs_dst, uint32_t n_rows,
                        uint32_t row_size);                   /* adamah.c:6584 */
int map_attn_softmax_abs_dev(uint32_t map_id, uint32_t locs_src, uint32_t locs_dst, uint32_t n_rows,
                             uint32_t row_size, float scale, float cap); /* adamah.c:6670 */
int map_layernorm_dev(uint32_t map_id, uint32_t locs_src, uint32_t locs_dst, uint32_t locs_gamma,
                      uint32_t locs_beta, uint32_t n_rows, uint32_t dim, float eps); /* adamah.c:7503 */
int map_argmax_dev(uint32_t map_id, uint32_t locs_src, uint32_t locs_dst, uint32_t n); /* adamah.c:6875 */
int map_topk_dev(uint32_t map_id, uint32_t locs_src, uint32_t locs_idx_dst, uint32_t locs_val_dst,
                 uint32_t n, uint32_t k);                     /* adamah.c:6978 (k <= 64) */
int map_topp_dev(uint32_t map_id, uint32_t locs_src, uint32_t locs_dst, uint32_t n, float temperature,
                 float top_p);                                /* adamah.c:7095 (n <= 64) */
int map_resolve_idx_dev(uint32_t map_id, uint32_t base_locs, uint32_t sel_locs, uint32_t dst_locs,
                        uint32_t n);                          /* adamah.c:7210 */
int map_sample_categorical_dev(uint32_t map_id, uint32_t locs_idx, uint32_t locs_prob, uint32_t rand_loc,
                               uint32_t dst_loc, uint32_t n); /* adamah.c:7286 (n <= 64) */
int map_repeat_penalty_dev(uint32_t map_id, uint32_t locs_src, uint32_t token_ids, uint32_t n_ids,
                           float penalty);                    /* adamah.c:6787 (n_ids <= 64) */
/* Logits of a quantised [N, K] matrix reduced to a sorted partial top-k list per group of
 * rows_per_group rows (256 in the forms without _ex); rows listed in penalty_ids get the repeat
 * penalty before ranking.  locs_idx_dst / locs_val_dst hold ceil(N / rows_per_group) * k entries.
 * k <= 64, n_penalty <= 64. */
int map_matvec_topk_t_xq4_dev(uint32_t map_act, uint32_t map_wt, uint32_t locs_a, uint32_t locs_b,
                              uint32_t penalty_ids, uint32_t locs_idx_dst, uint32_t locs_val_dst, uint32_t K,
                              uint32_t N, uint32_t k, uint32_t n_penalty, float repeat_penalty); /* adamah.c:9816 */
int map_matvec_topk_t_xq4_ex_dev(uint32_t map_act, uint32_t map_wt, uint32_t locs_a, uint32_t locs_b,
                                 uint32_t penalty_ids, uint32_t locs_idx_dst, uint32_t locs_val_dst, uint32_t K,
                                 uint32_t N, uint32_t k, uint32_t n_penalty, float repeat_penalty,
                                 uint32_t rows_per_group);    /* adamah.c:9727 */
int map_matvec_topk_t_xq8_dev(uint32_t map_act, uint32_t map_wt, uint32_t locs_a, uint32_t locs_b,
                              uint32_t penalty_ids, uint32_t locs_idx_dst, uint32_t locs_val_dst, uint32_t K,
                              uint32_t N, uint32_t k, uint32_t n_penalty, float repeat_penalty); /* adamah.c:10000 */
int map_matvec_topk_t_xq8_ex_dev(uint32_t map_act, uint32_t map_wt, uint32_t locs_a, uint32_t locs_b,
                                 uint32_t penalty_ids, uint32_t locs_idx_dst, uint32_t locs_val_dst, uint32_t K,
                                 uint32_t N, uint32_t k, uint32_t n_penalty, float repeat_penalty,
                                 uint32_t rows_per_group);    /* adamah.c:9911 */
/* Exact logits of n_ids <= 64 shortlisted rows: row = act[partial_idx_base[0] + uint(act[sel_locs[i]])]. */
int map_matvec_rerank_t_xq8_dev(uint32_t map_act, uint32_t map_wt, uint32_t locs_a, uint32_t locs_b,
                                uint32_t partial_idx_base, uint32_t sel_locs, uint32_t penalty_ids,
                                uint32_t locs_idx_dst, uint32_t locs_val_dst, uint32_t K, uint32_t n_ids,
                                uint32_t n_penalty, float repeat_penalty); /* adamah.c:10018 */

/* Projections that share one activation vector, in one call.  Every handle holds one element offset.
 * Matrices and results that lie back to back are computed by one launch. */
int map_fused_qkv_t_xq4_dev(uint32_t map_act, uint32_t map_wt, uint32_t locs_a, uint32_t locs_bq, uint32_t locs_bk,
                            uint32_t locs_bv, uint32_t locs_cq, uint32_t locs_ck, uint32_t locs_cv, uint32_t K,
                            uint32_t N_q, uint32_t N_k, uint32_t N_v);  /* adamah.c:8809 */
int map_fused_qkv_t_xq8_dev(uint32_t map_act, uint32_t map_wt, uint32_t locs_a, uint32_t locs_bq, uint32_t locs_bk,
                            uint32_t locs_bv, uint32_t locs_cq, uint32_t locs_ck, uint32_t locs_cv, uint32_t K,
                            uint32_t N_q, uint32_t N_k, uint32_t N_v);  /* adamah.c:9081 */
int map_fused_gateup_t_xq4_dev(uint32_t map_act, uint32_t map_wt, uint32_t locs_a, uint32_t locs_b_gate,
                               uint32_t locs_b_up, uint32_t locs_c_gate, uint32_t locs_c_up, uint32_t K,
                               uint32_t N_gate, uint32_t N_up);        /* adamah.c:8953 */
int map_fused_gateup_t_xq8_dev(uint32_t map_act, uint32_t map_wt, uint32_t locs_a, uint32_t locs_b_gate,
                               uint32_t locs_b_up, uint32_t locs_c_gate, uint32_t locs_c_up, uint32_t K,
                               uint32_t N_gate, uint32_t N_up);        /* adamah.c:9225 */
/* out[i] = silu(x . Wgate[i]) * (x . Wup[i]), i < N_ff */
int map_fused_gateup_act_t_xq8_dev(uint32_t map_act, uint32_t map_wt, uint32_t locs_a, uint32_t locs_b_gate,
                                   uint32_t locs_b_up, uint32_t locs_c_out, uint32_t K, uint32_t N_ff); /* adamah.c:9353 */

/* ---- decode hot path ----------------------------------------------------------------------- */
int map_rmsnorm_dev(uint32_t map_id, uint32_t locs_src, uint32_t locs_wt, uint32_t locs_dst,
                    uint32_t n_rows, uint32_t dim, float eps); /* adamah.c:7687 */
int map_rmsnorm_x_dev(uint32_t map_act, uint32_t map_wt, uint32_t locs_src, uint32_t locs_wt,
                      uint32_t locs_dst, uint32_t n_rows, uint32_t dim, float eps); /* adamah.c:8459 */
int map_rmsnorm_add_dev(uint32_t map_id, uint32_t locs_src, uint32_t locs_wt, uint32_t locs_resid,
                        uint32_t locs_dst, uint32_t n_rows, uint32_t dim, float eps); /* adamah.c:7786 */
int map_rope_dev(uint32_t map_id, uint32_t locs_src, uint32_t locs_dst, uint32_t n_tokens,
                 uint32_t n_heads, uint32_t head_dim, uint32_t pos_offset, float freq_base); /* adamah.c:7879 */
int map_qk_norm_rope_x_dev(uint32_t map_act, uint32_t map_wt, uint32_t locs_q_src, uint32_t locs_q_wt,
                           uint32_t locs_k_src, uint32_t locs_k_wt, uint32_t locs_qk_dst, uint32_t q_rows,
                           uint32_t q_dim, uint32_t k_rows, uint32_t k_dim, uint32_t pos_offset,
                           float freq_base);                  /* adamah.c:8586 */
int map_row_copy_dev(uint32_t map_id, uint32_t copy_spec, uint32_t src_base, uint32_t n_copies,
                     uint32_t row_size);                      /* adamah.c:8075 */
int map_row_copy_offset_dev(uint32_t map_id, uint32_t copy_spec, uint32_t src_base,
                            uint32_t dst_row_offset, uint32_t n_copies, uint32_t row_size); /* adamah.c:8061 */
int map_matmul_t_dev(uint32_t map_id, uint32_t locs_a, uint32_t locs_b, uint32_t locs_c, uint32_t M,
                     uint32_t K, uint32_t N, uint32_t n_ops); /* adamah.c:7894 */
int map_attn_softmax_value_dev(uint32_t map_id, uint32_t locs_scores, uint32_t locs_values,
                               uint32_t locs_out, uint32_t n_ops, uint32_t row_size, uint32_t value_dim,
                               float scale, float cap);       /* adamah.c:6768 */
int map_matmul_t_x_dev(uint32_t map_act, uint32_t map_wt, uint32_t locs_a, uint32_t locs_b, uint32_t locs_c,
                       uint32_t M, uint32_t K, uint32_t N, uint32_t n_ops); /* adamah.c:8180 */
int map_matmul_x_dev(uint32_t map_act, uint32_t map_wt, uint32_t locs_a, uint32_t locs_b, uint32_t locs_c,
                     uint32_t M, uint32_t K, uint32_t N, uint32_t n_ops);   /* adamah.c:8282 */
int map_matmul_t_xq4_dev(uint32_t map_act, uint32_t map_wt, uint32_t locs_a, uint32_t locs_b,
                         uint32_t locs_c, uint32_t M, uint32_t K, uint32_t N, uint32_t n_ops); /* adamah.c:8693 */
int map_matmul_xq4_dev(uint32_t map_act, uint32_t map_wt, uint32_t locs_a, uint32_t locs_b,
                       uint32_t locs_c, uint32_t M, uint32_t K, uint32_t N, uint32_t n_ops);   /* adamah.c:9468 */
int map_matmul_t_xq8_dev(uint32_t map_act, uint32_t map_wt, uint32_t locs_a, uint32_t locs_b,
                         uint32_t locs_c, uint32_t M, uint32_t K, uint32_t N, uint32_t n_ops); /* adamah.c:9834 */
int map_matmul_xq8_dev(uint32_t map_act, uint32_t map_wt, uint32_t locs_a, uint32_t locs_b,
                       uint32_t locs_c, uint32_t M, uint32_t K, uint32_t N, uint32_t n_ops);   /* adamah.c:10131 */
int map_row_gather_xq8_dev(uint32_t map_act, uint32_t map_wt, uint32_t src_base, uint32_t dst_base,
                           uint32_t row_idx, uint32_t row_size, float scale); /* adamah.c:10189 */
int map_matvec_argmax_t_xq4_dev(uint32_t map_act, uint32_t map_wt, uint32_t locs_a, uint32_t locs_b,
                                uint32_t locs_idx_tmp, uint32_t locs_val_tmp, uint32_t locs_dst,
                                uint32_t K, uint32_t N, uint32_t rows_per_group); /* adamah.c:9699 */
int map_matvec_argmax_t_xq8_dev(uint32_t map_act, uint32_t map_wt, uint32_t locs_a, uint32_t locs_b,
                                uint32_t locs_idx_tmp, uint32_t locs_val_tmp, uint32_t locs_dst,
                                uint32_t K, uint32_t N, uint32_t rows_per_group); /* adamah.c:9711 */

/* ---- decode plan ---------------------------------------------------------------------------- */
typedef struct AdamahDecodePlanOp {                           /* adamah.c:175-194 */
  uint32_t kind, map_id, map_id2, op_code, h0, h1, h2, h3, h4, h5, u0, u1, u2, u3, u4, u5;
  float f0, f1;
} AdamahDecodePlanOp;
int adamah_register_decode_plan(uint32_t plan_id, const AdamahDecodePlanOp* ops, uint32_t n_ops); /* adamah.c:10341 */
void adamah_clear_decode_plan(uint32_t plan_id);              /* adamah.c:10361 */
int adamah_decode_step(uint32_t plan_id, uint32_t pos, uint32_t seq_len); /* adamah.c:10367 */

/* ---- extensions with no counterpart in the reference ----------------------------------------- */
/* Declare elements [start, start+count) of float32 map `map_id` a KV cache kept in fp16: rows
 * copied into the range by map_row_copy(_offset)_dev are rounded to fp16, and the attention entry
 * points read the fp16 copy when their K/V operands lie inside it. */
int adamah_kv_cache_fp16(uint32_t map_id, uint32_t start, uint32_t count);
/* Causal attention of m consecutive tokens over one growing KV cache, as one call: for t = 0 .. m-1 exactly
 * the pair  map_matmul_t_dev(map_id, q_handles[t], locs_k, locs_scores, 1, head_dim, n_keys0 + t, n_heads);
 * map_attn_softmax_value_dev(map_id, locs_scores, locs_v, out_handles[t], n_heads, n_keys0 + t, value_dim,
 * scale, softcap)  (adamah.c:7894, adamah.c:6768) -- same results, same queueing inside a batch; it exists because a
 * prompt chunk of 512 tokens would otherwise cost the host 1024 calls per layer.  q_handles / out_handles:
 * m handle ids each (host arrays). */
int adamah_attn_causal_rows_dev(uint32_t map_id, const uint32_t* q_handles, uint32_t locs_k, uint32_t locs_scores,
                                uint32_t locs_v, const uint32_t* out_handles, uint32_t m, uint32_t head_dim,
                                uint32_t n_keys0, uint32_t n_heads, uint32_t value_dim, float scale, float softcap);
/* QK-norm + RoPE of m consecutive tokens in one call: for t = 0 .. m-1 exactly
 * map_qk_norm_rope_x_dev(map_act, map_wt, q_src_handles[t], locs_q_wt, k_src_handles[t], locs_k_wt,
 * dst_handles[t], q_rows, q_dim, k_rows, k_dim, pos0 + t, freq_base)  (adamah.c:8586) -- the companion of
 * adamah_attn_causal_rows_dev for models with per-head Q/K norms.  The three lists: m handle ids each. */
int adamah_qk_norm_rope_rows_dev(uint32_t map_act, uint32_t map_wt, const uint32_t* q_src_handles, uint32_t locs_q_wt,
                                 const uint32_t* k_src_handles, uint32_t locs_k_wt, const uint32_t* dst_handles,
                                 uint32_t m, uint32_t q_rows, uint32_t q_dim, uint32_t k_rows, uint32_t k_dim,
                                 uint32_t pos0, float freq_base);
/* map_matvec_topk_t_xq4_ex_dev for callers that cannot allocate.  No counterpart in the reference: it is for
 * callers under HIP graph capture, tight serving loops and harnesses that forbid hipMalloc.  Same arguments and
 * results; the logits go to a fixed 1 MiB device array that is part of the library's code object (one copy per
 * GPU, held until the process ends), so N <= 262144 (larger: -3 and a message on stderr).  Calls no hipMalloc /
 * hipFree.  Ops still queued in an open batch are not launched by this call (their launch could grow library
 * buffers): it returns -3 until adamah_sync or batch_end has launched them.  The array keeps the previous call's logits; every
 * call overwrites rows [0, N) before ranking them, nothing has to start at zero.  Calls that overlap on one GPU
 * (other streams, other threads) share the array and race. */
int adamah_matvec_topk_t_xq4_noalloc_dev(uint32_t map_act, uint32_t map_wt, uint32_t locs_a, uint32_t locs_b,
                                         uint32_t penalty_ids, uint32_t locs_idx_dst, uint32_t locs_val_dst,
                                         uint32_t K, uint32_t N, uint32_t k, uint32_t n_penalty,
                                         float repeat_penalty, uint32_t rows_per_group);
/* Token feedback without a host round trip per step.  No counterpart in the reference, whose loop reads the chosen
 * token back, looks its embedding row up (on the host for untied embeddings, adam/models/engine.py:2986-2992; with a
 * gather of host-made locations for tied ones, engine.py:2993-3010) and only then issues the next step.
 * embed_tokens: for r = 0 .. m-1, with tok_r = the float32 token id at element locs_tokens[r] of map_act, elements
 * [dst_start + r*E, dst_start + (r+1)*E) of map_act = scale * row tok_r of the [V, E] table that starts at element
 * src_row0 of map_src (float32, Q4 or Q8 map; quantised values decoded as map_gather_dev decodes them).  The result
 * is what map_gather_dev + map_scatter_dev + a multiplication by scale give for the same token.  A token id outside
 * [0, V) gives a row of zeros.  The destination must lie outside an fp16 KV range. */
int adamah_hip_embed_tokens_dev(uint32_t map_act, uint32_t map_src, uint32_t locs_tokens, uint32_t src_row0,
                                uint32_t dst_start, uint32_t m, uint32_t E, uint32_t V, float scale);
/* token_post: in stream order, copy the n <= 62 float32 values at locs_handle's elements of map_id into a ring of 8
 * slots in pinned host memory and then mark the slot with the post's ticket, which the call returns in *ticket
 * (1, 2, 3, ...: the library hands every ticket out once; slot = ticket % 8).
 * token_wait: poll the ticket's slot until it carries `ticket`, then copy its first n values to out.  It neither
 * synchronises the stream nor waits for work queued behind the post, so a caller can issue the next step first and
 * still read every token in order; ops queued in an open batch stay queued.  Returns ADAMAH_ERR_NOT_FOUND when the stream has drained and the ticket is not
 * there (never posted, or its slot taken by the post 8 tickets later). */
int adamah_hip_token_post(uint32_t map_id, uint32_t locs_handle, uint32_t n, uint32_t* ticket);
/* embed_post_tokens: embed_tokens and, in the same launch, token_post of the m <= 62 token values it reads (the
 * ticket comes back in *ticket): a loop that runs one step ahead then needs no launch of its own to hand step n's
 * token to the host -- the embedding launch of step n + 1 does it. */
int adamah_hip_embed_post_tokens_dev(uint32_t map_act, uint32_t map_src, uint32_t locs_tokens, uint32_t src_row0,
                                     uint32_t dst_start, uint32_t m, uint32_t E, uint32_t V, float scale, uint32_t* ticket);
int adamah_hip_token_wait(uint32_t ticket, float* out, uint32_t n);
/* ---- measurement and test helpers: not part of the op surface ------------------------------------
 * Nothing a model engine calls.  bench.py times launches with the stopwatch and calibrates profiler counters
 * with the probe; the parity tests read back what the kernels see through the other two. */
/* HIP-event stopwatch on the library's stream. begin: 0 on success; end: ms or <0. */
int adamah_hip_timer_begin(void);
float adamah_hip_timer_end(void);
/* Streaming calibration: average microseconds per launch of a plain read (mode 0) or copy (mode 1)
 * of bytes_per_launch bytes, walking a pool_bytes buffer; negative = error code. */
float adamah_hip_stream_probe(uint64_t bytes_per_launch, uint64_t pool_bytes, uint32_t mode, uint32_t wg_per_cu,
                              uint32_t launches);
/* Dequantise elements [start, start+count) of a Q4/Q8 map with the GEMV kernels' unpack code. */
int adamah_hip_debug_dequant(uint32_t map_id, uint64_t start, uint64_t count, float* out);
/* 0 = affine qparams only, 1 = fp16-scale block plane in use for the whole map, <0 = error. */
int adamah_hip_map_layout(uint32_t map_id);

#ifdef __cplusplus
}
#endif
#endif
