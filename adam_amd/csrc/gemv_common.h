// Device helpers and launch declarations shared by the quantised GEMV translation units.
#pragma once
#include "common.h"

namespace adamah {

enum { FMT_Q4_B16 = 0, FMT_Q4_AFF = 1, FMT_Q8_B16 = 2, FMT_Q8_AFF = 3 };
enum { EPI_STORE = 0, EPI_ARGMAX = 1 };

#define NEG_FLT_MAX (-3.402823466e+38f)
#define INVALID_IDX 0xffffffffu

__device__ __forceinline__ bool better(float cv, uint32_t ci, float bv, uint32_t bi) {
  // strict > or (== and lower index); an invalid best always loses (map_argmax.comp:15-19)
  if (bi == INVALID_IDX) return true;
  if (ci == INVALID_IDX) return false;
  return (cv > bv) || ((cv == bv) && (ci < bi));
}

__device__ __forceinline__ float wave_sum(float v) {
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) v += __shfl_xor(v, o, 64);
  return v;
}

// byte n of a 32-bit register -> float, one VALU op
template <int N> __device__ __forceinline__ float ubyte_f32(uint32_t w) {
  float r;
  if (N == 0) asm("v_cvt_f32_ubyte0 %0, %1" : "=v"(r) : "v"(w));
  else if (N == 1) asm("v_cvt_f32_ubyte1 %0, %1" : "=v"(r) : "v"(w));
  else if (N == 2) asm("v_cvt_f32_ubyte2 %0, %1" : "=v"(r) : "v"(w));
  else asm("v_cvt_f32_ubyte3 %0, %1" : "=v"(r) : "v"(w));
  return r;
}

// tanh-form GELU with the constants of the reference shader (map_op2.comp:34-44)
__device__ __forceinline__ float gelu_tanh(float a) {
  return 0.5f * a * (1.0f + tanhf(0.797884583f * (a + 0.0447149985f * a * a * a)));
}

// One quantised element of a map, affine form: code * scale + zero point of its group.
__device__ __forceinline__ float deq_elem(const uint8_t* W, const float2* qp, uint64_t idx, uint32_t group, bool q4) {
  uint32_t code = q4 ? ((W[idx >> 1] >> ((idx & 1u) * 4u)) & 0xFu) : W[idx];
  float2 p = qp[idx / group];
  return __fadd_rn(__fmul_rn((float)code, p.x), p.y);
}

#define DPP_ADD(v, ctrl, rmask)                                                                    \
  v += __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), ctrl, rmask, 0xF, false))

// Sum over the 64 lanes; the total is valid in lane 63.
__device__ __forceinline__ float wave_sum_to_lane63(float v) {
  DPP_ADD(v, 0xB1, 0xF);    // quad_perm [1,0,3,2]
  DPP_ADD(v, 0x4E, 0xF);    // quad_perm [2,3,0,1]
  DPP_ADD(v, 0x141, 0xF);   // row_half_mirror
  DPP_ADD(v, 0x140, 0xF);   // row_mirror: every lane of a 16-lane row holds the row sum
  DPP_ADD(v, 0x142, 0xA);   // row_bcast15 into rows 1 and 3
  DPP_ADD(v, 0x143, 0xC);   // row_bcast31 into rows 2 and 3
  return v;
}

// Launchers of the matrix-instruction Q4 kernels (gemv_mfma.hip).  One [N, K] Q4 matrix starting at
// element `b` of the weight map, activations at element `a` and the result at element `c` of the
// activation map (store), or per-group partial (index, value) pairs at lidx/lval (argmax).  The
// offsets are passed by value (the caller read them from the host copies of the handles), which
// spares the kernel a dependent load before its first weight load.  `fmt`: FMT_Q4_B16 / FMT_Q4_AFF.
//
// `fz` (optional) folds neighbouring row-wise ops into the launch: a prologue that produces the
// activation vector, and for the store variant an epilogue applied to the result rows.  Every folded
// op also stores its own result where it would have stored it alone.  Offsets are element offsets in
// the activation map unless noted.
enum { PRO_NONE = 0, PRO_RMSNORM = 1, PRO_NORM2 = 2, PRO_COMBINE = 3 };
enum { PRO_WPT = 2 };   // 8-element words a thread keeps in registers: K <= 16 * workgroup size
enum { EPIX_NONE = 0, EPIX_ADD = 1, EPIX_GEGLU = 2, EPIX_SWIGLU = 3 };
struct GemvFuse {
  // PRO_RMSNORM: x = rmsnorm(src; w, eps)                    -> p_dst
  // PRO_NORM2:   t = rmsnorm(src; w, eps) + res               -> p_tdst
  //              x = rmsnorm(t; w2, eps2)                     -> p_dst
  uint32_t pro;
  uint32_t p_src, p_src2;   // source vector; weight w (element offset in p_wt)
  uint32_t p_dst;
  float p_eps;
  const float* p_wt;
  uint32_t p_res, p_tdst, p_w2;   // residual, destination of t, weight w2 (element offset in p_wt2)
  float p_eps2;
  const float* p_wt2;
  // t usually goes back over the residual, which every workgroup reads.  Where it is stored:
  //   t_mode 0: by whichever workgroup draws the last ticket of `counter` (zero-initialised, left at zero);
  //   t_mode 1: by workgroup 0 at once (p_tdst lies clear of everything the launch reads);
  //   t_mode 2: workgroup 0 parks it at t_park, and a later launch that does not touch p_tdst copies it there
  //             (its d_src / d_dst / d_n): no atomic, whose reply would hold up the drawing wave's weight loads
  uint32_t* counter;
  uint32_t t_mode;
  float* t_park;
  // any prologue: d_n > 0: workgroup 0 copies d_n floats from d_src to element d_dst of the activation map
  const float* d_src;
  uint32_t d_dst, d_n;
  // PRO_COMBINE: x = merge of the split-sequence attention partials, heads side by side  -> p_dst
  //   partial[(head * c_splits + s) * (c_vd + 2)] = {max, sum, values[c_vd]}
  const float* c_partial;
  uint32_t c_splits, c_vd;
  //   c_qn > 0: the attention launch also left the token's prepared queries in scratch memory: c_qn floats from
  //   c_qsrc go to element c_qdst (workgroup 0)
  const float* c_qsrc;
  uint32_t c_qdst, c_qn;
  // EPIX_ADD:            e_dst[row] = e_res[row] + y[row]
  // EPIX_GEGLU / SWIGLU: the matrix is [gate rows; up rows], e_dst[i] = act(y[i]) * y[N/2 + i]
  uint32_t e_mode;
  uint32_t e_res, e_dst;
};
// Threads per workgroup the launchers will use for a matrix with N rows (store variant).
uint32_t mfma_store_threads(uint32_t K, uint32_t N);
// `out` (optional): the result rows go to out[c + row] instead of the activation map.
int launch_mfma_store(int fmt, const Map* ma, const Map* mw, uint32_t a, uint32_t b, uint32_t c, uint32_t K,
                      uint32_t N, const GemvFuse* fz = nullptr, float* out = nullptr);
int launch_mfma_argmax(int fmt, const Map* ma, const Map* mw, uint32_t a, uint32_t b, const uint32_t* lidx,
                       const uint32_t* lval, uint32_t K, uint32_t N, uint32_t rows_per_group,
                       const GemvFuse* fz = nullptr);
bool mfma_path_ok(const Map* mw, uint32_t K);
// Result placement of a matmul over several weight matrices stacked row-wise (Q, K, V or gate, up in one
// launch): rows [begin[s], begin[s + 1]) of the stack belong to matrix s, whose [M, n[s]] result starts
// at element c[s] of the activation map.
// add (count == 0, one matrix): a queued element-wise add that consumes the result, r + y, is stored as
// well: y goes to its own place, r[row * N + n] + y to dst[row * N + n] (element offsets res, dst).
// glu (count == 2, two matrices of N / 2 rows each, M <= 32): the gated activation over the two results that is
// queued behind them (op2 code 34 GEGLU / 35 SWIGLU: act(first) * second) is stored as well, at element dst.
struct GemmSegs {
  uint32_t count;
  uint32_t begin[5];
  uint32_t n[4];
  uint64_t c[4];
  uint32_t add;
  uint64_t res, dst;
  uint32_t glu;
};
// M > 1: fp16 matrix-core GEMM over Q4 block16 weights (gemm_q4_mfma.hip); operands already validated.
// q8: Q8 block16 weights instead (M <= 32).  out: the [M, N] result goes to this buffer instead of the
// activation map (one op).  a_host / c_host: element offsets of op 0's activations and result when the
// host knows them (n_ops == 1): lets consecutive matmuls over the same rows share one conversion.  b_host: likewise
// the element offset of op 0's weights; known offsets go to the kernels by value (no load in front of their first loads).
// segs (M <= 32, one op): the weights are several matrices back to back, results placed per segment.
uint32_t gemm_q4_k_shares(uint32_t M, uint32_t K, uint32_t N);   // > 1: the matmul runs over shares of K and may store an add
int launch_gemm_q4_mfma(const Map* ma, const Map* mw, const uint32_t* la, const uint32_t* lb, const uint32_t* lc,
                        uint32_t M, uint32_t K, uint32_t N, uint32_t n_ops, bool q8 = false, float* out = nullptr,
                        int64_t a_host = -1, int64_t c_host = -1, const GemmSegs* segs = nullptr, int64_t b_host = -1);
// For a kernel that produces the rows [M, K] of a coming batched matmul: the buffers of their fp16 form
// ((s, 1/s) per row; two planes of K halves per row: fp16(x s) and the fp16 remainder), grown as needed, and -- after that kernel's launch has been
// counted -- the note that rows [a, a + M K) of `buf` are converted, so the matmul skips its conversion.
bool gemm_act_slots(uint32_t M, uint32_t K, float** scale, __half** xh, __half** xl);
void gemm_act_forget();
// Gated activation (op2 34 GEGLU / 35 SWIGLU) of the [M, K] rows at elements a and b into the rows at d, and the fp16
// form of the result for the batched matmul that follows, in one launch.  false: not taken, nothing launched.
// Merge of the attention slices of M sequences (at most 8 slices, partial[(row * heads + head) * splits + s]) into the
// rows [M, K] at element o0, and the fp16 form of those rows for the matmul that follows, in one launch.  false: not
// taken, nothing launched.
bool launch_attn_merge_rows_f16(const Map* ma, const float* partial, uint32_t o0, uint32_t M, uint32_t K, uint32_t D,
                                uint32_t splits);
bool launch_glu_act_f16(const Map* ma, uint32_t op, uint32_t a, uint32_t b, uint32_t d, uint32_t M, uint32_t K);
void gemm_act_mark(const void* buf, uint64_t a, uint32_t M, uint32_t K);
// Second pass of the fused GEMV + argmax: best of the per-group partials, token id stored as float.
int launch_argmax_pairs(const Map* ma, const uint32_t* lidx, const uint32_t* lval, const uint32_t* ldst,
                        uint32_t n_groups);
int tuning(const char* name, int dflt);   // behaviour switch, from the environment
int knob(const char* name, int dflt);     // launch-shape number, fixed unless built with -DADAMAH_TUNING
// Preconditions of the block kernels, checked against the host copies of the handles: group size 32,
// K a multiple of 32, weight base block aligned, operands in range.  Returns the two element offsets.
bool block_path_ok(const Map* ma, const Map* mw, uint32_t ha, uint32_t hb, uint32_t K, uint32_t N, uint64_t* a_out,
                   uint64_t* b_out);
// Storage format (FMT_*) of the weights [b, b + n_w) of a quantised map.
int fmt_of(const Map* mw, uint64_t b, uint64_t n_w);
// gemv_q.hip: the block-layout GEMV (Q4 or Q8) with the result rows in `out`, device memory outside the maps
int launch_block_store_to(int fmt, const Map* ma, const Map* mw, const uint32_t* la, const uint32_t* lb, uint32_t K,
                          uint32_t N, float* out);

}  // namespace adamah
