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
int launch_mfma_store(int fmt, const Map* ma, const Map* mw, uint32_t a, uint32_t b, uint32_t c, uint32_t K,
                      uint32_t N);
int launch_mfma_argmax(int fmt, const Map* ma, const Map* mw, uint32_t a, uint32_t b, const uint32_t* lidx,
                       const uint32_t* lval, uint32_t K, uint32_t N, uint32_t rows_per_group);
bool mfma_path_ok(const Map* mw, uint32_t K);
int tuning(const char* name, int dflt);

}  // namespace adamah
