// Batched (M > 1) quantised matmul  C[M, N] = A[M, K] . W[N, K]^T  for Q4_0 weights on the fp16
// matrix cores: prefill chunks and batched decode.
//
// Reference: shaders/src/f32/map_matmul_t_xq4.comp:33-73 (one thread per output, scalar K loop;
// dispatch adamah.c:8693-8803).  With more than one activation row the weights are reused, so this
// is the one place on the path where the work is a dense contraction and belongs on MFMA.
//
// v_mfma_f32_16x16x32_f16:  D[i][j] += sum_k A[i][k] B[k][j];  lane l supplies A[l % 16][8g..8g+7] and
// B[8g..8g+7][l % 16] with g = l / 16, and receives D[4g..4g+3][l % 16].  Here i runs over 16 activation rows,
// j over 16 weight rows, and the 32 k of one instruction are ONE 32-weight block: lane (row, g) loads block g of
// the step's four blocks of its weight row as one 16-byte word group, a 4 x 4 transpose of words between the four
// lanes of a row (gfx950 row-swap instructions) leaves it with word g of every block, and the nibbles become
// fp16 (q - 8) exactly.  Each block's products are summed by the matrix core from zero and the block's fp16
// scale is applied to that sum in float32 (one fused multiply-add per output and block), so the weights need no
// rounding at all.  The activations of the tile are converted once per matmul to two fp16 planes (x s = xh + xl,
// s a power of two per row so that no row can overflow; divided out of the float32 result), in the element order
// the unpacking produces; two instructions per block (xh, xl), every product exact.
//
// Tiled form: workgroup = NW waves, each with R tiles of 16 weight rows = 16 NW R weight rows x 16 MT activation
// rows; one step = 128 weights of K (four blocks).
// K-split form (few activation rows): the waves share R tiles of 16 weight rows and take every NWV-th step of K
// each, so that small matrices still spread over the whole chip; their partial tiles are summed through LDS in
// a fixed order.
#include "gemv_common.h"
#include <algorithm>

namespace adamah {

typedef _Float16 h2q_t __attribute__((ext_vector_type(2)));
typedef _Float16 h4q_t __attribute__((ext_vector_type(4)));
typedef float f4q_t __attribute__((ext_vector_type(4)));
typedef float f4qu_t __attribute__((ext_vector_type(4), aligned(4)));
typedef uint32_t u2q_t __attribute__((ext_vector_type(2)));
typedef uint32_t u4q_t __attribute__((ext_vector_type(4)));
typedef _Float16 h8q_t __attribute__((ext_vector_type(8)));

// Two-term activations.  A product w * x of the reference is a float32 product of float32 values; one fp16
// rounding of an operand (2^-12 relative) is harmless in a single projection but adds up over the ~200
// projections of a forward pass (a 512-token chunk ended 1.3e-3 .. 6e-3 away from the token-by-token hidden
// state).  The activations are therefore fed as exact sums of two fp16 numbers,
//   x * s  = xh + xl          xh = fp16(x s), xl = fp16(x s - xh)                (22 significant bits),
// and the weights as the integers (q - 8) with the block scale applied afterwards in float32.  Q8_0 weights (the LM
// head of a lockstep batch, the last projection of a pass) keep one fp16 term for each operand.
__device__ __forceinline__ void split_pair(float a, float b, uint32_t* hi, uint32_t* lo) {
  const _Float16 ah = (_Float16)a, bh = (_Float16)b;
  const h2q_t h = {ah, bh}, l = {(_Float16)(a - (float)ah), (_Float16)(b - (float)bh)};
  *hi = __builtin_bit_cast(uint32_t, h);
  *lo = __builtin_bit_cast(uint32_t, l);
}
// eight consecutive activations (already scaled) -> the 16-byte pieces of both planes, pairs in the order the
// nibble unpacking produces: (0,4)(1,5)(2,6)(3,7)
__device__ __forceinline__ void split_word(const float* v, uint4* hi, uint4* lo) {
  split_pair(v[0], v[4], &hi->x, &lo->x);
  split_pair(v[1], v[5], &hi->y, &lo->y);
  split_pair(v[2], v[6], &hi->z, &lo->z);
  split_pair(v[3], v[7], &hi->w, &lo->w);
}

// The activations are converted once per matmul (or by the kernel that produced them) to the two fp16
// planes the matrix cores consume: rows scaled by their power of two, elements of every 8-word in the
// order (0,4)(1,5)(2,6)(3,7).  The matmul workgroups then copy 16-byte pieces into LDS.  One workgroup per
// row; also stores (s, 1/s).  xl = second plane (same indexing as xh).
__global__ void __launch_bounds__(256)
k_act_f16(const float* act, const uint32_t* __restrict__ la, uint32_t M, uint32_t K, float* scale, uint4* xh, uint4* xl) {
  __shared__ float red[4];
  const uint32_t row = blockIdx.x, op = blockIdx.y, tid = threadIdx.x;
  const float* x = act + (uint64_t)la[op] + (uint64_t)row * K;
  float m = 0.f;
  for (uint32_t i = tid; i < K; i += 256u) m = fmaxf(m, fabsf(x[i]));
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) m = fmaxf(m, __shfl_xor(m, o, 64));
  if ((tid & 63u) == 0) red[tid >> 6] = m;
  __syncthreads();
  m = fmaxf(fmaxf(red[0], red[1]), fmaxf(red[2], red[3]));
  const uint32_t e = (__float_as_uint(m) >> 23) & 0xFFu;
  float s = 1.f, inv = 1.f;
  if (e >= 14u && e <= 254u) { s = __uint_as_float((267u - e) << 23); inv = __uint_as_float((e - 13u) << 23); }
  if (tid == 0) {
    scale[2 * ((uint64_t)op * M + row)] = s;
    scale[2 * ((uint64_t)op * M + row) + 1] = inv;
  }
  const uint64_t o0 = ((uint64_t)op * M + row) * (K >> 3);
  for (uint32_t w = tid; w < (K >> 3); w += 256u) {
    const f4qu_t v0 = *(const f4qu_t*)(x + w * 8u), v1 = *(const f4qu_t*)(x + w * 8u + 4u);
    const float v[8] = {v0.x * s, v0.y * s, v0.z * s, v0.w * s, v1.x * s, v1.y * s, v1.z * s, v1.w * s};
    uint4 hi, lo;
    split_word(v, &hi, &lo);
    xh[o0 + w] = hi;
    xl[o0 + w] = lo;
  }
}

// nibbles of one 32-bit word -> the four fp16 pairs (q - 8) exactly: (1024 + n) - 1032 and (64 + n) - 72
struct DeqK { uint32_t magic_lo, magic_hi, nib_lo, nib_hi; h2q_t off_lo, off_hi; };
__device__ __forceinline__ void deq_ints(uint32_t w, const DeqK& c, h2q_t* t) {
  const uint32_t w8 = w >> 8;
  t[0] = __builtin_bit_cast(h2q_t, (w & c.nib_lo) | c.magic_lo) + c.off_lo;
  t[1] = __builtin_bit_cast(h2q_t, (w & c.nib_hi) | c.magic_hi) + c.off_hi;
  t[2] = __builtin_bit_cast(h2q_t, (w8 & c.nib_lo) | c.magic_lo) + c.off_lo;
  t[3] = __builtin_bit_cast(h2q_t, (w8 & c.nib_hi) | c.magic_hi) + c.off_hi;
}
// one word of a block -> the operand fragment (q - 8), exact in fp16, eight weights in the order deq_ints makes
__device__ __forceinline__ u4q_t deq_word(uint32_t w, const DeqK& c) {
  h2q_t t[4];
  deq_ints(w, c, t);
  return (u4q_t){__builtin_bit_cast(uint32_t, t[0]), __builtin_bit_cast(uint32_t, t[1]), __builtin_bit_cast(uint32_t, t[2]),
                 __builtin_bit_cast(uint32_t, t[3])};
}
// Lanes l, l + 16, l + 32, l + 48 hold the four 32-weight blocks of one step of a weight row, four words each.
// One matrix instruction is to cover ONE block (so that the block's scale can be applied to its result), i.e.
// lane group g has to supply word g of that block: a 4 x 4 transpose of words between the four lanes, done with
// the row-swap instructions of gfx950 (v_permlane32_swap: upper half of the first register <-> lower half of the
// second; v_permlane16_swap: odd 16-lane rows of the first <-> even rows of the second).  Afterwards word b of
// the result is word g of block b.
typedef uint32_t u2s_t __attribute__((ext_vector_type(2)));
__device__ __forceinline__ u4q_t transpose_blocks(u4q_t q) {
  const u2s_t a = __builtin_amdgcn_permlane32_swap(q.x, q.z, false, false);
  const u2s_t b = __builtin_amdgcn_permlane32_swap(q.y, q.w, false, false);
  const u2s_t c = __builtin_amdgcn_permlane16_swap(a.x, b.x, false, false);
  const u2s_t d = __builtin_amdgcn_permlane16_swap(a.y, b.y, false, false);
  return (u4q_t){c.x, c.y, d.x, d.y};
}
// the scales of the four blocks (lane group g holds block g's): all four to every lane, as float
__device__ __forceinline__ f4q_t gather_scales(_Float16 d) {
  const uint32_t v = (uint32_t)__builtin_bit_cast(uint16_t, d);
  const u2s_t a = __builtin_amdgcn_permlane32_swap(v, v, false, false);        // {d0 d1 d0 d1}, {d2 d3 d2 d3} by lane group
  const u2s_t lo = __builtin_amdgcn_permlane16_swap(a.x, a.x, false, false);   // {d0 d0 d0 d0}, {d1 d1 d1 d1}
  const u2s_t hi = __builtin_amdgcn_permlane16_swap(a.y, a.y, false, false);   // {d2 ...}, {d3 ...}
  auto f = [](uint32_t b) { return (float)__builtin_bit_cast(_Float16, (uint16_t)b); };
  return (f4q_t){f(lo.x), f(lo.y), f(hi.x), f(hi.y)};
}
#define DEQK_INIT(c)                                                                           \
  DeqK c = {0x64006400u, 0x54005400u, 0x000F000Fu, 0x00F000F0u,                                \
            {(_Float16)-1032.f, (_Float16)-1032.f}, {(_Float16)-72.f, (_Float16)-72.f}};       \
  asm volatile("" : "+v"(c.magic_lo)); /* opaque: lets instruction selection use the three-operand and-or */ \
  asm volatile("" : "+v"(c.magic_hi));                                                         \
  asm volatile("" : "+s"(c.nib_lo));                                                           \
  asm volatile("" : "+s"(c.nib_hi))
#define MFMA_F16(a, b, c) __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(h8q_t, a), __builtin_bit_cast(h8q_t, b), c, 0, 0, 0)

// Workgroup = NW waves, each with R tiles of 16 weight rows = 16 NW R weight rows x 16 MT activation rows.
// A pair of activation fragments (both planes) read from LDS feeds 2 R matrix instructions; the weights of a
// wave's R tiles are unpacked in its registers, block by block as the K loop needs them.  One step = 128 weights
// of K; the next step's weight words and activation pieces are loaded into registers while the matrix cores work
// on the current one.  The activation tile is staged by every workgroup, so wide workgroups (eight waves) move
// fewer bytes per flop: 28672x4096 at M = 512 went 434 -> 344 us with 256 instead of 128 weight rows per workgroup.
template <int MT, int R, int NW>
__global__ void __launch_bounds__(64 * NW)
k_gemm_q4_f16_tiled(const uint8_t* __restrict__ W, const __half* __restrict__ d16, const u4q_t* __restrict__ xh, const u4q_t* __restrict__ xl,
                     uint32_t K, uint32_t N, uint32_t M, uint32_t b_val, uint32_t c_val, uint32_t by_val, float* out,
                     const uint32_t* __restrict__ lb, const uint32_t* __restrict__ lc, const float* __restrict__ scale,
                     GemmSegs segs, uint32_t ksplit, uint32_t kper, float* __restrict__ part) {
  // (the first 14 dwords of the arguments are in registers when a wave starts; by_val bit 0 / 1: the weights' / the
  // result's element offset of op 0 is b_val / c_val -- known on the host -- instead of a load from lb / lc, which
  // the first weight loads would have to wait for)
  // ksplit > 1 (one op): blockIdx.z is a share of K -- kper blocks, a multiple of 4 -- and the tile's raw sums go to
  // part[share][row][n] for k_gemm_splitk_sum; wide tiles then still give every CU a workgroup on a narrow matrix.
  constexpr uint32_t BM = 16u * MT, ROWB = 272u;
  __shared__ __attribute__((aligned(16))) uint8_t xs[2u * BM * ROWB];   // first plane, then second plane
  uint8_t* const xs2 = xs + BM * ROWB;
  const uint32_t tid = threadIdx.x, lane = tid & 63u, wave = tid >> 6;
  const uint32_t r16 = lane & 15u, g = lane >> 4;
  constexpr uint32_t NT = 64u * NW, NP = 256u * MT / NT;       // threads; 16-byte pieces per thread, plane and step
  const uint32_t n0 = blockIdx.x * (16u * NW * R) + wave * (16u * R), m0 = blockIdx.y * BM;
  const uint32_t op = ksplit > 1u ? 0u : blockIdx.z, kz = ksplit > 1u ? blockIdx.z : 0u;
  const uint64_t c_off = (by_val & 2u) ? (uint64_t)c_val : (uint64_t)lc[op], gbase = ((by_val & 1u) ? (uint64_t)b_val : (uint64_t)lb[op]) >> 5;
  const uint32_t nblk = K >> 5, kw = K >> 3;                   // blocks and 16-byte pieces per row
  const uint32_t kb_lo = kz * kper, kb_hi = min(nblk, kb_lo + kper);   // this workgroup's blocks of K
  uint32_t nrow[R];
#pragma unroll
  for (int r = 0; r < R; r++) nrow[r] = min(n0 + r * 16u + r16, N - 1u);   // rows past N: clamped, not stored

  f4q_t acc[R][MT];
#pragma unroll
  for (int r = 0; r < R; r++)
#pragma unroll
    for (int t = 0; t < MT; t++) acc[r][t] = (f4q_t){0.f, 0.f, 0.f, 0.f};
  DEQK_INIT(dk);

  // staging: the tile's 16 pieces per row, plane and step; thread -> (row, piece) pairs, NP per thread
  uint64_t xoff[NP];
#pragma unroll
  for (uint32_t u = 0; u < NP; u++) {
    const uint32_t w = tid + u * NT, row = min(m0 + (w >> 4), M - 1u);   // rows past M: clamped, not stored
    xoff[u] = ((uint64_t)op * M + row) * kw + (w & 15u);
  }
  u4q_t xn[NP], xln[NP], qn[R];
  _Float16 dn[R];
  // always executed; the step past K re-reads the last one and is not used
#define GEMM_FETCH(kb_raw)                                                        \
  do {                                                                            \
    const uint32_t kb_ = min((kb_raw), kb_hi - 4u);                               \
    _Pragma("unroll") for (int r = 0; r < R; r++) {                               \
      const uint64_t gi = gbase + (uint64_t)nrow[r] * nblk + kb_ + g;             \
      qn[r] = *(const u4q_t*)(W + (gi << 4));                                     \
      dn[r] = __builtin_bit_cast(_Float16, d16[gi]);                              \
    }                                                                             \
    _Pragma("unroll") for (uint32_t u = 0; u < NP; u++) {                         \
      xn[u] = xh[xoff[u] + kb_ * 4u];                                             \
      xln[u] = xl[xoff[u] + kb_ * 4u];                                            \
    }                                                                             \
  } while (0)
  GEMM_FETCH(kb_lo);

  for (uint32_t kb0 = kb_lo; kb0 < kb_hi; kb0 += 4u) {
#pragma unroll
    for (uint32_t u = 0; u < NP; u++) {
      const uint32_t w = tid + u * NT;
      *(u4q_t*)(xs + (w >> 4) * ROWB + (w & 15u) * 16u) = xn[u];
      *(u4q_t*)(xs2 + (w >> 4) * ROWB + (w & 15u) * 16u) = xln[u];
    }
    u4q_t q[R];
    f4q_t ds[R];
#pragma unroll
    for (int r = 0; r < R; r++) { q[r] = transpose_blocks(qn[r]); ds[r] = gather_scales(dn[r]); }
    __syncthreads();
    GEMM_FETCH(kb0 + 4u);
#pragma unroll
    for (int b = 0; b < 4; b++) {      // one 32-weight block of the step at a time
      u4q_t wq[R];
#pragma unroll
      for (int r = 0; r < R; r++) wq[r] = deq_word(b == 0 ? q[r].x : b == 1 ? q[r].y : b == 2 ? q[r].z : q[r].w, dk);
      // TG activation tiles at a time: their first-plane instructions, then the second-plane ones (each depends on
      // one issued TG * R instructions earlier), then the scaling of the block results
      constexpr int TG = R >= 4 ? 2 : MT >= 4 ? 4 : MT;
#pragma unroll
      for (int t0 = 0; t0 < MT; t0 += TG) {
        u4q_t ah[TG], al[TG];
        f4q_t blk[TG][R];
#pragma unroll
        for (int t = 0; t < TG; t++) {
          const uint32_t xo = ((t0 + t) * 16u + r16) * ROWB + b * 64u + g * 16u;
          ah[t] = *(const u4q_t*)(xs + xo); al[t] = *(const u4q_t*)(xs2 + xo);
        }
#pragma unroll
        for (int t = 0; t < TG; t++)
#pragma unroll
          for (int r = 0; r < R; r++) blk[t][r] = MFMA_F16(ah[t], wq[r], ((f4q_t){0.f, 0.f, 0.f, 0.f}));
#pragma unroll
        for (int t = 0; t < TG; t++)
#pragma unroll
          for (int r = 0; r < R; r++) blk[t][r] = MFMA_F16(al[t], wq[r], blk[t][r]);
#pragma unroll
        for (int t = 0; t < TG; t++)
#pragma unroll
          for (int r = 0; r < R; r++) {
            const float d = ds[r][b];
#pragma unroll
            for (int i = 0; i < 4; i++) acc[r][t0 + t][i] = fmaf(blk[t][r][i], d, acc[r][t0 + t][i]);
          }
      }
    }
    __syncthreads();
  }
  // lane (r16, g) holds D[4g + i][r16]: activation rows m0 + 16 t + 4g + i, weight row n0 + 16 r + r16
#pragma unroll
  for (int t = 0; t < MT; t++)
#pragma unroll
    for (int i = 0; i < 4; i++) {
      const uint32_t row = m0 + t * 16u + 4u * g + i;
      if (row >= M) continue;
      if (ksplit > 1u) {   // raw sums of this share of K; scale and placement are k_gemm_splitk_sum's
        float* pr = part + ((uint64_t)kz * M + row) * N;
#pragma unroll
        for (int r = 0; r < R; r++) {
          const uint32_t n = n0 + r * 16u + r16;
          if (n < N) pr[n] = acc[r][t][i];
        }
        continue;
      }
      const float inv = scale[2 * ((uint64_t)op * M + row) + 1];
      float* c = out + c_off + (uint64_t)row * N;
#pragma unroll
      for (int r = 0; r < R; r++) {
        const uint32_t n = n0 + r * 16u + r16;
        if (n >= N) continue;
        if (segs.count) {   // stacked matrices: the row's own matrix and its result base
          uint32_t sgi = 0;
#pragma unroll
          for (uint32_t q = 1; q < 4; q++) sgi += (q < segs.count && n >= segs.begin[q]) ? 1u : 0u;
          out[segs.c[sgi] + (uint64_t)row * segs.n[sgi] + (n - segs.begin[sgi])] = acc[r][t][i] * inv;
        } else c[n] = acc[r][t][i] * inv;
      }
    }
}

#undef GEMM_FETCH

// The shares of K of a split launch of the kernel above, summed in the order of the shares, scaled by the row's factor
// and stored where the unsplit launch would have stored them (one op).  Four results per thread.
__global__ void __launch_bounds__(256)
k_gemm_splitk_sum(const float* __restrict__ part, uint32_t ksplit, uint32_t M, uint32_t N, float* out, uint32_t c_val,
                  uint32_t by_val, const uint32_t* __restrict__ lc, const float* __restrict__ scale, GemmSegs segs) {
  const uint64_t total = (uint64_t)M * N, i0 = ((uint64_t)blockIdx.x * 256u + threadIdx.x) * 4u;
  if (i0 >= total) return;
  const uint64_t c_off = (by_val & 2u) ? (uint64_t)c_val : (uint64_t)lc[0];
  float v[4];
  const bool whole = (N & 3u) == 0u;      // the four are one row's: one 16-byte load per share
  if (whole) {
    f4q_t a = *(const f4q_t*)(part + i0);
    for (uint32_t z = 1; z < ksplit; z++) {
      const f4q_t b = *(const f4q_t*)(part + z * total + i0);
      a[0] += b[0]; a[1] += b[1]; a[2] += b[2]; a[3] += b[3];
    }
    v[0] = a[0]; v[1] = a[1]; v[2] = a[2]; v[3] = a[3];
  } else {
#pragma unroll
    for (int e = 0; e < 4; e++) {
      float a = i0 + e < total ? part[i0 + e] : 0.f;
      for (uint32_t z = 1; z < ksplit; z++) a += i0 + e < total ? part[z * total + i0 + e] : 0.f;
      v[e] = a;
    }
  }
#pragma unroll
  for (int e = 0; e < 4; e++) {
    const uint64_t i = i0 + e;
    if (i >= total) break;
    const uint32_t row = (uint32_t)(i / N), n = (uint32_t)(i % N);
    const float y = v[e] * scale[2 * (uint64_t)row + 1];
    if (segs.count) {
      uint32_t sgi = 0;
#pragma unroll
      for (uint32_t q = 1; q < 4; q++) sgi += (q < segs.count && n >= segs.begin[q]) ? 1u : 0u;
      out[segs.c[sgi] + (uint64_t)row * segs.n[sgi] + (n - segs.begin[sgi])] = y;
    } else {
      out[c_off + (uint64_t)row * N + n] = y;
      if (segs.add) out[segs.dst + (uint64_t)row * N + n] = out[segs.res + (uint64_t)row * N + n] + y;   // the add behind it
    }
  }
}

// Few activation rows (M <= 32): the weights are read once and nothing is reused, so the work is
// bound by how fast they stream.  The NWV waves of a workgroup share R tiles of 16 weight rows and
// take every NWV-th step of K each (a matrix with few rows still spreads over the whole chip); every
// wave stages its own activation tile (both planes) from the fp16 copy into its own piece of LDS, so no
// workgroup barrier sits in the K loop.  The partial tiles are summed in wave order at the end.
// Eight waves keep twice as many loads in flight for matrices with few weight rows.
//
// Q8: the weights are Q8_0 blocks in the same block16 layout (32 code bytes, w = d (code - 128)): two 16-byte
// loads per block, bytes widened with a byte permute into the fp16 pairs (1024 + code), then -1152 and d
// (one term each for weights and activations).  `lc` null: the result rows go to out[row * N + n] (a scratch
// buffer of the caller).
template <int MT, int R, int NWV, bool Q8>
__global__ void __launch_bounds__(64 * NWV)
k_gemm_q4_f16_ksplit(const uint8_t* __restrict__ W, const __half* __restrict__ d16, const u4q_t* __restrict__ xh, const u4q_t* __restrict__ xl,
                     uint32_t K, uint32_t N, uint32_t M, uint32_t b_val, uint32_t c_val, uint32_t by_val, float* out,
                     const uint32_t* __restrict__ lb, const uint32_t* __restrict__ lc, const float* __restrict__ scale,
                     GemmSegs segs) {
  // (the first 14 dwords of the arguments are in registers when a wave starts; by_val bit 0 / 1: the weights' / the
  // result's element offset of op 0 is b_val / c_val -- known on the host -- instead of a load from lb / lc, which
  // the first weight loads would have to wait for)
  constexpr uint32_t BM = 16u * MT, ROWB = 272u, NP = 4u * MT;      // pieces per lane, plane and step
  constexpr uint32_t PLANES = Q8 ? 1u : 2u;
  constexpr uint32_t TILE = BM * ROWB, PART = (NWV - 1u) * R * MT * 4u * 64u * 4u;
  __shared__ __attribute__((aligned(16))) uint8_t xs_all[(NWV * PLANES * TILE > PART) ? NWV * PLANES * TILE : PART];
  const uint32_t tid = threadIdx.x, lane = tid & 63u;
  const uint32_t wave = (uint32_t)__builtin_amdgcn_readfirstlane((int)(tid >> 6));
  const uint32_t r16 = lane & 15u, g = lane >> 4;
  uint8_t* xs = xs_all + wave * PLANES * TILE;
  uint8_t* const xs2 = xs + TILE;
  const uint32_t n0 = blockIdx.x * (16u * R), m0 = blockIdx.y * BM, op = blockIdx.z;
  const uint64_t c_off = (by_val & 2u) ? (uint64_t)c_val : lc ? (uint64_t)lc[op] : 0ull;
  const uint64_t gbase = ((by_val & 1u) ? (uint64_t)b_val : (uint64_t)lb[op]) >> 5;
  const uint32_t nblk = K >> 5, kw = K >> 3;
  // Weight loads: lane -> (row lane / 4, block lane % 4 of the step), so the four lanes of a quad read 64
  // contiguous bytes of one row -- one request to the L1 instead of one per lane, which is what the
  // matrix-instruction layout (lane -> row lane % 16, block lane / 16) costs when loaded directly.
  // A cross-lane permute brings each 16-byte block (and its scale) to the lane that consumes it.
  const uint32_t lrow = lane >> 2, lblk = lane & 3u;
  const int perm_addr = (int)((4u * r16 + g) << 2);
  // segs.glu (R = 2, the matrix is [gate rows; up rows], N / 2 a multiple of 16): the workgroup's first tile is 16
  // gate rows and its second the 16 up rows that belong to them, so the gated activation can be stored from here
  const bool glum = R == 2 && segs.glu != 0u;
  uint32_t trow0[R], nrow[R];
#pragma unroll
  for (int r = 0; r < R; r++) {
    trow0[r] = glum ? (uint32_t)r * (N >> 1) + blockIdx.x * 16u : n0 + r * 16u;
    nrow[r] = min(trow0[r] + lrow, N - 1u);
  }

  f4q_t acc[R][MT];
#pragma unroll
  for (int r = 0; r < R; r++)
#pragma unroll
    for (int t = 0; t < MT; t++) acc[r][t] = (f4q_t){0.f, 0.f, 0.f, 0.f};
  DEQK_INIT(dk);
  const h2q_t off_q8 = {(_Float16)-1152.f, (_Float16)-1152.f};

  uint64_t xoff[NP];
#pragma unroll
  for (uint32_t u = 0; u < NP; u++) {
    const uint32_t w = lane + u * 64u, row = min(m0 + (w >> 4), M - 1u);
    xoff[u] = ((uint64_t)op * M + row) * kw + (w & 15u);
  }
  u4q_t xn[NP], xln[Q8 ? 1 : NP], qn[R], qn2[Q8 ? R : 1];
  _Float16 dn[R];
#define GEMM_FETCH(kb_raw)                                                        \
  do {                                                                            \
    const uint32_t kb_ = min((kb_raw), nblk - 4u);                                \
    _Pragma("unroll") for (int r = 0; r < R; r++) {                               \
      const uint64_t gi = gbase + (uint64_t)nrow[r] * nblk + kb_ + lblk;          \
      if (Q8) {                                                                   \
        qn[r] = *(const u4q_t*)(W + (gi << 5));                                   \
        qn2[r] = *(const u4q_t*)(W + (gi << 5) + 16);                             \
      } else qn[r] = *(const u4q_t*)(W + (gi << 4));                              \
      dn[r] = __builtin_bit_cast(_Float16, d16[gi]);                              \
    }                                                                             \
    _Pragma("unroll") for (uint32_t u = 0; u < NP; u++) {                         \
      xn[u] = xh[xoff[u] + kb_ * 4u];                                             \
      if (!Q8) xln[u] = xl[xoff[u] + kb_ * 4u];                                   \
    }                                                                             \
  } while (0)
  GEMM_FETCH(wave * 4u);

  for (uint32_t kb0 = wave * 4u; kb0 < nblk; kb0 += 4u * NWV) {
#pragma unroll
    for (uint32_t u = 0; u < NP; u++) {
      const uint32_t w = lane + u * 64u;
      *(u4q_t*)(xs + (w >> 4) * ROWB + (w & 15u) * 16u) = xn[u];
      if (!Q8) *(u4q_t*)(xs2 + (w >> 4) * ROWB + (w & 15u) * 16u) = xln[u];
    }
    // the step's blocks and scales, moved to the lanes that consume them
    u4q_t q[R], q2[Q8 ? R : 1];
    f4q_t ds[Q8 ? 1 : R];
    h2q_t d2[Q8 ? R : 1];
#pragma unroll
    for (int r = 0; r < R; r++) {
#define PERM_U4(v) (u4q_t){(uint32_t)__builtin_amdgcn_ds_bpermute(perm_addr, (int)(v).x), (uint32_t)__builtin_amdgcn_ds_bpermute(perm_addr, (int)(v).y), \
                           (uint32_t)__builtin_amdgcn_ds_bpermute(perm_addr, (int)(v).z), (uint32_t)__builtin_amdgcn_ds_bpermute(perm_addr, (int)(v).w)}
      q[r] = PERM_U4(qn[r]);
      if (Q8) q2[r] = PERM_U4(qn2[r]);
#undef PERM_U4
      const uint32_t dbits = (uint32_t)__builtin_amdgcn_ds_bpermute(perm_addr, (int)__builtin_bit_cast(uint16_t, dn[r]));
      const _Float16 dl = __builtin_bit_cast(_Float16, (uint16_t)dbits);
      if (Q8) d2[r] = (h2q_t){dl, dl};
      else { q[r] = transpose_blocks(q[r]); ds[r] = gather_scales(dl); }
    }
    __builtin_amdgcn_wave_barrier();
    GEMM_FETCH(kb0 + 4u * NWV);
    if (Q8) {
      // Q8_0 blocks: lane group g holds block g whole; instruction j takes code bytes 8j .. 8j+7 of each of the
      // four blocks, scaled before the product (one term each for weights and activations)
#pragma unroll
      for (int j = 0; j < 4; j++) {
        u4q_t wq[R];
#pragma unroll
        for (int r = 0; r < R; r++) {
          // piece j = code bytes 8j .. 8j+7 in two words; pair p = (byte p of the first, byte p of the second)
          const uint32_t w0 = j == 0 ? q[r].x : j == 1 ? q[r].z : j == 2 ? q2[r].x : q2[r].z;
          const uint32_t w1 = j == 0 ? q[r].y : j == 1 ? q[r].w : j == 2 ? q2[r].y : q2[r].w;
          uint32_t o[4];
#pragma unroll
          for (uint32_t p = 0; p < 4; p++) {
            const uint32_t t = __builtin_amdgcn_perm(w1, w0, 0x0C000C00u | ((4u + p) << 16) | p) | dk.magic_lo;
            o[p] = __builtin_bit_cast(uint32_t, (h2q_t)((__builtin_bit_cast(h2q_t, t) + off_q8) * d2[r]));
          }
          wq[r] = (u4q_t){o[0], o[1], o[2], o[3]};
        }
#pragma unroll
        for (int t = 0; t < MT; t++) {
          const u4q_t ah = *(const u4q_t*)(xs + (t * 16u + r16) * ROWB + g * 64u + j * 16u);
#pragma unroll
          for (int r = 0; r < R; r++) acc[r][t] = MFMA_F16(ah, wq[r], acc[r][t]);
        }
      }
    } else {
#pragma unroll
      for (int b = 0; b < 4; b++) {      // one 32-weight block of the step at a time
        u4q_t wq[R];
#pragma unroll
        for (int r = 0; r < R; r++) wq[r] = deq_word(b == 0 ? q[r].x : b == 1 ? q[r].y : b == 2 ? q[r].z : q[r].w, dk);
#pragma unroll
        for (int t = 0; t < MT; t++) {
          const uint32_t xo = (t * 16u + r16) * ROWB + b * 64u + g * 16u;
          const u4q_t ah = *(const u4q_t*)(xs + xo), al = *(const u4q_t*)(xs2 + xo);
          f4q_t blk[R];
#pragma unroll
          for (int r = 0; r < R; r++) blk[r] = MFMA_F16(ah, wq[r], ((f4q_t){0.f, 0.f, 0.f, 0.f}));
#pragma unroll
          for (int r = 0; r < R; r++) blk[r] = MFMA_F16(al, wq[r], blk[r]);
#pragma unroll
          for (int r = 0; r < R; r++) {
            const float d = ds[r][b];
#pragma unroll
            for (int i = 0; i < 4; i++) acc[r][t][i] = fmaf(blk[r][i], d, acc[r][t][i]);
          }
        }
      }
    }
    __builtin_amdgcn_wave_barrier();
  }
  // sum the waves' tiles in wave order; wave 0 stores
  __syncthreads();
  float* part = (float*)xs_all;
  if (wave > 0) {
#pragma unroll
    for (int r = 0; r < R; r++)
#pragma unroll
      for (int t = 0; t < MT; t++)
#pragma unroll
        for (int i = 0; i < 4; i++) part[((((wave - 1u) * R + r) * MT + t) * 4u + i) * 64u + lane] = acc[r][t][i];
  }
  __syncthreads();
  if (wave > 0) return;
#pragma unroll
  for (uint32_t w = 0; w < NWV - 1u; w++)
#pragma unroll
    for (int r = 0; r < R; r++)
#pragma unroll
      for (int t = 0; t < MT; t++)
#pragma unroll
        for (int i = 0; i < 4; i++) acc[r][t][i] += part[(((w * R + r) * MT + t) * 4u + i) * 64u + lane];
  // lane (r16, g) holds D[4g + i][r16]: activation rows m0 + 16 t + 4g + i, weight row n0 + 16 r + r16
#pragma unroll
  for (int t = 0; t < MT; t++)
#pragma unroll
    for (int i = 0; i < 4; i++) {
      const uint32_t row = m0 + t * 16u + 4u * g + i;
      if (row >= M) continue;
      const float inv = scale[2 * ((uint64_t)op * M + row) + 1];
      float* c = out + c_off + (uint64_t)row * N;
#pragma unroll
      for (int r = 0; r < R; r++) {
        const uint32_t n = trow0[r] + r16;
        if (n >= N) continue;
        if (segs.count) {   // stacked matrices: the row's own matrix and its result base
          uint32_t sgi = 0;
#pragma unroll
          for (uint32_t q = 1; q < 4; q++) sgi += (q < segs.count && n >= segs.begin[q]) ? 1u : 0u;
          out[segs.c[sgi] + (uint64_t)row * segs.n[sgi] + (n - segs.begin[sgi])] = acc[r][t][i] * inv;
        } else {
          const float y = acc[r][t][i] * inv;
          c[n] = y;
          if (segs.add) out[segs.dst + (uint64_t)row * N + n] = out[segs.res + (uint64_t)row * N + n] + y;
        }
      }
      if (glum && trow0[0] + r16 < (N >> 1)) {   // act(gate) * up, as the element-wise op computes it
        const float a = acc[0][t][i] * inv, b = acc[R - 1][t][i] * inv;
        out[segs.dst + (uint64_t)row * (N >> 1) + trow0[0] + r16] =
            segs.glu == 34u ? gelu_tanh(a) * b : (a / (1.0f + expf(-a))) * b;
      }
    }
}
#undef GEMM_FETCH

// M <= 16 and many weight rows: the waves of a workgroup take 16 weight rows each and share ONE activation tile per
// step of K, staged through LDS once for all of them (the K-split form above stages a tile per wave: the tile, both
// planes of all 16 rows, is 7x the bytes of a wave's weights, and those requests to the L1, not HBM, set its pace).
// A macro step is two steps of K (256 weights).  Registers hold rings of what is on its way: the workgroup's next
// four activation macro tiles (a thread's share: one or two pieces per plane each) and each wave's weights of the next
// four macro steps, so a CU keeps ~10 KB per wave in flight; LDS holds two macro tiles, one being read by the matrix
// instructions while the next is written, with one barrier per macro step.  Every load is issued on every path
// (clamped to the last step of K): the waits stay counted.
// segs.count: stacked matrices, as above.  segs.glu: [gate rows; up rows]: the first half of the waves takes gate
// tiles, the second half the up tiles that belong to them; the up waves hand their results over in LDS and the
// gate waves also store act(gate) * up at segs.dst.
#define R16_MS 2u
template <int NW>
__global__ void __launch_bounds__(64 * NW)
k_gemm_q4_f16_rows16(const uint8_t* __restrict__ W, const __half* __restrict__ d16, const u4q_t* __restrict__ xh, const u4q_t* __restrict__ xl,
                     uint32_t K, uint32_t N, uint32_t M, uint32_t b_val, uint32_t c_val, uint32_t by_val, float* out,
                     const uint32_t* __restrict__ lb, const uint32_t* __restrict__ lc, const float* __restrict__ scale,
                     GemmSegs segs) {
  // (the first 14 dwords of the arguments are in registers when a wave starts; by_val bit 0 / 1: the weights' / the
  // result's element offset of op 0 is b_val / c_val -- known on the host -- instead of a load from lb / lc, which
  // the first weight loads would have to wait for)
  constexpr uint32_t ROWB = 272u, TILE = 16u * ROWB, NT = 64u * NW;
  constexpr uint32_t PIECES = R16_MS * 256u;                 // 16-byte pieces per plane and macro step
  constexpr uint32_t NP = (PIECES + NT - 1u) / NT;           // per thread
  __shared__ __attribute__((aligned(16))) uint8_t xs_all[2u * 2u * R16_MS * TILE];   // [buffer][plane][step of the macro step]
  const uint32_t tid = threadIdx.x, lane = tid & 63u;
  const uint32_t wave = (uint32_t)__builtin_amdgcn_readfirstlane((int)(tid >> 6));
  const uint32_t r16 = lane & 15u, g = lane >> 4, op = blockIdx.z;
  const bool glum = segs.glu != 0u;
  // first weight row of the wave's tile (glu: tb = the tile's first row within its half of the matrix)
  const uint32_t tb = glum ? blockIdx.x * (8u * NW) + (wave % (NW / 2u)) * 16u : blockIdx.x * (16u * NW) + wave * 16u;
  const uint32_t n0 = glum && wave >= NW / 2u ? (N >> 1) + tb : tb;
  const uint64_t c_off = (by_val & 2u) ? (uint64_t)c_val : lc ? (uint64_t)lc[op] : 0ull;
  const uint64_t gbase = ((by_val & 1u) ? (uint64_t)b_val : (uint64_t)lb[op]) >> 5;
  const uint32_t nblk = K >> 5, kw = K >> 3, steps = nblk >> 2, macros = (steps + R16_MS - 1u) / R16_MS;
  const uint32_t lrow = lane >> 2, lblk = lane & 3u;
  const int perm_addr = (int)((4u * r16 + g) << 2);
  const uint64_t wrow = gbase + (uint64_t)min(n0 + lrow, N - 1u) * nblk + lblk;
  DEQK_INIT(dk);
  f4q_t acc = {0.f, 0.f, 0.f, 0.f};

  // a thread's pieces of a macro tile: piece w -> (step w / 256, row (w / 16) % 16, piece w % 16)
  uint64_t xoff[NP];
  uint32_t xlds[NP], xst[NP];
#pragma unroll
  for (uint32_t u = 0; u < NP; u++) {
    const uint32_t w = min(tid + u * NT, PIECES - 1u), row = (w >> 4) & 15u, pc = w & 15u;
    xst[u] = w >> 8;
    xoff[u] = ((uint64_t)op * M + min(row, M - 1u)) * kw + pc;     // + 16 pieces per step of K
    xlds[u] = xst[u] * TILE + row * ROWB + pc * 16u;
  }
  struct ActR { u4q_t h[NP], l[NP]; };
  struct WtR { u4q_t q[R16_MS]; uint32_t d[R16_MS]; };
  ActR a0, a1, a2, a3;
  WtR w0, w1, w2, w3;
  // (steps past the end of K ask for the last step again: not used)
  auto fetch_a = [&](ActR& a, uint32_t m) {
#pragma unroll
    for (uint32_t u = 0; u < NP; u++) {
      const uint64_t at = xoff[u] + min(m * R16_MS + xst[u], steps - 1u) * 16u;
      a.h[u] = xh[at]; a.l[u] = xl[at];
    }
  };
  auto fetch_w = [&](WtR& w, uint32_t m) {
#pragma unroll
    for (uint32_t s = 0; s < R16_MS; s++) {
      const uint64_t gi = wrow + min(m * R16_MS + s, steps - 1u) * 4u;
      w.q[s] = *(const u4q_t*)(W + (gi << 4));
      w.d[s] = (uint32_t)((const uint16_t*)d16)[gi];
    }
  };
  auto put_a = [&](const ActR& a, uint32_t buf) {
    uint8_t* b = xs_all + buf * (2u * R16_MS * TILE);
#pragma unroll
    for (uint32_t u = 0; u < NP; u++)
      if (NT * NP == PIECES || tid + u * NT < PIECES) {
        *(u4q_t*)(b + xlds[u]) = a.h[u];
        *(u4q_t*)(b + R16_MS * TILE + xlds[u]) = a.l[u];
      }
  };
  auto compute = [&](const WtR& w, uint32_t m, uint32_t buf) {
    const uint8_t* b0 = xs_all + buf * (2u * R16_MS * TILE);
#pragma unroll
    for (uint32_t s = 0; s < R16_MS; s++) {
      u4q_t q = {(uint32_t)__builtin_amdgcn_ds_bpermute(perm_addr, (int)w.q[s].x), (uint32_t)__builtin_amdgcn_ds_bpermute(perm_addr, (int)w.q[s].y),
                 (uint32_t)__builtin_amdgcn_ds_bpermute(perm_addr, (int)w.q[s].z), (uint32_t)__builtin_amdgcn_ds_bpermute(perm_addr, (int)w.q[s].w)};
      const uint32_t dbits = (uint32_t)__builtin_amdgcn_ds_bpermute(perm_addr, (int)w.d[s]);
      q = transpose_blocks(q);
      const f4q_t ds = gather_scales(__builtin_bit_cast(_Float16, (uint16_t)dbits));
      if (m * R16_MS + s < steps) {     // (uniform; the last macro step of an odd number of steps is half empty)
        const uint8_t* xs = b0 + s * TILE;
        const uint8_t* xs2 = xs + R16_MS * TILE;
#pragma unroll
        for (int b = 0; b < 4; b++) {
          const u4q_t wq = deq_word(b == 0 ? q.x : b == 1 ? q.y : b == 2 ? q.z : q.w, dk);
          const uint32_t xo = r16 * ROWB + b * 64u + g * 16u;
          const u4q_t ah = *(const u4q_t*)(xs + xo), al = *(const u4q_t*)(xs2 + xo);
          f4q_t blk = MFMA_F16(ah, wq, ((f4q_t){0.f, 0.f, 0.f, 0.f}));
          blk = MFMA_F16(al, wq, blk);
          const float d = ds[b];
#pragma unroll
          for (int i = 0; i < 4; i++) acc[i] = fmaf(blk[i], d, acc[i]);
        }
      }
    }
  };
  // prologue: activation tiles 0 .. 4 and weights 0 .. 3, in the order the loop issues them (a tile, then the weights
  // that go with it: loads return in order, and the tile is waited for first), so that the loop's first wait finds
  // the same loads behind its tile whether it is entered from here or from its own end
  fetch_a(a0, 0u);
  fetch_a(a1, 1u); fetch_w(w0, 0u); fetch_a(a2, 2u); fetch_w(w1, 1u); fetch_a(a3, 3u); fetch_w(w2, 2u);
  asm volatile("" ::: "memory");   // the loads stay here: none of them is moved below the first tile's wait
  __builtin_amdgcn_sched_barrier(0);
  put_a(a0, 0u);
  __builtin_amdgcn_sched_barrier(0);
  fetch_a(a0, 4u); fetch_w(w3, 3u);
  asm volatile("" ::: "memory");
  __builtin_amdgcn_sched_barrier(0);
  __syncthreads();
  // macro step m: tile m + 1 goes to LDS, tile m + 5 and the weights of m + 4 are asked for, m is computed
#define R16_STEP(AR, WR, mm)                                       \
  {                                                                \
    put_a(AR, ((mm) + 1u) & 1u);                                   \
    __builtin_amdgcn_sched_barrier(0);                             \
    fetch_a(AR, (mm) + 5u);                                        \
    __builtin_amdgcn_sched_barrier(0);                             \
    compute(WR, (mm), (mm) & 1u);                                  \
    __builtin_amdgcn_sched_barrier(0);                             \
    fetch_w(WR, (mm) + 4u);                                        \
    __builtin_amdgcn_sched_barrier(0);                             \
    __syncthreads();                                               \
  }
  // (four macro steps per round and one way out: steps past the end of K compute nothing)
  for (uint32_t m = 0; m < macros; m += 4u) {
    R16_STEP(a1, w0, m);
    R16_STEP(a2, w1, m + 1u);
    R16_STEP(a3, w2, m + 2u);
    R16_STEP(a0, w3, m + 3u);
  }
#undef R16_STEP
  // lane (r16, g) holds D[4g + i][r16]: activation row 4g + i, weight row n0 + r16
  const uint32_t n = n0 + r16;
  float y[4];
#pragma unroll
  for (int i = 0; i < 4; i++) {
    const uint32_t row = min(4u * g + i, M - 1u);
    y[i] = acc[i] * scale[2 * ((uint64_t)op * M + row) + 1];
  }
  float* ybuf = (float*)xs_all;            // the up waves' tiles, [wave - NW / 2][i][lane]
  if (glum && wave >= NW / 2u) {
#pragma unroll
    for (int i = 0; i < 4; i++) ybuf[((wave - NW / 2u) * 4u + i) * 64u + lane] = y[i];
  }
  if (glum) __syncthreads();
  const bool n_ok = glum ? tb + r16 < (N >> 1) : n < N;
#pragma unroll
  for (int i = 0; i < 4; i++) {
    const uint32_t row = 4u * g + i;
    if (row >= M || !n_ok) continue;
    if (segs.count) {
      uint32_t sgi = 0;
#pragma unroll
      for (uint32_t q = 1; q < 4; q++) sgi += (q < segs.count && n >= segs.begin[q]) ? 1u : 0u;
      out[segs.c[sgi] + (uint64_t)row * segs.n[sgi] + (n - segs.begin[sgi])] = y[i];
    } else out[c_off + (uint64_t)row * N + n] = y[i];
    if (glum && wave < NW / 2u) {
      const float a = y[i], b = ybuf[(wave * 4u + i) * 64u + lane];
      out[segs.dst + (uint64_t)row * (N >> 1) + n] = segs.glu == 34u ? gelu_tanh(a) * b : (a / (1.0f + expf(-a))) * b;
    }
  }
}

// The same conversion with the row held in registers: 1024 threads, thread t owns the 8-element words
// t, t + 1024, ... (NW of them; K <= 8192 NW), so the row makes one trip from memory instead of two
// dependent passes -- the rows of a decode batch are few and each workgroup's latency is the launch's.
// GLU: the rows are first produced here, as the gated activation of two inputs (element offsets glu.a, glu.b; the
// float32 result goes to glu.d, as the element-wise op stores it: op2 34 = GELU(a) b, 35 = SiLU(a) b), so the op and
// the conversion of its result are one launch and one trip.
struct GluSrc { uint32_t op, a, b, d; };
template <int NW, bool GLU>
__global__ void __launch_bounds__(1024)
k_act_f16_regs(const float* act, uint32_t K, uint32_t M, uint32_t a_val, uint32_t a_by_val, uint4* xh, uint4* xl, float* scale,
               float* act_out, const uint32_t* __restrict__ la, GluSrc glu) {
  // (a_by_val: the rows start at element a_val -- known on the host -- instead of la[op], a load the rows' loads
  // would wait for; with GLU a_val is glu.a)
  __shared__ float red[16];
  const uint32_t row = blockIdx.x, op = blockIdx.y, tid = threadIdx.x, kw = K >> 3;
  const float* x = act + (a_by_val ? (uint64_t)a_val : (uint64_t)la[op]) + (uint64_t)row * K;
  f4qu_t v0[NW], v1[NW];
  float m = 0.f;
#pragma unroll
  for (int u = 0; u < NW; u++) {
    const uint32_t w = tid + 1024u * u;
    if (w < kw) {
      v0[u] = *(const f4qu_t*)(x + w * 8u);
      v1[u] = *(const f4qu_t*)(x + w * 8u + 4u);
      if (GLU) {
        const float* y = act + (uint64_t)glu.b + (uint64_t)row * K + w * 8u;
        const f4qu_t y0 = *(const f4qu_t*)y, y1 = *(const f4qu_t*)(y + 4);
        auto f = [&](float a, float b) { return glu.op == 34u ? gelu_tanh(a) * b : (a / (1.0f + expf(-a))) * b; };
        v0[u] = (f4qu_t){f(v0[u].x, y0.x), f(v0[u].y, y0.y), f(v0[u].z, y0.z), f(v0[u].w, y0.w)};
        v1[u] = (f4qu_t){f(v1[u].x, y1.x), f(v1[u].y, y1.y), f(v1[u].z, y1.z), f(v1[u].w, y1.w)};
        float* d = act_out + (uint64_t)glu.d + (uint64_t)row * K + w * 8u;
        *(f4qu_t*)d = v0[u];
        *(f4qu_t*)(d + 4) = v1[u];
      }
      m = fmaxf(m, fmaxf(fmaxf(fmaxf(fabsf(v0[u].x), fabsf(v0[u].y)), fmaxf(fabsf(v0[u].z), fabsf(v0[u].w))),
                         fmaxf(fmaxf(fabsf(v1[u].x), fabsf(v1[u].y)), fmaxf(fabsf(v1[u].z), fabsf(v1[u].w)))));
    }
  }
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) m = fmaxf(m, __shfl_xor(m, o, 64));
  if ((tid & 63u) == 0) red[tid >> 6] = m;
  __syncthreads();
  m = red[0];
#pragma unroll
  for (int i = 1; i < 16; i++) m = fmaxf(m, red[i]);
  const uint32_t e = (__float_as_uint(m) >> 23) & 0xFFu;
  float s = 1.f, inv = 1.f;
  if (e >= 14u && e <= 254u) { s = __uint_as_float((267u - e) << 23); inv = __uint_as_float((e - 13u) << 23); }
  if (tid == 0) {
    scale[2 * ((uint64_t)op * M + row)] = s;
    scale[2 * ((uint64_t)op * M + row) + 1] = inv;
  }
  const uint64_t o0 = ((uint64_t)op * M + row) * kw;
#pragma unroll
  for (int u = 0; u < NW; u++) {
    const uint32_t w = tid + 1024u * u;
    if (w >= kw) continue;
    const float v[8] = {v0[u].x * s, v0[u].y * s, v0[u].z * s, v0[u].w * s, v1[u].x * s, v1[u].y * s, v1[u].z * s, v1[u].w * s};
    uint4 hi, lo;
    split_word(v, &hi, &lo);
    xh[o0 + w] = hi;
    xl[o0 + w] = lo;
  }
}

static float* g_scale_buf = nullptr;
static uint4* g_xh_buf = nullptr;     // fp16 activations: first plane, then the second plane at g_xh_plane bytes
static size_t g_xh_cap = 0;           // in bytes (both planes)
static size_t g_scale_cap = 0;
// The rows last converted into g_xh_buf / g_scale_buf, and the launch and upload counts right after the
// matmul that used them: while both counts stand still nothing has written device memory since, so a
// matmul over the same rows (K and V after Q, up after gate) skips the conversion launch.  plane = byte
// offset of the second plane those rows were written with.
static struct { const void* buf; uint64_t a; uint32_t M, K; uint64_t dispatch, mem_gen; size_t plane; bool valid; } g_xh_key = {};

static float* g_part_buf = nullptr;   // raw sums of the shares of a K-split launch
static size_t g_part_cap = 0;
static bool ensure_part_buf(size_t floats) {
  if (floats <= g_part_cap) return true;
  layout_changed();
  if (g_part_buf) { hipStreamSynchronize(g.stream); hipFree(g_part_buf); }
  g_part_cap = floats;
  if (hipMalloc((void**)&g_part_buf, g_part_cap * sizeof(float)) != hipSuccess) { (void)hipGetLastError(); g_part_buf = nullptr; g_part_cap = 0; return false; }
  return true;
}

static bool ensure_act_bufs(size_t scale_floats, size_t xh_bytes) {
  if (scale_floats > g_scale_cap) {
    layout_changed();
    if (g_scale_buf) { hipStreamSynchronize(g.stream); hipFree(g_scale_buf); }
    g_xh_key.valid = false;
    g_scale_cap = std::max<size_t>(scale_floats, 8192);
    if (hipMalloc((void**)&g_scale_buf, g_scale_cap * sizeof(float)) != hipSuccess) { g_scale_buf = nullptr; g_scale_cap = 0; return false; }
  }
  if (xh_bytes > g_xh_cap) {
    layout_changed();
    if (g_xh_buf) { hipStreamSynchronize(g.stream); hipFree(g_xh_buf); }
    g_xh_key.valid = false;
    g_xh_cap = xh_bytes;
    if (hipMalloc((void**)&g_xh_buf, g_xh_cap) != hipSuccess) { g_xh_buf = nullptr; g_xh_cap = 0; return false; }
  }
  return true;
}

bool gemm_act_slots(uint32_t M, uint32_t K, float** scale, __half** xh, __half** xl) {
  if (tuning("ADAMAH_GEMM_REUSE", 1) == 0) return false;
  const size_t plane = (size_t)M * K * 2;
  if (!ensure_act_bufs((size_t)2 * M, 2 * plane)) return false;
  g_xh_key.valid = false;   // the buffers are about to be rewritten
  *scale = g_scale_buf;
  *xh = (__half*)g_xh_buf;
  *xl = (__half*)((uint8_t*)g_xh_buf + plane);
  return true;
}

void gemm_act_mark(const void* buf, uint64_t a, uint32_t M, uint32_t K) {
  g_xh_key = {buf, a, M, K, g.stats.dispatch, g.mem_gen, (size_t)M * K * 2, true};
}

// Gated activation (op2 34 / 35) of the [M, K] rows at a and b into the rows at d, together with the fp16 form of
// the result that a batched matmul over those rows reads: one launch, and the matmul that follows skips its
// conversion.  false: not taken (nothing launched).
bool launch_glu_act_f16(const Map* ma, uint32_t op, uint32_t a, uint32_t b, uint32_t d, uint32_t M, uint32_t K) {
  if (K > 16384u || (K & 7u) || M == 0 || knob("ADAMAH_ACT_REGS", 1) == 0) return false;
  float* scale; __half *xh, *xl;
  if (!gemm_act_slots(M, K, &scale, &xh, &xl)) return false;
  float* act = (float*)ma->buf;
  const GluSrc glu = {op, a, b, d};
  if (K <= 8192) k_act_f16_regs<1, true><<<dim3(M, 1), 1024, 0, g.stream>>>(act, K, M, a, 1u, (uint4*)xh, (uint4*)xl, scale, act, nullptr, glu);
  else k_act_f16_regs<2, true><<<dim3(M, 1), 1024, 0, g.stream>>>(act, K, M, a, 1u, (uint4*)xh, (uint4*)xl, scale, act, nullptr, glu);
  count_launch();
  gemm_act_mark(ma->buf, d, M, K);
  return true;
}

// Merge of the attention slices of a lockstep step, one workgroup per sequence: the outputs of all the sequence's
// heads (partial[(row * heads + head) * splits + s] = {max, sum, values[D]}, at most 8 slices) are merged with the
// operations of the stand-alone merge kernel in their order, stored as the float32 row out[o0 + row * K ...]
// (K = heads * D), and converted to the fp16 form the O-projection's matmul reads -- the row is in registers, so its
// maximum costs one workgroup-wide reduction instead of a launch.
template <int NW>
__global__ void __launch_bounds__(1024)
k_attn_merge_rows_f16(float* out, const float* __restrict__ partial, uint32_t o0, uint32_t M, uint32_t K, uint32_t D,
                      uint32_t splits, float* scale, uint4* xh, uint4* xl) {
  __shared__ float red[16];
  const uint32_t row = blockIdx.x, tid = threadIdx.x, kw = K >> 3, heads = K / D, stride = D + 2u, last = splits - 1u;
  float v[NW][8];
  float m = 0.f;
#pragma unroll
  for (int u = 0; u < NW; u++) {
    const uint32_t w = min(tid + 1024u * u, kw - 1u), head = (w * 8u) / D, j0 = (w * 8u) % D;
    const float* pp = partial + (uint64_t)(row * heads + head) * splits * stride;
    float ms[8], ls[8];
#pragma unroll
    for (uint32_t sp = 0; sp < 8u; sp++) { const float* ps = pp + (uint64_t)min(sp, last) * stride; ms[sp] = ps[0]; ls[sp] = ps[1]; }
    float Mx = -9.99999968e+37f;
#pragma unroll
    for (uint32_t sp = 0; sp < 8u; sp++) Mx = sp < splits ? fmaxf(Mx, ms[sp]) : Mx;
    float e[8], t[8];
#pragma unroll
    for (uint32_t sp = 0; sp < 8u; sp++) {
      e[sp] = sp < splits ? expf(ms[sp] - Mx) : 0.f;
      t[sp] = sp < splits ? fmaf(ls[sp], e[sp], 0.f) : 0.f;
    }
    // the sum of a 64-lane butterfly over lanes 0 .. 7, as the merge kernel takes it
    const float invL = 1.0f / (((t[0] + t[4]) + (t[2] + t[6])) + ((t[1] + t[5]) + (t[3] + t[7])));
    float o[8] = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (uint32_t half = 0; half < 2u; half++) {
      if (half == 1u && splits <= 4u) break;
      f4qu_t a[4], b[4];
#pragma unroll
      for (uint32_t q = 0; q < 4u; q++) {
        const float* ps = pp + (uint64_t)min(half * 4u + q, last) * stride + 2 + j0;
        a[q] = *(const f4qu_t*)ps; b[q] = *(const f4qu_t*)(ps + 4);
      }
#pragma unroll
      for (uint32_t q = 0; q < 4u; q++) {
        const uint32_t sp = half * 4u + q;
        const float wg = e[sp];
        if (sp < splits) {
          o[0] += fmaf(a[q].x, wg, 0.f); o[1] += fmaf(a[q].y, wg, 0.f); o[2] += fmaf(a[q].z, wg, 0.f); o[3] += fmaf(a[q].w, wg, 0.f);
          o[4] += fmaf(b[q].x, wg, 0.f); o[5] += fmaf(b[q].y, wg, 0.f); o[6] += fmaf(b[q].z, wg, 0.f); o[7] += fmaf(b[q].w, wg, 0.f);
        }
      }
    }
#pragma unroll
    for (int k = 0; k < 8; k++) v[u][k] = o[k] * invL;
    if (tid + 1024u * u < kw) {
      float* d = out + (uint64_t)o0 + (uint64_t)row * K + w * 8u;
      *(f4qu_t*)d = (f4qu_t){v[u][0], v[u][1], v[u][2], v[u][3]};
      *(f4qu_t*)(d + 4) = (f4qu_t){v[u][4], v[u][5], v[u][6], v[u][7]};
#pragma unroll
      for (int k = 0; k < 8; k++) m = fmaxf(m, fabsf(v[u][k]));
    }
  }
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) m = fmaxf(m, __shfl_xor(m, o, 64));
  if ((tid & 63u) == 0) red[tid >> 6] = m;
  __syncthreads();
  m = red[0];
#pragma unroll
  for (int i = 1; i < 16; i++) m = fmaxf(m, red[i]);
  const uint32_t ex = (__float_as_uint(m) >> 23) & 0xFFu;
  float s = 1.f, inv = 1.f;
  if (ex >= 14u && ex <= 254u) { s = __uint_as_float((267u - ex) << 23); inv = __uint_as_float((ex - 13u) << 23); }
  if (tid == 0) { scale[2 * (uint64_t)row] = s; scale[2 * (uint64_t)row + 1] = inv; }
#pragma unroll
  for (int u = 0; u < NW; u++) {
    const uint32_t w = tid + 1024u * u;
    if (w >= kw) continue;
    const float x[8] = {v[u][0] * s, v[u][1] * s, v[u][2] * s, v[u][3] * s, v[u][4] * s, v[u][5] * s, v[u][6] * s, v[u][7] * s};
    uint4 hi, lo;
    split_word(x, &hi, &lo);
    xh[(uint64_t)row * kw + w] = hi;
    xl[(uint64_t)row * kw + w] = lo;
  }
}

// The launch of the kernel above: M sequences' merged heads as rows [M, K] at element o0 of the map, plus their fp16
// form for the matmul that follows.  false: not taken (nothing launched).
bool launch_attn_merge_rows_f16(const Map* ma, const float* partial, uint32_t o0, uint32_t M, uint32_t K, uint32_t D,
                                uint32_t splits) {
  if (K > 8192u || (K & 7u) || (D & 7u) || K % D || splits < 2 || splits > 8 || M == 0 || knob("ADAMAH_ACT_REGS", 1) == 0) return false;
  float* scale; __half *xh, *xl;
  if (!gemm_act_slots(M, K, &scale, &xh, &xl)) return false;
  k_attn_merge_rows_f16<1><<<M, 1024, 0, g.stream>>>((float*)ma->buf, partial, o0, M, K, D, splits, scale, (uint4*)xh, (uint4*)xl);
  count_launch();
  gemm_act_mark(ma->buf, o0, M, K);
  return true;
}

// Forget converted rows (after a stream capture: the launch count is rewound there, and the note must not
// survive into a later state with the same count).
void gemm_act_forget() { g_xh_key.valid = false; }

// Preconditions (checked by the caller against the host copies of the handles): Q4 map whose blocks
// in range are in the block16 layout, K a multiple of 128, weight bases block aligned, all operands
// in range.
// Shares of K a one-op Q4 matmul of M rows is cut into (1: one launch): 2 .. 4 where the widest tile (256 weight rows
// x 128 rows) would give fewer than three quarters of the CUs a workgroup and the shares fill them, each share at
// least 1024 elements long.
uint32_t gemm_q4_k_shares(uint32_t M, uint32_t K, uint32_t N) {
  if (M < 128 || tuning("ADAMAH_GEMM_SPLITK", 1) == 0) return 1;
  const uint64_t w256 = (uint64_t)cdiv(N, 256) * cdiv(M, 128);
  if (w256 * 4 >= 3ull * (uint64_t)g.n_cu) return 1;
  uint32_t sp = (uint32_t)std::min<uint64_t>(4, (uint64_t)g.n_cu / std::max<uint64_t>(1, w256));
  while (sp > 1 && K / sp < 1024u) sp--;
  return sp > 1 && w256 * sp * 4 >= 3ull * (uint64_t)g.n_cu ? sp : 1u;
}

int launch_gemm_q4_mfma(const Map* ma, const Map* mw, const uint32_t* la, const uint32_t* lb, const uint32_t* lc,
                        uint32_t M, uint32_t K, uint32_t N, uint32_t n_ops, bool q8, float* out, int64_t a_host,
                        int64_t c_host, const GemmSegs* segs, int64_t b_host) {
  // offsets of op 0 the host knows go to the kernels by value
  const uint32_t b_val = b_host >= 0 ? (uint32_t)b_host : 0u, c_val = c_host >= 0 ? (uint32_t)c_host : 0u;
  const uint32_t by_val = n_ops == 1 ? ((b_host >= 0 ? 1u : 0u) | (c_host >= 0 ? 2u : 0u)) : 0u;
  if (((q8 || out) && M > 32) || ((out || segs) && n_ops != 1) || (out && segs) || (segs && segs->glu && M > 32) ||
      (segs && segs->add && M > 32 && (n_ops != 1 || q8 || gemm_q4_k_shares(M, K, N) < 2)))
    return ADAMAH_ERR_INVALID;
  GemmSegs sg = {};
  if (segs) sg = *segs;
  const size_t need = (size_t)2 * M * n_ops;
  const size_t plane = (size_t)n_ops * M * K * 2;
  const bool reuse = g_xh_key.valid && n_ops == 1 && a_host >= 0 && g_xh_key.buf == ma->buf && g_xh_key.a == (uint64_t)a_host &&
                     g_xh_key.M == M && g_xh_key.K == K && g_xh_key.dispatch == g.stats.dispatch &&
                     g_xh_key.mem_gen == g.mem_gen && g_xh_key.plane == plane && tuning("ADAMAH_GEMM_REUSE", 1) != 0;
  g_xh_key.valid = false;
  // after the matmul: the converted rows stay usable if the result did not land on them
  auto keep = [&]() {
    if (n_ops != 1 || a_host < 0 || (c_host < 0 && !out)) return;
    const uint64_t a0 = (uint64_t)a_host, a1 = a0 + (uint64_t)M * K, c0 = (uint64_t)c_host, c1 = c0 + (uint64_t)M * N;
    if (!out && c0 < a1 && a0 < c1) return;
    g_xh_key = {ma->buf, a0, M, K, g.stats.dispatch, g.mem_gen, plane, true};
  };
  if (!reuse && !ensure_act_bufs(need, 2 * plane)) return ADAMAH_ERR_MEMORY;
  float* act = (float*)ma->buf;
  uint32_t mt = M <= 16 ? 1 : M <= 32 ? 2 : M <= 64 ? 4 : 8;
  uint4* const xh = g_xh_buf;
  uint4* const xl = (uint4*)((uint8_t*)g_xh_buf + plane);
  if (!reuse) {
    if (K <= 16384 && knob("ADAMAH_ACT_REGS", 1) != 0) {
      if (K <= 8192) k_act_f16_regs<1, false><<<dim3(M, n_ops), 1024, 0, g.stream>>>(act, K, M, a_host >= 0 ? (uint32_t)a_host : 0u, (a_host >= 0 && n_ops == 1) ? 1u : 0u, xh, xl, g_scale_buf, act, la, GluSrc{});
      else k_act_f16_regs<2, false><<<dim3(M, n_ops), 1024, 0, g.stream>>>(act, K, M, a_host >= 0 ? (uint32_t)a_host : 0u, (a_host >= 0 && n_ops == 1) ? 1u : 0u, xh, xl, g_scale_buf, act, la, GluSrc{});
    } else
      k_act_f16<<<dim3(M, n_ops), 256, 0, g.stream>>>(act, la, M, K, g_scale_buf, xh, xl);
    count_launch();
  }
  auto wgs = [&](uint32_t rows_per_wg, uint32_t t) { return (uint64_t)cdiv(N, rows_per_wg) * cdiv(M, 16 * t) * n_ops; };
  const uint64_t want = 2ull * (uint64_t)g.n_cu;
  if (mt <= 2) {
    // few activation rows: the K-split form, as many weight-row tiles per workgroup as still fill the chip
    uint32_t R = wgs(64, mt) >= want ? 4 : wgs(32, mt) >= want ? 2 : 1;
    R = (uint32_t)knob("ADAMAH_GEMM_R", (int)R);
    R = R >= 4 ? 4 : R >= 2 ? 2 : 1;
    if (q8 && R > 2) R = 2;   // a Q8 tile holds twice the registers
    if (sg.glu) {             // a workgroup pairs one gate tile with its up tile
      if (sg.count != 2 || sg.n[0] != sg.n[1] || (sg.n[0] & 15u)) return ADAMAH_ERR_INVALID;
      R = 2;
    }
    // many weight rows under at most 16 activation rows: the form whose eight waves share the activation tile, when
    // its workgroups of 128 weight rows still cover three quarters of the CUs (28672x4096: 28.5 against 32.5 us)
    {
      const bool glu_ok = !sg.glu || (sg.count == 2 && sg.n[0] == sg.n[1] && (sg.n[0] & 15u) == 0);
      const uint32_t wgs16 = cdiv(sg.glu ? N / 2 : N, sg.glu ? 64u : 128u);
      if (mt == 1 && !q8 && !sg.add && glu_ok && (uint64_t)wgs16 * 4 >= 3ull * (uint64_t)g.n_cu &&
          tuning("ADAMAH_GEMM_ROWS16", 1) != 0) {
        dim3 gridr(wgs16, 1, n_ops);
        k_gemm_q4_f16_rows16<8><<<gridr, 512, 0, g.stream>>>(mw->buf, mw->d16, (const u4q_t*)xh, (const u4q_t*)xl, K, N, M, b_val, c_val,
                                                            out ? (by_val & 1u) : by_val, out ? out : act, lb, out ? nullptr : lc,
                                                            g_scale_buf, sg);
        count_launch();
        keep();
        return check_launch();
      }
    }
    dim3 grid(cdiv(N, 16 * R), cdiv(M, 16 * mt), n_ops);
    float* dst = out ? out : act;
    const uint32_t* lcd = out ? nullptr : lc;
    // eight waves where the matrix has too few weight rows for larger tiles (measured: no gain otherwise)
    const uint32_t nwv = mt == 1 && !q8 ? (uint32_t)knob("ADAMAH_GEMM_NWV", R == 1 ? 8 : 4) : 4u;
#define GK(T, RR, W, Q) k_gemm_q4_f16_ksplit<T, RR, W, Q><<<grid, 64 * W, 0, g.stream>>>(mw->buf, mw->d16, (const u4q_t*)xh, (const u4q_t*)xl, K, N, M, b_val, c_val, out ? (by_val & 1u) : by_val, dst, lb, lcd, g_scale_buf, sg)
    if (q8) {
      if (mt == 1) { if (R == 2) GK(1, 2, 4, true); else GK(1, 1, 4, true); }
      else { if (R == 2) GK(2, 2, 4, true); else GK(2, 1, 4, true); }
    }
    else if (mt == 1 && nwv >= 8) { if (R == 4) GK(1, 4, 8, false); else if (R == 2) GK(1, 2, 8, false); else GK(1, 1, 8, false); }
    else if (mt == 1) { if (R == 4) GK(1, 4, 4, false); else if (R == 2) GK(1, 2, 4, false); else GK(1, 1, 4, false); }
    else { if (R == 4) GK(2, 4, 4, false); else if (R == 2) GK(2, 2, 4, false); else GK(2, 1, 4, false); }
#undef GK
    count_launch();
    keep();
    return check_launch();
  }
  // Tile per workgroup: 16 NW R weight rows x 16 MT activation rows (NW waves with R tiles of 16 weight rows each).
  // Every workgroup stages its activation tile (two fp16 planes: 64 KB per step of 128 weights at MT = 8) from L2,
  // while its weights are 4.5 bits each, so the bytes a workgroup moves per flop fall with the number of weight
  // rows it covers: 512 (eight waves, R = 4) where the matrix still gives most CUs a workgroup, else 128 / 64.
  uint32_t R = 1, NW = 4;
  if (mt == 8) {
    if (wgs(256, 8) * 4 >= 3ull * (uint64_t)g.n_cu) { R = 2; NW = 8; }
    else if (wgs(128, 8) >= want) R = 2;
    else if (wgs(64, 8) >= want) R = 1;
    else mt = 4;
  }
  if (mt == 8 && knob("ADAMAH_GEMM_MT", 8) == 4) { mt = 4; NW = 4; R = 1; }
  R = (uint32_t)knob("ADAMAH_GEMM_R", (int)R);
  NW = (uint32_t)knob("ADAMAH_GEMM_NW", (int)NW) >= 8 ? 8 : 4;
  R = R >= 4 && mt == 4 ? 4 : R >= 2 ? 2 : 1;
  if (mt == 4 && NW == 8 && R == 1) R = 2;
  // A narrow matrix under many rows (N = 4096 / 6144 at M = 512) gives the widest tile (256 weight rows x 128 rows)
  // too few workgroups for the chip, and the smaller tiles that do fill it re-stage more activations per flop: there
  // the widest tile is launched over 2 .. 4 shares of K, raw sums into scratch, and a second launch adds the shares.
  uint32_t ksplit = 1, kper = K >> 5;
  {
    const uint32_t sp = n_ops == 1 && !q8 && !out ? gemm_q4_k_shares(M, K, N) : 1u;
    if (sp > 1 && ensure_part_buf((size_t)sp * M * N)) {
      ksplit = sp; mt = 8; R = 2; NW = 8;
      kper = cdiv(cdiv(K >> 5, ksplit), 4u) * 4u;
      ksplit = cdiv(K >> 5, kper);
    } else if (sg.add && M > 32) return ADAMAH_ERR_MEMORY;   // (only the split launch stores the add of many rows)
  }
  dim3 grid(cdiv(N, 16 * NW * R), cdiv(M, 16 * mt), ksplit > 1 ? ksplit : n_ops);
#define GT(T, RR, W) k_gemm_q4_f16_tiled<T, RR, W><<<grid, 64 * W, 0, g.stream>>>(mw->buf, mw->d16, (const u4q_t*)xh, (const u4q_t*)xl, K, N, M, b_val, c_val, by_val, act, lb, lc, g_scale_buf, sg, ksplit, kper, g_part_buf)
  if (ksplit > 1) {
    GT(8, 2, 8);
    count_launch();
    const uint64_t quads = ((uint64_t)M * N + 3) / 4;
    k_gemm_splitk_sum<<<cdiv(quads, 256), 256, 0, g.stream>>>(g_part_buf, ksplit, M, N, act, c_val, by_val, lc, g_scale_buf, sg);
  }
  else if (mt == 4 && NW == 8) { if (R == 4) GT(4, 4, 8); else GT(4, 2, 8); }
  else if (mt == 4) { if (R == 4) GT(4, 4, 4); else if (R == 2) GT(4, 2, 4); else GT(4, 1, 4); }
  else if (NW == 8) { if (R == 2) GT(8, 2, 8); else GT(8, 1, 8); }
  else { if (R == 2) GT(8, 2, 4); else GT(8, 1, 4); }
#undef GT
  count_launch();
  keep();
  return check_launch();
}

void gemm_q4_mfma_release() {
  if (g_scale_buf) hipFree(g_scale_buf);
  g_scale_buf = nullptr;
  g_scale_cap = 0;
  if (g_xh_buf) hipFree(g_xh_buf);
  g_xh_buf = nullptr;
  g_xh_cap = 0;
  g_xh_key.valid = false;
  if (g_part_buf) hipFree(g_part_buf);
  g_part_buf = nullptr;
  g_part_cap = 0;
}

}  // namespace adamah
