// Q4 dequant-GEMV with the 4x4x4 int8 matrix instruction used as a dot-product unit.
//
// Semantics as in gemv_q.hip (reference: shaders/src/f32/map_matvec_t_xq4.comp:49-135; argmax tail
// map_matvec_argmax_t_xq4.comp:66-158, map_argmax_pairs.comp:34-67).
//
// Why not plain VALU: with one convert and one FMA per weight (or one v_dot2 per two weights plus
// unpacking) the kernel keeps the vector ALUs busy for most of its run time: it is bound by
// instruction issue, not by HBM.  v_mfma_i32_4x4x4_16B_i8 multiplies sixteen independent 4x4x4
// blocks per instruction; block g lives in lanes 4g..4g+3, operand A row i and operand B column j
// both come from lane 4g+i / 4g+j (four k values, one byte each), and lane 4g+j receives column j
// of the result.  Used here as
//   B column j = four 4-bit codes of lane j's own weight row, one per byte:  w & 0x0F0F0F0F and
//                (w >> 4) & 0x0F0F0F0F are all the unpacking there is (3 VALU ops per 8 weights);
//   A row i    = digit i of the matching four activations, which are held as 22-bit fixed point
//                x * 2^e = d0 * 2^14 + d1 * 2^7 + d2  (d0 signed, d1, d2 in 0..127; e per 32-block
//                from the block's max |x|), rows 0..2 used, row 3 repeats row 0;
// so every lane ends up with  sum q * d_i  for its own row and its own 32-weight block, exactly, in
// int32.  The lane recombines the digits, subtracts the format's zero point through the precomputed
// integer block sum of the activations, converts once to float and applies scale * 2^-e.
// Everything up to that conversion is exact integer arithmetic; the activations keep 21 bits below
// their block maximum.
//
// Lane = 4 * column + row: a wave works on bundles of four rows, the 16 columns are consecutive
// 32-weight blocks.  Per step every lane loads four 16-byte blocks of its row (the wave covers
// 4 rows x 2048 weights) and the next step's loads are issued before the current step is computed.
#include "gemv_common.h"
#include <algorithm>

namespace adamah {

typedef int i4_t __attribute__((ext_vector_type(4)));
typedef float f4u_t __attribute__((ext_vector_type(4), aligned(4)));
typedef uint32_t u4v_t __attribute__((ext_vector_type(4)));

// A step of the row loop covers 16 * U blocks of a 4-row bundle: U 16-byte blocks per lane.  U = 4 for rows that fill
// whole steps (K a multiple of 2048); U = 3 wastes fewer block slots on some rows that do not (K = 1152: 36 blocks
// in one step of 48 instead of one of 64).


// lane ^ 1 and lane ^ 2 within a quad (quad_perm [1,0,3,2] and [2,3,0,1]): a register move, no trip through LDS
__device__ __forceinline__ float quad_x1(float v) {
  int r = __builtin_amdgcn_update_dpp(0, __float_as_int(v), 0xB1, 0xF, 0xF, false);
  asm volatile("" : "+v"(r));   // kept an instruction of its own, see quad_b3
  return __int_as_float(r);
}
__device__ __forceinline__ float quad_x2(float v) {
  int r = __builtin_amdgcn_update_dpp(0, __float_as_int(v), 0x4E, 0xF, 0xF, false);
  asm volatile("" : "+v"(r));
  return __int_as_float(r);
}

// Lane 3 of every quad to the whole quad (quad_perm [3,3,3,3]).  The result is made opaque so that the move stays
// an instruction of its own: with the move folded into the consuming subtract / multiply the kernel returned wrong
// sums on the device although the generated code read as equivalent.
__device__ __forceinline__ uint32_t quad_b3(uint32_t v) {
  int r = __builtin_amdgcn_update_dpp(0, (int)v, 0xFF, 0xF, 0xF, false);
  asm volatile("" : "+v"(r));
  return (uint32_t)r;
}

// LDS layout: 128 bytes per activation block = 8 chunks of 16 bytes.  Chunk 2*d + h holds digit d of
// words 2h, 2h+1 as {even(2h), odd(2h), even(2h+1), odd(2h+1)} (even/odd = elements 0,2,4,6 / 1,3,5,7 of
// the 8-element word, one byte each, matching the byte order of the unpacked codes); chunk 6 holds
// {zero-point term, 2^-e, sum(x) as float, 0}.  Chunk c of block b sits at position c ^ (b & 7), which
// spreads the 16 blocks a wave reads at once over all banks.
__device__ __forceinline__ uint32_t chunk_off(uint32_t c, uint32_t blk) { return ((c ^ (blk & 7u)) << 4); }

template <int U>
struct PreMT {
  uint4 q[U];
  __half h[U];
  float2 p[U];
  float res;   // EPIX_ADD: the residual of this lane's result row, fetched with the weights of the bundle's last step
};

// PRO selects where the activation vector comes from: the map as it is, or the result of preceding
// row-wise ops that have been folded into this kernel (RMSNorm of another vector; or RMSNorm +
// residual followed by a second RMSNorm).  Every workgroup recomputes those small ops while it
// stages the activations; their results are also stored where the unfused ops would have put them.
template <int FMT, int EPI, bool RAGGED, int PRO, int MF_U>
__global__ void __launch_bounds__(1024)
k_gemv_mfma(const float* xp, const uint8_t* __restrict__ W, const __half* __restrict__ d16, const float* nwp, uint32_t K, uint32_t N,
            uint32_t cfg, uint32_t w0, uint32_t w1, uint32_t w2,
            const float* act, float* act_out, uint32_t c_out, const float2* __restrict__ qp, const uint32_t* __restrict__ lidx,
            const uint32_t* __restrict__ lval, uint32_t n_groups, GemvFuse fz) {
  // The first 14 dwords of the arguments are in registers when a wave starts; the rest is fetched from the argument
  // block, a trip to memory that nothing in front of a wave's first loads may wait for.  So everything those loads
  // need stands in front, with the offsets folded into the pointers by the launcher: xp = the activation vector (or
  // the source of the first folded norm, whose weights start at nwp), W / d16 (and, behind, qp) = the matrix's first
  // block, K, N, cfg = ks | waves per workgroup << 3 | epilogue << 8 | (share shift - 28) << 10 | (slices - 1) << 14 |
  // value_dim / 8 << 22 (the last two: PRO_COMBINE, whose partials start at nwp), and w0..w2 = the multiply-and-shift
  // form of the waves' row shares (store) or, w0, the rows per group (argmax).
  const uint32_t ks = cfg & 7u, e_mode = (cfg >> 8) & 3u;
  const float* c_partial = nwp;
  const uint32_t c_splits = ((cfg >> 14) & 0xFFu) + 1u, c_vd = (cfg >> 22) << 3;
  // Gated activation, split form (bit 14 of cfg where the prologue is not the merge): half of a workgroup's waves take
  // gate rows, the other half the matching up rows, plain bundles of four neighbouring rows each; the results meet in
  // LDS at the end of the workgroup.  (In the paired form a bundle is two gate rows and their two up rows, and every
  // wave reads from both halves of the matrix, which costs about a microsecond at 28672 x 4096.)
  const bool glu_split = EPI == EPI_STORE && PRO != PRO_COMBINE && ((cfg >> 14) & 1u) != 0u;
  using PreM = PreMT<MF_U>;
  constexpr uint32_t SB = 16u * MF_U;                 // blocks per step
  constexpr bool B16 = (FMT == FMT_Q4_B16);
  extern __shared__ uint4 smem_u4[];
  uint8_t* xs = (uint8_t*)smem_u4;                    // nblk * 128 bytes
  __shared__ float red_f[16];
  __shared__ uint32_t red_i[16];
  __shared__ float red_g[16];                         // per-wave partial sums of the prologue's last norm
  __shared__ float part[16 * 64];                     // ks > 1: per-wave partial sums of a shared bundle
  const uint32_t nblk = K >> 5;
  const uint32_t C = (nblk + SB - 1u) / SB;           // steps per row bundle

  const uint32_t tid = threadIdx.x, lane = tid & 63u, nwav = (cfg >> 3) & 31u, nthr = nwav << 6;
  const uint32_t wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const uint32_t l = lane & 3u, bcol = lane >> 2;      // row in bundle, block column 0..15

  // ---- this wave's rows: store = contiguous balanced share of the 4-row bundles (waves that share
  // a SIMD, w % 4, take neighbouring shares so that every SIMD gets the same load); argmax = the
  // workgroup takes whole argmax groups, its waves interleave the bundles of a group ------------
  // ks > 1 (store only, short matrices with long rows): ks neighbouring waves share one bundle and take
  // every ks-th step of K each; a workgroup holds nwav / ks bundles, one round.
  uint32_t grp = blockIdx.x, first, stride, seg_end;
  uint32_t glu_base = 0, glu_slot = 0, glu_rows = 0;   // split gated form: first row of the workgroup's region, LDS slot, rows
  const uint32_t ksh = ks >> 1;                        // ks is 1, 2 or 4: its logarithm
  const uint32_t kpart = wave & (ks - 1u);
  if (EPI == EPI_STORE && ks > 1u) {
    const uint32_t bundle = blockIdx.x * (nwav >> ksh) + (wave >> ksh);
    first = bundle * 4u;
    seg_end = kpart < C ? min(N, first + 4u) : 0u;      // nothing to do: no bundle, or no step of K left for this wave
    if (first >= N) seg_end = 0u;
    stride = 4u;
  } else if (glu_split) {
    // workgroup b: gate bundles [F(b), F(b + 1)), F(b) = floor(b * n_gb / workgroups) in the multiply-and-shift form
    // (w0..w2 are for the grid here); its waves: region r (0 gate, 1 up) and part p of the region's `half` parts,
    // waves that share a SIMD (w % 4) taking parts of both regions that differ in size as little as possible
    auto share = [&](uint32_t gq) -> uint32_t {
      return gq * w0 + (uint32_t)(((uint64_t)(gq * w1) * w2) >> (28u + ((cfg >> 10) & 15u)));
    };
    const uint32_t f0 = share(blockIdx.x), nb = share(blockIdx.x + 1u) - f0;
    const uint32_t half = nwav >> 1, hsh = (uint32_t)__builtin_ctz(half);
    uint32_t r, p;
    if (nwav == 4u) { r = wave >> 1; p = wave & 1u; }
    else {
      const uint32_t sd = wave & 3u, q = wave >> 2, per = nwav >> 3;   // per: q-levels per region (1 or 2)
      r = q / per;
      p = (q % per) * 4u + ((sd + 2u * r) & 3u);
    }
    const uint32_t rb = r * (N >> 1), re = rb + (N >> 1);
    first = rb + (f0 + ((p * nb) >> hsh)) * 4u;
    seg_end = min(re, rb + (f0 + (((p + 1u) * nb) >> hsh)) * 4u);
    stride = 4u;
    glu_base = rb + f0 * 4u;
    glu_slot = r * 512u;
    glu_rows = nb * 4u;
  } else if (EPI == EPI_STORE) {
    const uint32_t slot = (wave & 3u) * (nwav >> 2) + (wave >> 2);
    // balanced shares without a division: a 64-bit quotient here is a few hundred instructions
    // and two jumps to the far end of the kernel, in front of the wave's first loads and with a cold instruction cache
    const uint32_t gw = blockIdx.x * nwav + slot;
    // wave g takes bundles [f(g), f(g + 1)), f(g) = floor(g * n_q / wt) = g * w0 + floor(g * w1 / wt) with
    // w0 = n_q / wt, w1 = n_q % wt and the last quotient as a multiplication by w2 = ceil(2^s / wt) and a shift
    // (exact for g * w1 < 2^28)
    auto share = [&](uint32_t gq) -> uint32_t {
      return gq * w0 + (uint32_t)(((uint64_t)(gq * w1) * w2) >> (28u + ((cfg >> 10) & 15u)));
    };
    first = share(gw) * 4u;
    seg_end = min(N, share(gw + 1u) * 4u);
    stride = 4u;
  } else {
    first = grp * w0 + wave * 4u;
    seg_end = min(N, (grp + 1) * w0);
    stride = 4u * nwav;
  }

  // Row of lane-row l in the bundle that starts at row0.  With the gated-activation epilogue the
  // matrix is [gate rows; up rows] (N/2 each) and a bundle pairs two gate rows with their up rows.
  const bool glu = EPI == EPI_STORE && !glu_split && (e_mode == EPIX_GEGLU || e_mode == EPIX_SWIGLU);
  auto row_of = [&](uint32_t row0, uint32_t end) -> uint32_t {
    if (glu) return (row0 >> 1) + (l & 1u) + (l >> 1) * (N >> 1);
    return min(row0 + l, end - 1u);
  };
  // Loads use their own lane mapping, lane -> (bundle row lane / 16, block column lane % 16): sixteen
  // consecutive lanes read 256 contiguous bytes of one row, so a quad's 64 bytes are one request to the
  // L1 (with the compute mapping a quad is four rows, i.e. four requests per quad, 64 per instruction).
  // compute() moves every block and its scale to the lane that owns it with a cross-lane permute.
  const uint32_t ll = lane >> 4, lbcol = lane & 15u;
  auto load = [&](PreM& R, uint32_t row0, uint32_t chunk, uint32_t end) {
    const uint32_t row = glu ? (row0 >> 1) + (ll & 1u) + (ll >> 1) * (N >> 1) : min(row0 + ll, end - 1u);
    const uint64_t g0 = (uint64_t)row * nblk + chunk * SB + lbcol;
#pragma unroll
    for (uint32_t u = 0; u < MF_U; u++) {
      uint64_t gi = g0 + u * 16u;
      // blocks past the end of the row are clamped, not skipped: the number of loads per step has to be
      // fixed for the prefetch to stay ahead (see the step loop)
      if (RAGGED) gi = (uint64_t)row * nblk + min(chunk * SB + u * 16u + lbcol, nblk - 1u);
      // the codes are read once per launch and not again before the next token: non-temporal, so that they do not
      // push the step's small, re-read data (activations, KV rows, slice partials) out of the L2
      const u4v_t t = __builtin_nontemporal_load((const u4v_t*)(W + (gi << 4)));
      R.q[u] = make_uint4(t.x, t.y, t.z, t.w);
      if (B16) R.h[u] = d16[gi];
      else R.p[u] = qp[gi];
    }
    // The add epilogue needs one residual value per result row: asked for here, in the compute mapping (lane =
    // 4 * column + row, column 0 stores), so it has arrived long before the row sum is complete.  Every lane asks at
    // every step (without the epilogue: for a word of the activations, not used): a load under a branch would leave
    // the compiler unable to count the loads in flight, and it then waits for all of them wherever it waits for one.
    if (EPI == EPI_STORE) R.res = *(e_mode == EPIX_ADD ? act + ((uint64_t)fz.e_res + min(row0 + l, end - 1u)) : xp);
  };

  PreM A, B;   // A's first loads stay in flight while the activations are staged
  // (a wave without rows asks for the matrix's first rows: same number of loads on every path, see load())
  auto first_loads = [&]() {
    const bool has = first < seg_end;
    load(A, has ? first : 0u, has ? kpart : 0u, has ? seg_end : min(N, 4u));
  };
  // Loads come back in order: the activation loads (cache hits) go out ahead of the first weights, so
  // the conversion does not wait for the weights' trip to memory as well.

  // ---- activations -> fixed-point digits; one 8-element word per thread and pass, four threads per
  // block.  stage() turns one word into digits; the prologues below decide what the word is. ------
  const uint32_t nw = nblk * 4u;
  auto stage = [&](uint32_t i, bool live, const float* x) {
    float m = 0.f, poison = 0.f;          // poison turns NaN as soon as one element is Inf or NaN
#pragma unroll
    for (int k = 0; k < 8; k++) { m = fmaxf(m, fabsf(x[k])); poison = fmaf(x[k], 0.f, poison); }
    // the four threads of a block are a quad: lane ^ 1 and lane ^ 2 through the data-parallel crossbar
    m = fmaxf(m, quad_x1(m)); m = fmaxf(m, quad_x2(m));
    poison += quad_x1(poison); poison += quad_x2(poison);
    const uint32_t e = (__float_as_uint(m) >> 23) & 0xFFu;
    float s = 1.f, fs = 1.f;              // |x * s| < 2^21 when the block is finite and not tiny
    if (e >= 21u && e <= 254u) { s = __uint_as_float((274u - e) << 23); fs = __uint_as_float((e - 20u) << 23); }
    if (poison != poison) fs = poison;    // the block's result is NaN, as it would be in float arithmetic
    int d0[8], d1[8], d2[8], sx = 0;
#pragma unroll
    for (int k = 0; k < 8; k++) {
      int xi = (e >= 21u && e <= 254u) ? (int)rintf(x[k] * s) : 0;
      xi = min(max(xi, -(1 << 21)), (1 << 21) - 1);
      sx += xi;
      d0[k] = xi >> 14; d1[k] = (xi >> 7) & 127; d2[k] = xi & 127;
    }
    sx += __float_as_int(quad_x1(__int_as_float(sx))); sx += __float_as_int(quad_x2(__int_as_float(sx)));
    if (live) {
      const uint32_t blk = i >> 2, j = i & 3u;
      uint8_t* bp = xs + (size_t)blk * 128u;
      auto pack = [](const int* d, int o) {
        return (uint32_t)(d[o] & 255) | ((uint32_t)(d[o + 2] & 255) << 8) | ((uint32_t)(d[o + 4] & 255) << 16) |
               ((uint32_t)(d[o + 6] & 255) << 24);
      };
      const uint32_t h = j >> 1, wo = (j & 1u) * 8u;
      *(uint2*)(bp + chunk_off(0u + h, blk) + wo) = make_uint2(pack(d0, 0), pack(d0, 1));
      *(uint2*)(bp + chunk_off(2u + h, blk) + wo) = make_uint2(pack(d1, 0), pack(d1, 1));
      *(uint2*)(bp + chunk_off(4u + h, blk) + wo) = make_uint2(pack(d2, 0), pack(d2, 1));
      if (j == 0) {
        uint4 prm;
        prm.x = (uint32_t)(B16 ? 8 * sx : 0);              // zero-point term of the block format, integer
        prm.y = __float_as_uint(fs);
        prm.z = __float_as_uint((float)sx * fs);           // sum of the block's activations (affine format)
        prm.w = 0;
        *(uint4*)(bp + chunk_off(6u, blk)) = prm;
      }
    }
  };
  auto load8 = [&](const float* p, float* v) {
    const f4u_t v0 = ((const f4u_t*)p)[0], v1 = ((const f4u_t*)p)[1];
    v[0] = v0.x; v[1] = v0.y; v[2] = v0.z; v[3] = v0.w; v[4] = v1.x; v[5] = v1.y; v[6] = v1.z; v[7] = v1.w;
  };
  auto block_sum = [&](float v) {     // sum over the workgroup, same value in every thread
    v = wave_sum_to_lane63(v);
    __syncthreads();                  // red_f may still be read from the previous use
    if (lane == 63u) red_f[wave] = v;
    __syncthreads();
    float t = 0.f;
    for (uint32_t w = 0; w < nwav; w++) t += red_f[w];
    return t;
  };

  float nrm1 = 1.f, nrm_late = 1.f;   // nrm_late: the prologue's last norm, applied to the row sums
  uint32_t ticket = 0;
  if (PRO == PRO_NONE) {
    // four passes of loads are issued before the first word is converted; the first round stands outside the loop,
    // in straight-line code with the first weight loads behind it, so that the conversion waits for exactly the
    // activation loads
    auto x_round = [&](uint32_t i0, bool with_weights) {
      float x[4][8];
#pragma unroll
      for (uint32_t u = 0; u < 4; u++) load8(xp + (uint64_t)min(i0 + u * nthr + tid, nw - 1u) * 8u, x[u]);
      if (with_weights) {
        __builtin_amdgcn_sched_barrier(0);
        first_loads();
        __builtin_amdgcn_sched_barrier(0);
      }
#pragma unroll
      for (uint32_t u = 0; u < 4; u++)
        if (i0 + u * nthr + (tid & ~63u) < nw)   // wave-uniform: waves without words skip the conversion
          stage(i0 + u * nthr + tid, i0 + u * nthr + tid < nw, x[u]);
    };
    x_round(0u, true);
    for (uint32_t i0 = 4u * nthr; i0 < nw; i0 += 4u * nthr) x_round(i0, false);
  } else if (PRO == PRO_COMBINE) {
    // Folded merge of the attention partials (same arithmetic as the stand-alone merge kernel):
    // M = max m_s, w_s = e^(m_s - M), L = sum l_s w_s, x = sum_s o_s w_s / L, per head.
    const uint32_t stride = c_vd + 2u;
    // At most eight slices and two threads per word: straight-line form.  A thread merges four elements: every value
    // it needs and the slices' (max, sum) pairs are asked for in one round, ahead of the first weights (loads return
    // in order: behind the weights they would wait for the weights' trip to memory as well).  Slices past the last
    // are clamped, not skipped, so that the waits stay counted.  The (max, sum) pair of slice s comes from lane s of
    // the thread's group of eight lanes, which all work on the same head (value_dim a multiple of 32).  The merged
    // elements meet in LDS (in the digits' place, before there are digits), where each word's thread picks them up.
    // Same order of operations per element as the loops below.
    const bool few = EPI == EPI_STORE && c_splits <= 8u && 2u * nw <= nthr && c_vd % 32u == 0u;
    if (few) {
      const uint32_t e0 = min(tid, 2u * nw - 1u) * 4u, head = e0 / c_vd, j0 = e0 % c_vd, last = c_splits - 1u;
      const float* pp = c_partial + (uint64_t)head * c_splits * stride;
      const float* pm = pp + (uint64_t)min(lane & 7u, last) * stride;
      const float m_own = pm[0], l_own = pm[1];
      f4u_t o[8];
#pragma unroll
      for (uint32_t sp = 0; sp < 8u; sp++) o[sp] = *(const f4u_t*)(pp + (uint64_t)min(sp, last) * stride + 2 + j0);
      __builtin_amdgcn_sched_barrier(0);
      first_loads();
      __builtin_amdgcn_sched_barrier(0);
      float mv[8], lv[8], M = -9.99999968e+37f, L = 0.f;
#pragma unroll
      for (uint32_t sp = 0; sp < 8u; sp++) {
        mv[sp] = __shfl(m_own, (int)((lane & ~7u) + sp), 64);
        lv[sp] = __shfl(l_own, (int)((lane & ~7u) + sp), 64);
      }
#pragma unroll
      for (uint32_t sp = 0; sp < 8u; sp++) M = sp < c_splits ? fmaxf(M, mv[sp]) : M;
      f4u_t x4 = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
      for (uint32_t sp = 0; sp < 8u; sp++) {
        const float wgt = expf(mv[sp] - M);
        const bool on = sp < c_splits;
        L = on ? fmaf(lv[sp], wgt, L) : L;
        x4.x = on ? fmaf(o[sp].x, wgt, x4.x) : x4.x; x4.y = on ? fmaf(o[sp].y, wgt, x4.y) : x4.y;
        x4.z = on ? fmaf(o[sp].z, wgt, x4.z) : x4.z; x4.w = on ? fmaf(o[sp].w, wgt, x4.w) : x4.w;
      }
      const float invL = 1.0f / L;
      x4.x *= invL; x4.y *= invL; x4.z *= invL; x4.w *= invL;
      float* xf = (float*)xs;
      if (tid < 2u * nw) {
        *(f4u_t*)(xf + tid * 4u) = x4;
        if (blockIdx.x == 0) *(f4u_t*)(act_out + fz.p_dst + (uint64_t)tid * 4u) = x4;
      }
      __syncthreads();
      float x[8];
      load8(xf + min(tid, nw - 1u) * 8u, x);
      __syncthreads();
      if ((tid & ~63u) < nw) stage(tid, tid < nw, x);
    } else {
      first_loads();
      for (uint32_t i0 = 0; i0 < nw; i0 += nthr) {
        const uint32_t i = i0 + tid, ic = min(i, nw - 1u);
        const uint32_t head = (ic * 8u) / c_vd, j0 = (ic * 8u) % c_vd;
        const float* pp = c_partial + (uint64_t)head * c_splits * stride;
        float M = -9.99999968e+37f;
        for (uint32_t sp = 0; sp < c_splits; sp++) M = fmaxf(M, pp[(uint64_t)sp * stride]);
        float L = 0.f, x[8] = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
        for (uint32_t sp = 0; sp < c_splits; sp++) {
          const float wgt = expf(pp[(uint64_t)sp * stride] - M);
          L = fmaf(pp[(uint64_t)sp * stride + 1], wgt, L);
          float o[8];
          load8(pp + (uint64_t)sp * stride + 2 + j0, o);
#pragma unroll
          for (int k = 0; k < 8; k++) x[k] = fmaf(o[k], wgt, x[k]);
        }
        const float invL = 1.0f / L;
#pragma unroll
        for (int k = 0; k < 8; k++) x[k] *= invL;
        if (i0 + (tid & ~63u) >= nw) continue;   // wave-uniform: nothing of this pass belongs to the wave
        if (blockIdx.x == 0 && i < nw) {
          f4u_t* o = (f4u_t*)(act_out + fz.p_dst + (uint64_t)i * 8u);
          o[0] = (f4u_t){x[0], x[1], x[2], x[3]}; o[1] = (f4u_t){x[4], x[5], x[6], x[7]};
        }
        stage(i, i < nw, x);
      }
    }
    if (blockIdx.x == 0)
      for (uint32_t i = tid; i < fz.c_qn; i += nthr) act_out[(uint64_t)fz.c_qdst + i] = fz.c_qsrc[i];
  } else {
    // Folded row-wise ops.  Every thread keeps its (at most PRO_WPT) words in registers from one
    // round of loads, so the norms cost block reductions but no further trips to memory.
    //   PRO_RMSNORM:  x = src * rsqrt(mean(src^2) + eps) * w                       (stored at p_dst)
    //   PRO_NORM2:    t = src * rsqrt(mean(src^2) + eps) * w + res                 (stored at p_tdst)
    //                 x = t * rsqrt(mean(t^2) + eps2) * w2                          (stored at p_dst)
    float v[PRO_WPT][8], wv[PRO_WPT][8], rv[PRO_WPT][8], w2v[PRO_WPT][8];
    bool live[PRO_WPT];
    float ss = 0.f;
    bool mine[PRO_WPT];   // wave-uniform: the wave has words in this pass at all
#pragma unroll
    for (uint32_t u = 0; u < PRO_WPT; u++) {
      const uint32_t i = u * nthr + tid;
      live[u] = i < nw;
      mine[u] = u * nthr + (tid & ~63u) < nw;
#pragma unroll
      for (int k = 0; k < 8; k++) { v[u][k] = 0.f; wv[u][k] = 0.f; rv[u][k] = 0.f; w2v[u][k] = 0.f; }
      // (waves without words of their own load the row's last word: every path issues the same loads)
      const uint64_t e0 = (uint64_t)min(i, nw - 1u) * 8u;
      load8(xp + e0, v[u]);
      load8(nwp + e0, wv[u]);
    }
    if (PRO == PRO_NORM2) {
      // the second norm's operands are addressed from the part of the argument block that is fetched from memory:
      // behind a fence, so that the loads above do not wait for it
      __builtin_amdgcn_sched_barrier(0);
#pragma unroll
      for (uint32_t u = 0; u < PRO_WPT; u++) {
        const uint64_t e0 = (uint64_t)min(u * nthr + tid, nw - 1u) * 8u;
        load8(act + fz.p_res + e0, rv[u]);
        load8(fz.p_wt2 + fz.p_w2 + e0, w2v[u]);
      }
    }
    __builtin_amdgcn_sched_barrier(0);   // activation loads first: they are waited for first
    first_loads();
    __builtin_amdgcn_sched_barrier(0);
#pragma unroll
    for (uint32_t u = 0; u < PRO_WPT; u++)
      if (mine[u]) {
#pragma unroll
        for (int k = 0; k < 8; k++) if (live[u]) ss = fmaf(v[u][k], v[u][k], ss);
      }
    // The ticket taken below tells other workgroups that this one has read `res`: its loads must have
    // returned, not merely been issued.  Naming the registers as inputs of an (empty) asm makes the
    // compiler wait for exactly those loads here.
    if (PRO == PRO_NORM2) {
#pragma unroll
      for (uint32_t u = 0; u < PRO_WPT; u++)
#pragma unroll
        for (int k = 0; k < 8; k++) asm volatile("" ::"v"(rv[u][k]));
    }
    // The LAST norm of the prologue is not applied to the activations but to the row sums: y = W (u n) = n (W u)
    // with u = t w (elementwise) and n = rsqrt(mean(t^2) + eps) a scalar.  The workgroup-wide sum behind n then
    // runs beside the staging of u instead of before it; it is needed only when the first row sum is complete.
    float ss_last = ss;
    if (PRO == PRO_NORM2) {
      nrm1 = 1.0f / sqrtf(block_sum(ss) / (float)K + fz.p_eps);
      const float nrm = nrm1;
      // Every thread of this workgroup has consumed `res` (the reduction above ends in a barrier).
      // t usually goes back into `res` (residual updated in place), which other workgroups may not
      // have read yet, so it is stored by whichever workgroup draws the last ticket.  The ticket is
      // drawn here and looked at after staging, so nobody waits for the atomic's round trip.
      if (fz.t_mode == 0u && wave == 0 && lane == 0) ticket = atomicAdd(fz.counter, 1u);
      float ss2 = 0.f;
#pragma unroll
      for (uint32_t u = 0; u < PRO_WPT; u++)
        if (mine[u]) {
#pragma unroll
          for (int k = 0; k < 8; k++) {
            v[u][k] = v[u][k] * nrm * wv[u][k] + rv[u][k];
            if (live[u]) ss2 = fmaf(v[u][k], v[u][k], ss2);
          }
          if (fz.t_mode != 0u && blockIdx.x == 0 && live[u]) {   // t: in place at once, or parked for a later launch
            float* td = fz.t_mode == 1u ? act_out + fz.p_tdst : fz.t_park;
            f4u_t* o = (f4u_t*)(td + (uint64_t)(u * nthr + tid) * 8u);
            o[0] = (f4u_t){v[u][0], v[u][1], v[u][2], v[u][3]}; o[1] = (f4u_t){v[u][4], v[u][5], v[u][6], v[u][7]};
          }
#pragma unroll
          for (int k = 0; k < 8; k++) v[u][k] *= w2v[u][k];
        }
      ss_last = ss2;
    } else {
#pragma unroll
      for (uint32_t u = 0; u < PRO_WPT; u++)
        if (mine[u]) {
#pragma unroll
          for (int k = 0; k < 8; k++) v[u][k] *= wv[u][k];
        }
    }
#pragma unroll
    for (uint32_t u = 0; u < PRO_WPT; u++)
      if (mine[u]) stage(u * nthr + tid, live[u], v[u]);
    ss_last = wave_sum_to_lane63(ss_last);
    if (lane == 63u) red_g[wave] = ss_last;
    __syncthreads();          // the staged activations and the waves' partial sums are in LDS
    float tot = 0.f;
    for (uint32_t w = 0; w < nwav; w++) tot += red_g[w];
    nrm_late = 1.0f / sqrtf(tot / (float)K + (PRO == PRO_NORM2 ? fz.p_eps2 : fz.p_eps));
    if (blockIdx.x == 0) {    // the normalised vector itself, where the norm op would have stored it
#pragma unroll
      for (uint32_t u = 0; u < PRO_WPT; u++)
        if (mine[u] && live[u]) {
          f4u_t* o = (f4u_t*)(act_out + fz.p_dst + (uint64_t)(u * nthr + tid) * 8u);
          o[0] = (f4u_t){v[u][0] * nrm_late, v[u][1] * nrm_late, v[u][2] * nrm_late, v[u][3] * nrm_late};
          o[1] = (f4u_t){v[u][4] * nrm_late, v[u][5] * nrm_late, v[u][6] * nrm_late, v[u][7] * nrm_late};
        }
    }
  }
  if (PRO == PRO_NONE || PRO == PRO_COMBINE) __syncthreads();
  uint32_t nib = 0x0F0F0F0Fu;
  asm volatile("" : "+s"(nib));             // opaque, so it stays in a register instead of a literal per use
  // Lanes 0..2 of a block read digit 0..2 (operand rows 0..2); the fourth operand row is not needed, so lane 3 reads
  // the block's parameters instead and hands them to its three neighbours through the data-parallel crossbar:
  // two LDS reads per lane and block where digits plus parameters would be three.
  const uint32_t x_off0 = l < 3u ? chunk_off(2u * l, bcol) : chunk_off(6u, bcol);
  const uint32_t x_off1 = l < 3u ? chunk_off(2u * l + 1u, bcol) : chunk_off(6u, bcol);
  float acc = 0.f;
  float best_v = NEG_FLT_MAX;
  uint32_t best_i = INVALID_IDX;

  const int perm_addr = (int)((16u * l + bcol) << 2);   // the lane that loaded this lane's (row, block column)
  float res_keep = 0.f;                                  // ks > 1: residual of the bundle, from this wave's last step
  auto compute = [&](const PreM& Rl, uint32_t row0, uint32_t chunk, uint32_t end) {
    PreM R;
#pragma unroll
    for (uint32_t u = 0; u < MF_U; u++) {
      R.q[u] = make_uint4((uint32_t)__builtin_amdgcn_ds_bpermute(perm_addr, (int)Rl.q[u].x),
                          (uint32_t)__builtin_amdgcn_ds_bpermute(perm_addr, (int)Rl.q[u].y),
                          (uint32_t)__builtin_amdgcn_ds_bpermute(perm_addr, (int)Rl.q[u].z),
                          (uint32_t)__builtin_amdgcn_ds_bpermute(perm_addr, (int)Rl.q[u].w));
      if (B16) {
        const uint32_t hb = (uint32_t)__builtin_amdgcn_ds_bpermute(perm_addr, (int)__half_as_ushort(Rl.h[u]));
        R.h[u] = __ushort_as_half((unsigned short)hb);
      } else {
        R.p[u].x = __int_as_float(__builtin_amdgcn_ds_bpermute(perm_addr, __float_as_int(Rl.p[u].x)));
        R.p[u].y = __int_as_float(__builtin_amdgcn_ds_bpermute(perm_addr, __float_as_int(Rl.p[u].y)));
      }
    }
    const uint8_t* base = xs + (size_t)(chunk * SB + bcol) * 128u;
    uint4 xa[MF_U], xb[MF_U];
    bool valid[MF_U];
    i4_t d[MF_U];
#pragma unroll
    for (uint32_t u = 0; u < MF_U; u++) {
      valid[u] = true;
      const uint8_t* bp = base + u * 2048u;
      if (RAGGED) {
        const uint32_t blk_raw = chunk * SB + u * 16u + bcol;
        valid[u] = blk_raw < nblk;
        bp = xs + (size_t)min(blk_raw, nblk - 1u) * 128u;
      }
      xa[u] = *(const uint4*)(bp + x_off0); xb[u] = *(const uint4*)(bp + x_off1);
      d[u] = (i4_t){0, 0, 0, 0};
    }
    // eight dependent matrix instructions per block; the U blocks of a step are interleaved so that
    // consecutive instructions are independent
#define MF_STEP(XV, WV, SH)                                                                                   \
  _Pragma("unroll") for (uint32_t u = 0; u < MF_U; u++)                                                       \
      d[u] = __builtin_amdgcn_mfma_i32_4x4x4i8((int)XV, (int)(((WV) >> SH) & nib), d[u], 0, 0, 0)
    MF_STEP(xa[u].x, R.q[u].x, 0); MF_STEP(xa[u].y, R.q[u].x, 4);
    MF_STEP(xa[u].z, R.q[u].y, 0); MF_STEP(xa[u].w, R.q[u].y, 4);
    MF_STEP(xb[u].x, R.q[u].z, 0); MF_STEP(xb[u].y, R.q[u].z, 4);
    MF_STEP(xb[u].z, R.q[u].w, 0); MF_STEP(xb[u].w, R.q[u].w, 4);
#undef MF_STEP
#pragma unroll
    for (uint32_t u = 0; u < MF_U; u++) {
      // |d0| <= 15*128*32, so the recombination stays below 2^31
      const int sq = d[u][0] * 16384 + d[u][1] * 128 + d[u][2];
      // a block past the end of the row (ragged K) was clamped to a valid address: drop what it read
      // lane 3's first read is {zero-point term, 2^-e, block sum}: quad_perm [3,3,3,3]
      const uint32_t prm_x = quad_b3(xa[u].x), prm_y = quad_b3(xa[u].y);

      const float fsb = valid[u] ? __uint_as_float(prm_y) : 0.f;
      if (B16) {
        const float sc = valid[u] ? __half2float(R.h[u]) : 0.f;
        acc = fmaf(sc, (float)(sq - (int)prm_x) * fsb, acc);
      } else {
        const uint32_t prm_z = quad_b3(xa[u].z);
        const float sxb = valid[u] ? __uint_as_float(prm_z) : 0.f;
        const float sc = valid[u] ? R.p[u].x : 0.f, zp = valid[u] ? R.p[u].y : 0.f;
        acc = fmaf(sc, (float)sq * fsb, fmaf(zp, sxb, acc));
      }
    }
    if (ks > 1u) {
      if (chunk + ks >= C) { part[wave * 64u + lane] = acc; res_keep = Rl.res; }   // this wave's share of the bundle is done
    } else if (chunk == C - 1u) {   // row bundle complete: sum the 16 lanes that share a row
      float y = acc;
      y += __shfl_xor(y, 4, 64); y += __shfl_xor(y, 8, 64);
      y += __shfl_xor(y, 16, 64); y += __shfl_xor(y, 32, 64);
      if (PRO == PRO_RMSNORM || PRO == PRO_NORM2) y *= nrm_late;
      acc = 0.f;
      if (glu) {
        // lanes 0, 1 hold gate rows, lanes 2, 3 the matching up rows
        const float yu = __shfl_down(y, 2, 64);
        if (lane < 4u) {
          const uint32_t row = row_of(row0, end);
          act_out[(uint64_t)c_out + row] = y;
          if (lane < 2u) {
            const float t = e_mode == EPIX_GEGLU ? gelu_tanh(y) * yu : (y / (1.0f + expf(-y))) * yu;
            act_out[(uint64_t)fz.e_dst + row] = t;
          }
        }
      } else {
        const uint32_t row = row0 + l;
        if (row < end && bcol == 0u) {
          if (EPI == EPI_STORE) {
            act_out[(uint64_t)c_out + row] = y;
            if (glu_split) part[glu_slot + (row - glu_base)] = y;
            if (e_mode == EPIX_ADD) act_out[(uint64_t)fz.e_dst + row] = Rl.res + y;
          } else if (better(y, row, best_v, best_i)) { best_v = y; best_i = row; }
        }
      }
    }
  };

  // PRO_NORM2, last ticket: every other workgroup has read the residual, so t may now be stored over
  // it.  Looked at only here, after the workgroup's own rows, so that nobody waits for the atomic; the
  // whole workgroup then recomputes t for the row.
  auto finish_norm2 = [&]() {
    if (PRO != PRO_NORM2 || fz.t_mode != 0u) return;
    if (wave == 0 && lane == 0) red_i[0] = ticket;
    __syncthreads();
    if (red_i[0] != gridDim.x - 1u) return;
    if (tid == 0) atomicExch(fz.counter, 0u);      // ready for the next launch on the stream
    const f4u_t* ps = (const f4u_t*)(act + fz.p_src);
    const f4u_t* pw = (const f4u_t*)(fz.p_wt + fz.p_src2);
    const f4u_t* pr = (const f4u_t*)(act + fz.p_res);
    f4u_t* pd = (f4u_t*)(act_out + fz.p_tdst);
    for (uint32_t i = tid; i < (K >> 2); i += nthr) {
      const f4u_t sv = ps[i], wv4 = pw[i], rv4 = pr[i];
      pd[i] = (f4u_t){sv.x * nrm1 * wv4.x + rv4.x, sv.y * nrm1 * wv4.y + rv4.y, sv.z * nrm1 * wv4.z + rv4.z,
                      sv.w * nrm1 * wv4.w + rv4.w};
    }
  };

  while (true) {
    if (first < seg_end) {
      // steps t = 0..T-1 in (row bundle, chunk) order; register set A holds step 0 on entry.  The
      // prefetch of the following step is issued unconditionally (past the end it re-reads the last
      // rows, clamped in load()), so the number of loads in flight at every wait is known statically.
      const uint32_t Cw = (C - kpart + ks - 1u) >> ksh;     // steps of K this wave takes per bundle
      // (stride is 4 or 4 * waves per workgroup: a power of two)
      const uint32_t T = ((seg_end - first + stride - 1u) >> (EPI == EPI_STORE ? 2u : (uint32_t)__builtin_ctz(stride))) * Cw;
      uint32_t row_a = first, ch_a = kpart, row_b, ch_b, row_n = first, ch_n = kpart;
      if ((ch_n += ks) >= C) { ch_n = kpart; row_n += stride; }
      if (T == 1) compute(A, first, kpart, seg_end);   // nothing to prefetch
      else for (uint32_t t = 0; t < T; t += 2) {
        row_b = row_n; ch_b = ch_n;
        load(B, row_b, ch_b, seg_end);
        __builtin_amdgcn_sched_barrier(0);   // keep the prefetch ahead of the arithmetic
        if ((ch_n += ks) >= C) { ch_n = kpart; row_n += stride; }
        compute(A, row_a, ch_a, seg_end);
        if (t + 1 >= T) break;
        row_a = row_n; ch_a = ch_n;
        load(A, row_a, ch_a, seg_end);
        __builtin_amdgcn_sched_barrier(0);
        if ((ch_n += ks) >= C) { ch_n = kpart; row_n += stride; }
        compute(B, row_b, ch_b, seg_end);
      }
    }
    if (EPI == EPI_STORE && ks > 1u) {
      // the ks waves of a bundle meet: the first of them adds the shares in wave order and stores
      if (!(first < seg_end)) part[wave * 64u + lane] = 0.f;
      __syncthreads();
      if (kpart == 0u && first < N) {
        float y = part[wave * 64u + lane];
        for (uint32_t pk = 1; pk < ks; pk++) y += part[(wave + pk) * 64u + lane];
        y += __shfl_xor(y, 4, 64); y += __shfl_xor(y, 8, 64);
        y += __shfl_xor(y, 16, 64); y += __shfl_xor(y, 32, 64);
        if (PRO == PRO_RMSNORM || PRO == PRO_NORM2) y *= nrm_late;
        const uint32_t row = first + l;
        if (row < N && bcol == 0u) {
          act_out[(uint64_t)c_out + row] = y;
          if (e_mode == EPIX_ADD) act_out[(uint64_t)fz.e_dst + row] = res_keep + y;
        }
      }
      break;
    }
    if (EPI == EPI_STORE && glu_split) {
      // gate and up results of the workgroup's rows meet: act(gate) * up, one row per thread
      __syncthreads();
      const uint32_t g0 = glu_base - (glu_slot ? (N >> 1) : 0u);          // the workgroup's first gate row
      const uint32_t f1 = min(N >> 1, g0 + 512u);
      for (uint32_t i = tid; g0 + i < f1 && i < glu_rows; i += nthr) {
        const float y = part[i], yu = part[512u + i];
        const float t = e_mode == EPIX_GEGLU ? gelu_tanh(y) * yu : (y / (1.0f + expf(-y))) * yu;
        act_out[(uint64_t)fz.e_dst + g0 + i] = t;
      }
      break;
    }
    if (EPI == EPI_STORE) break;
    // argmax: next group's first loads go out before this group's partial is merged
    const uint32_t done = grp;
    grp += gridDim.x;
    const bool more = grp < n_groups;
    if (more) {
      first = grp * w0 + wave * 4u;
      seg_end = min(N, (grp + 1) * w0);
      if (first < seg_end) load(A, first, 0, seg_end);
    }
    // lanes 0..3 hold the best of their own rows
#pragma unroll
    for (int o = 1; o <= 2; o <<= 1) {
      const float ov = __shfl_xor(best_v, o, 64);
      const uint32_t oi = __shfl_xor(best_i, o, 64);
      if (better(ov, oi, best_v, best_i)) { best_v = ov; best_i = oi; }
    }
    if (lane == 0u) { red_f[wave] = best_v; red_i[wave] = best_i; }
    __syncthreads();
    if (tid == 0) {
      float bv = red_f[0]; uint32_t bi = red_i[0];
      for (uint32_t w = 1; w < nwav; w++)
        if (better(red_f[w], red_i[w], bv, bi)) { bv = red_f[w]; bi = red_i[w]; }
      act_out[lidx[done]] = (float)(bi == INVALID_IDX ? 0u : bi);
      act_out[lval[done]] = bv;
    }
    __syncthreads();
    best_v = NEG_FLT_MAX; best_i = INVALID_IDX;
    if (!more) break;
  }
  finish_norm2();
  // a row an earlier launch parked: to its place (nothing in this launch touches it)
  if (blockIdx.x == 0)
    for (uint32_t i = tid; i < fz.d_n; i += nthr) const_cast<float*>(act)[(uint64_t)fz.d_dst + i] = fz.d_src[i];
}

// ---- host side -----------------------------------------------------------------------------------
static size_t mfma_smem(uint32_t K) { return (size_t)(K >> 5) * 128; }

bool mfma_path_ok(const Map* mw, uint32_t K) {
  return mw->dtype == DTYPE_Q4 && mw->group_size == 32 && K >= 32 && (K & 31u) == 0 && mfma_smem(K) <= 64000;
}

// Blocks per lane and step for rows of K elements (the block16 format; the affine format always takes 4): 3 where
// that takes no more steps than 4 and leaves fewer block slots of the last step empty (K = 1152: one step of 48 slots
// for 36 blocks instead of one of 64; 13824 x 1152 6.4 -> 5.5 us, 6912 x 1152 4.6 -> 4.4 us).  More but shorter steps
// lose: K = 6912 in five steps of 48 instead of four of 64, 5.1 -> 5.7 us.
static uint32_t mfma_step_u(uint32_t K) {
  const uint32_t nblk = K >> 5;
  const uint32_t c4 = cdiv(nblk, 64u), c3 = cdiv(nblk, 48u);
  uint32_t best = (c3 <= c4 && c3 * 48u < c4 * 64u) ? 3u : 4u;
  const int forced = knob("ADAMAH_MFMA_U", 0);
  if (forced == 3 || forced == 4) best = (uint32_t)forced;
  return best;
}

template <int EPI, int PRO>
static void launch_mfma_p(int fmt, uint32_t grid, uint32_t threads, const Map* ma, const Map* mw, uint32_t a, uint32_t b,
                          uint32_t c, const uint32_t* lidx, const uint32_t* lval, uint32_t K, uint32_t N, uint32_t rpg,
                          uint32_t n_groups, uint32_t ks, const GemvFuse& fz, float* out) {
  float* act = (float*)ma->buf;
  float* act_out = out ? out : act;
  const size_t smem = mfma_smem(K);
  const uint32_t U = fmt == FMT_Q4_B16 ? mfma_step_u(K) : 4u;
  const bool ragged = (K & 2047u) != 0;              // of steps of 64 blocks
  const bool norm = PRO == PRO_RMSNORM || PRO == PRO_NORM2;
  const uint32_t x_src = norm ? fz.p_src : a;
  const float* n_wt = norm ? fz.p_wt : act;
  // (the kernel's argument list says what goes where and why)
  uint32_t w0 = rpg, w1 = 0, w2 = 0, sh = 0;
  if (EPI == EPI_STORE && ks == 1u) {   // the shares of the bundles
    while (grid * (threads >> 6) > 16384u) grid >>= 1;   // keeps g * w1 below 2^28 (no launch shape comes near)
    const uint32_t n_q = cdiv(N, 4u), wt = grid * (threads >> 6);
    uint32_t lg = 0;
    while ((1u << lg) < wt) lg++;
    sh = lg;
    w0 = n_q / wt; w1 = n_q % wt; w2 = (uint32_t)((((uint64_t)1 << (28u + lg)) + wt - 1u) / wt);
  }
  // gated activation: the split form (see the kernel) where a workgroup's rows fit its LDS slots and the average
  // wave has two steps or more (Llama shape, 28672 x 4096, 3.5 steps per wave: 594 -> 612 tok/s; Gemma shape,
  // 13824 x 1152, under one step per wave: the closing barrier costs more than the rows' order gains, 1154 -> 1150)
  const bool gated = EPI == EPI_STORE && (fz.e_mode == EPIX_GEGLU || fz.e_mode == EPIX_SWIGLU);
  const int split_mode = tuning("ADAMAH_GLU_SPLIT", 1);
  const uint64_t wave_steps = (uint64_t)cdiv(N, 4u) * cdiv(K, 512u * U);
  bool glu_split = gated && ks == 1u && PRO != PRO_COMBINE && (N & 7u) == 0 &&
                   (split_mode == 2 || (split_mode == 1 && wave_steps >= 2ull * grid * (threads >> 6)));
  if (glu_split) {
    const uint32_t n_gb = N >> 3;                       // bundles of four gate rows
    if (grid > 16384u || 4u * (n_gb / grid + 1u) > 512u) glu_split = false;
    else {
      uint32_t lg = 0;
      while ((1u << lg) < grid) lg++;
      sh = lg;
      w0 = n_gb / grid; w1 = n_gb % grid; w2 = (uint32_t)((((uint64_t)1 << (28u + lg)) + grid - 1u) / grid);
    }
  }
  uint32_t cfg = ks | ((threads >> 6) << 3) | ((EPI == EPI_STORE ? fz.e_mode : 0u) << 8) | (sh << 10) | (glu_split ? 1u << 14 : 0u);
  if (PRO == PRO_COMBINE) cfg |= ((fz.c_splits - 1u) & 0xFFu) << 14 | (fz.c_vd >> 3) << 22;   // (the fold checks the ranges)
  const float* nwp = PRO == PRO_COMBINE ? fz.c_partial : n_wt + fz.p_src2;
  const uint64_t blk0 = (uint64_t)b >> 5;
  const uint8_t* Wp = (const uint8_t*)mw->buf + (blk0 << 4);
  const __half* d16p = mw->d16 ? mw->d16 + blk0 : nullptr;
  const float2* qpp = mw->qp ? mw->qp + blk0 : nullptr;
#define MK(F, R, UU)                                                                                              \
  k_gemv_mfma<F, EPI, R, PRO, UU><<<grid, threads, smem, g.stream>>>(act + x_src, Wp, d16p, nwp, K, N, cfg, w0, w1, w2,    \
                                                                     act, act_out, c, qpp, lidx, lval, n_groups, fz)
  // (the shorter steps exist in the clamping form only: they are chosen for rows that do not fill steps of 64)
  if (fmt == FMT_Q4_B16) {
    if (U == 3u) MK(FMT_Q4_B16, true, 3);
    else if (ragged) MK(FMT_Q4_B16, true, 4);
    else MK(FMT_Q4_B16, false, 4);
  } else { if (ragged) MK(FMT_Q4_AFF, true, 4); else MK(FMT_Q4_AFF, false, 4); }
#undef MK
}

template <int EPI>
static int launch_mfma(int fmt, uint32_t grid, uint32_t threads, const Map* ma, const Map* mw, uint32_t a, uint32_t b,
                       uint32_t c, const uint32_t* lidx, const uint32_t* lval, uint32_t K, uint32_t N, uint32_t rpg,
                       uint32_t n_groups, uint32_t ks, const GemvFuse* fzp, float* out = nullptr) {
  GemvFuse fz = {};
  if (fzp) fz = *fzp;
#define MP(P) launch_mfma_p<EPI, P>(fmt, grid, threads, ma, mw, a, b, c, lidx, lval, K, N, rpg, n_groups, ks, fz, out)
  switch (fz.pro) {
    case PRO_RMSNORM: MP(PRO_RMSNORM); break;
    case PRO_NORM2: MP(PRO_NORM2); break;
    case PRO_COMBINE: MP(PRO_COMBINE); break;
    default: MP(PRO_NONE); break;
  }
#undef MP
  count_launch();
  return check_launch();
}

// Launch shape for `units` wave-sized pieces of work: workgroups of 4, 8 or 16 waves (the activations
// are converted once per workgroup), as many as give every SIMD four waves.
static void mfma_shape(uint32_t K, uint32_t units, uint32_t* grid, uint32_t* threads) {
  // largest workgroup (16, 8 or 4 waves) that still leaves a workgroup for every CU
  uint32_t waves = 16;
  while (waves > 4 && cdiv(units, waves) < (uint32_t)g.n_cu) waves >>= 1;
  waves = (uint32_t)knob("ADAMAH_MFMA_WAVES", (int)waves);
  waves = waves >= 16 ? 16 : waves >= 8 ? 8 : 4;
  uint32_t per_simd = (uint32_t)std::max(1, knob("ADAMAH_MFMA_PERSIMD", 2));
  // rows of at most 4096 elements (16 KB of staged activations): two workgroups of 8 waves per CU instead of one of 16,
  // so that one's staging and barriers run beside the other's arithmetic (28672x4096 alone 15.8 -> 14.7 us, LM head
  // 262144x1152 + argmax 49 -> 41 us; inside the Llama-shape step, behind a norm prologue, no difference)
  if (waves == 16u && mfma_smem(K) <= (size_t)knob("ADAMAH_MFMA_SMALLWG", 16384)) { waves = 8u; per_simd = 4u; }
  const size_t lds_fit = std::max<size_t>(1, (160 * 1024) / (mfma_smem(K) + 256));
  const uint32_t wg_per_cu = (uint32_t)std::max<size_t>(1, std::min<size_t>(lds_fit, (size_t)per_simd * 4 / waves));
  *threads = waves * 64;
  *grid = std::max(1u, std::min<uint32_t>(cdiv(units, waves), (uint32_t)g.n_cu * wg_per_cu));
}

// Store launches of short matrices leave most SIMDs without work when a bundle of four rows belongs to one wave:
// there, 2 or 4 waves share a bundle and split K (one step of 2048 at a time), as far as that keeps the launch
// within the 4096 waves the device holds at once.  A wave then has one or two steps, all of whose loads are in
// flight from the start: such launches are bound by one trip to memory, not by arithmetic.
static uint32_t mfma_ksplit(uint32_t K, uint32_t N, bool paired_rows) {
  const uint32_t C = cdiv(K, 512u * mfma_step_u(K)), n_q = cdiv(N, 4u);
  const uint32_t want = (uint32_t)std::max(1, knob("ADAMAH_MFMA_KSPLIT_WAVES", 4096));
  uint32_t ks = 1;
  while (ks < 4u && ks * 2u <= C && n_q * ks * 2u <= want) ks *= 2u;
  const int forced = knob("ADAMAH_MFMA_KS", 0);
  if (forced == 1 || forced == 2 || forced == 4) ks = std::min<uint32_t>((uint32_t)forced, std::max(1u, C));
  if (ks == 3u) ks = 2u;
  return paired_rows ? 1u : ks;
}

static void mfma_store_shape(uint32_t K, uint32_t N, uint32_t ks, uint32_t* grid, uint32_t* threads) {
  const uint32_t n_q = cdiv(N, 4u);
  mfma_shape(K, n_q * ks, grid, threads);
  if (ks > 1u) {
    // one bundle per ks waves, one round.  Every workgroup stages the activations, so the workgroup size is the
    // one with the fewest (rounds over the CUs) x (waves per workgroup); ties go to the larger workgroup.
    uint32_t best_w = 4, best_cost = ~0u;
    for (uint32_t w = 4; w <= 16; w *= 2) {
      const uint32_t cost = cdiv(cdiv(n_q * ks, w), (uint32_t)g.n_cu) * w;
      if (cost <= best_cost) { best_cost = cost; best_w = w; }
    }
    const int fw = knob("ADAMAH_MFMA_WAVES", 0);
    if (fw > 0) best_w = fw >= 16 ? 16 : fw >= 8 ? 8 : 4;
    *threads = best_w * 64u;
    *grid = cdiv(n_q, best_w / ks);
  }
}

uint32_t mfma_store_threads(uint32_t K, uint32_t N) {
  uint32_t grid, t1, tk;
  mfma_store_shape(K, N, 1u, &grid, &t1);
  mfma_store_shape(K, N, mfma_ksplit(K, N, false), &grid, &tk);
  return std::min(t1, tk);
}

int launch_mfma_store(int fmt, const Map* ma, const Map* mw, uint32_t a, uint32_t b, uint32_t c, uint32_t K,
                      uint32_t N, const GemvFuse* fz, float* out) {
  uint32_t grid, threads;
  const bool paired = fz && (fz->e_mode == EPIX_GEGLU || fz->e_mode == EPIX_SWIGLU);
  const uint32_t ks = mfma_ksplit(K, N, paired);
  mfma_store_shape(K, N, ks, &grid, &threads);
  return launch_mfma<EPI_STORE>(fmt, grid, threads, ma, mw, a, b, c, nullptr, nullptr, K, N, 0, 0, ks, fz, out);
}

int launch_mfma_argmax(int fmt, const Map* ma, const Map* mw, uint32_t a, uint32_t b, const uint32_t* lidx,
                       const uint32_t* lval, uint32_t K, uint32_t N, uint32_t rows_per_group, const GemvFuse* fz) {
  const uint32_t n_groups = cdiv(N, rows_per_group);
  uint32_t grid, threads;
  mfma_shape(K, n_groups * 16u, &grid, &threads);   // one workgroup per group at a time
  grid = std::min(grid, n_groups);
  return launch_mfma<EPI_ARGMAX>(fmt, grid, threads, ma, mw, a, b, 0, lidx, lval, K, N, rows_per_group, n_groups, 1u, fz);
}

}  // namespace adamah

