// Sparse-mask prediction and INT8 Q/K quantisation for gfx950.
//
// Kernels (one 16-byte load per lane, 64-lane wavefront reductions; the K mean and the pooling / quantisation kernels run
// at the rates the machine gives a bare read and a bare 2-bytes-in / 1-byte-out copy, the selection is bound by the
// exact arithmetic it carries):
//   km_partial / km_final      K column mean                          (spas_sage_attn/core.py:119-120)
//   pool_sim_quant             pool + self-similarity + INT8 quant    (spas_sage_attn/utils.py:161-214, 89-159)
//   block_select_wave / block_select   compressed QK^T softmax, top-k / CDF selection, block map, delta LUT: pooled
//                              scores on the binary64 matrix unit and one wavefront per row with the row in registers
//                              (nk <= 2048), one workgroup per row beyond
//                                                                     (spas_sage_attn/utils.py:386-420, 54-87, 282-316)
//   map_to_lut                 user block mask -> LUT                 (spas_sage_attn/utils.py:54-87)
//
// Arithmetic contract: reductions whose addends are exactly representable run in binary64 (exact, hence
// order independent); every tensor the reference materialises in the input dtype is rounded exactly once
// (round-to-nearest-even, straight from binary64); fp32 quantisation steps use IEEE divide / sqrt; the
// compressed softmax uses a fixed binary64 operation sequence and a fixed summation tree.  This file must be
// compiled with -ffp-contract=off.
#include "common.h"
#include "launch.h"

#include <atomic>
#include <type_traits>

namespace spg {

// =============================================================================================
// K column mean
// =============================================================================================
template <int D, int DT>
__global__ __launch_bounds__(256) void km_partial_kernel(const uint16_t *__restrict__ k, const Strides ks, int H,
                                                         double *__restrict__ part, int N, int rows_per_chunk) {
  constexpr int TPR = D / 8;      // lanes per row (16 B each)
  constexpr int RPP = 256 / TPR;  // rows per pass of the workgroup
  const int bh = blockIdx.y, chunk = blockIdx.x, nchunk = gridDim.x;
  const int c = threadIdx.x % TPR, r = threadIdx.x / TPR;
  const int row0 = chunk * rows_per_chunk;
  const int row1 = min(N, row0 + rows_per_chunk);
  const uint16_t *base = k + (size_t)(bh / H) * ks.sb + (size_t)(bh % H) * ks.sh + c * 8;
  double acc[8];
#pragma unroll
  for (int e = 0; e < 8; e++) acc[e] = 0.0;
#pragma unroll 4
  for (int row = row0 + r; row < row1; row += RPP) {
    const uint4 v = load_stream_u4(base + (size_t)row * ks.sn);
    const uint32_t w[4] = {v.x, v.y, v.z, v.w};
#pragma unroll
    for (int e = 0; e < 4; e++) {
      acc[2 * e] += (double)elem_to_f32<DT>((uint16_t)(w[e] & 0xffffu));
      acc[2 * e + 1] += (double)elem_to_f32<DT>((uint16_t)(w[e] >> 16));
    }
  }
  __shared__ double sm[RPP][D];
#pragma unroll
  for (int e = 0; e < 8; e++) sm[r][c * 8 + e] = acc[e];
  __syncthreads();
  if (threadIdx.x < D) {
    double s = 0.0;
    for (int i = 0; i < RPP; i++) s += sm[i][threadIdx.x];
    part[((size_t)bh * nchunk + chunk) * D + threadIdx.x] = s;
  }
}

// One workgroup per (batch, head), blockDim = (D, 8): eight threads share a column's partial sums (exact, so the order of
// the additions is free), thread (d, 0) adds the eight sub-sums and rounds.
template <int DT>
__global__ void km_final_kernel(const double *__restrict__ part, uint16_t *__restrict__ km, int nchunk, int D, int N) {
  __shared__ double s_sub[8][128];
  const int bh = blockIdx.x, d = threadIdx.x, y = threadIdx.y;
  double s = 0.0;
#pragma unroll 4
  for (int i = y; i < nchunk; i += 8) s += part[((size_t)bh * nchunk + i) * D + d];
  s_sub[y][d] = s;
  __syncthreads();
  if (y == 0) {
    double t = 0.0;
#pragma unroll
    for (int u = 0; u < 8; u++) t += s_sub[u][d];
    km[(size_t)bh * D + d] = f64_to_elem<DT>(t / (double)N);
  }
}

// =============================================================================================
// pool + sim + INT8 quantisation.  One workgroup per (block, b*h).
// =============================================================================================
// IEEE binary32 quotient a/b with a reciprocal shared by many numerators: r = RN(1/b) (one correctly rounded
// division), then q = RN(a*r), one exact residual and one correction (Markstein).  div_selftest_kernel below
// compares it with the hardware's correctly rounded division for every finite binary16/bfloat16 numerator with
// |a| >= 2^-100 against pseudo-random divisors: the only difference is the sign of a zero quotient, which no user of
// the result can see.
// Valid while b stays in [2^-60, 2^60] (no scaling of the operands is done); quotients below 2^-100 in magnitude
// may be off in the last place, far below anything the callers resolve.
__device__ __forceinline__ float exact_rcp(float b) { return 1.0f / b; }
__device__ __forceinline__ float div_by(float a, float b, float r) {
  const float q = a * r;
  const float e = __builtin_fmaf(-b, q, a);
  return __builtin_fmaf(e, r, q);
}
__device__ __forceinline__ bool rcp_safe(float b) { return b >= 0x1p-60f && b <= 0x1p60f; }

// Self-test of div_by: divisor number i is a hash of (seed, i) with exponent in [-40, 40); every finite 16-bit
// numerator of both element types with |a| >= 2^-100 and 2^-100 <= |a/b| <= 2^100 is divided both ways.  counts[0] += comparisons,
// counts[1] += differing bit patterns other than a differently signed zero.
__global__ __launch_bounds__(256) void div_selftest_kernel(unsigned long long *counts, int n_div, uint32_t seed) {
  auto hash32 = [](uint32_t x) { x ^= x >> 16; x *= 0x7feb352du; x ^= x >> 15; x *= 0x846ca68bu; x ^= x >> 16; return x; };
  const uint32_t bi = blockIdx.x * 256u + threadIdx.x;
  if (bi >= (uint32_t)n_div) return;
  const uint32_t h = hash32(bi * 2654435761u + seed);
  const int ex = (int)(hash32(h) % 80u) - 40;
  const float b = __builtin_bit_cast(float, ((uint32_t)(127 + ex) << 23) | (h & 0x7fffffu));
  const float r = exact_rcp(b);
  unsigned long long bad = 0, tot = 0;
  for (uint32_t pat = 0; pat < 65536u; pat++) {
#pragma unroll
    for (int kind = 0; kind < 2; kind++) {
      const float a = kind == 0 ? elem_to_f32<1>((uint16_t)pat) : elem_to_f32<0>((uint16_t)pat);
      if (!__builtin_isfinite(a) || (__builtin_fabsf(a) < 0x1p-100f && a != 0.0f)) continue;
      const float want = a / b, got = div_by(a, b, r);
      const float mag = __builtin_fabsf(want);
      if (want != 0.0f && !(mag >= 0x1p-100f && mag <= 0x1p100f)) continue;   // outside the range the callers use
      tot++;
      if (__builtin_bit_cast(uint32_t, want) != __builtin_bit_cast(uint32_t, got) && !(want == 0.0f && got == 0.0f)) bad++;
    }
  }
  atomicAdd(&counts[0], tot);
  atomicAdd(&counts[1], bad);
}

// binary64 -> 16-bit pattern (round to nearest even) through binary32 where that provably gives the same bits: the
// first rounding (to 24 bits) can only change the second one when it lands exactly on a rounding tie of the 16-bit
// format, so every other value inside the format's normal range takes two hardware conversions instead of the 64-bit
// integer arithmetic of f64_to_elem; ties, zero-range, subnormal and overflowing values go the exact way.
template <int DT>
__device__ __forceinline__ uint16_t f64_to_elem_fast(double x) {
  const float r = (float)x;                                        // v_cvt_f32_f64
  const uint32_t b = __builtin_bit_cast(uint32_t, r);
  const uint32_t mag = b & 0x7fffffffu;
  constexpr uint32_t DROP = DT == 1 ? 16u : 13u;                   // binary32 mantissa bits the 16-bit format drops
  constexpr uint32_t LOW = (1u << DROP) - 1u, TIE = 1u << (DROP - 1u);
  constexpr uint32_t LO = DT == 1 ? 0x00800000u : 0x38800000u;     // 2^-126 / 2^-14: smallest normal of the format
  constexpr uint32_t HI = DT == 1 ? 0x7f000000u : 0x47000000u;     // 2^127 / 2^15: well below the overflow threshold
  const bool safe = mag == 0u || (mag >= LO && mag < HI && (b & LOW) != TIE);
  return safe ? f32_to_elem<DT>(r) : f64_to_elem<DT>(x);
}

// Packed 16-bit helpers.  A tile is kept in registers as the 16-bit patterns it was loaded with (two per register) and
// widened where it is used: half the registers of a binary32 copy, which is what lets enough workgroups share a CU to
// keep HBM busy.
typedef unsigned short u16x2_t __attribute__((ext_vector_type(2)));
__device__ __forceinline__ uint32_t pk_max_u16(uint32_t a, uint32_t b) {
  return __builtin_bit_cast(uint32_t, __builtin_elementwise_max(__builtin_bit_cast(u16x2_t, a), __builtin_bit_cast(u16x2_t, b)));
}
template <int DT> __device__ __forceinline__ void unpack2(uint32_t w, float &lo, float &hi) {
  lo = elem_to_f32<DT>((uint16_t)(w & 0xffffu));
  hi = elem_to_f32<DT>((uint16_t)(w >> 16));
}
// two binary32 values -> two 16-bit patterns, round to nearest even
template <int DT> __device__ __forceinline__ uint32_t pack_round2(float a, float b);
template <> __device__ __forceinline__ uint32_t pack_round2<0>(float a, float b) {
  typedef _Float16 h2 __attribute__((ext_vector_type(2)));
  typedef float f2 __attribute__((ext_vector_type(2)));
  const f2 v = {a, b};
  return __builtin_bit_cast(uint32_t, __builtin_convertvector(v, h2));
}
template <> __device__ __forceinline__ uint32_t pack_round2<1>(float a, float b) {
  typedef __bf16 bf2 __attribute__((ext_vector_type(2)));
  typedef float f2 __attribute__((ext_vector_type(2)));
  const f2 v = {a, b};
  return __builtin_bit_cast(uint32_t, __builtin_convertvector(v, bf2));   // v_cvt_pk_bf16_f32
}
// (int)y truncated toward zero, its low 8 bits written to byte B of acc: one instruction per element (the conversion's
// sub-dword destination select) instead of a conversion plus shifts and ors.  Byte 0 clears the other three bytes, bytes
// 1-3 keep them, so four calls in ascending order build a packed word without an initial value.
template <int B>
__device__ __forceinline__ void cvt_trunc_to_byte(uint32_t &acc, float y) {
  if constexpr (B == 0) asm("v_cvt_i32_f32_sdwa %0, %1 dst_sel:BYTE_0 dst_unused:UNUSED_PAD src0_sel:DWORD" : "=v"(acc) : "v"(y));
  else if constexpr (B == 1) asm("v_cvt_i32_f32_sdwa %0, %1 dst_sel:BYTE_1 dst_unused:UNUSED_PRESERVE src0_sel:DWORD" : "+v"(acc) : "v"(y));
  else if constexpr (B == 2) asm("v_cvt_i32_f32_sdwa %0, %1 dst_sel:BYTE_2 dst_unused:UNUSED_PRESERVE src0_sel:DWORD" : "+v"(acc) : "v"(y));
  else asm("v_cvt_i32_f32_sdwa %0, %1 dst_sel:BYTE_3 dst_unused:UNUSED_PRESERVE src0_sel:DWORD" : "+v"(acc) : "v"(y));
}
// Hides a register's value from the optimiser: placed between two passes over the packed tile, it keeps the compiler
// from carrying the widened (binary32) copies of one pass over to the next, which would double the registers again.
__device__ __forceinline__ void forget(uint32_t &v) { asm volatile("" : "+v"(v)); }
__device__ __forceinline__ uint32_t wave_max_u32(uint32_t v) {
#pragma unroll
  for (int o = 32; o >= 1; o >>= 1) v = max(v, (uint32_t)__shfl_xor((int)v, o, SPG_WAVE));
  return v;
}

// One workgroup handles 128 consecutive rows of one (batch, head): one 128-row block or two 64-row blocks (SUB), so
// that the per-block tail (column reduction, pooled mean, flag, scale) is spread over all four wavefronts in both cases.
// QR = rows that share one INT8 scale: BS (per-block granularity, what the reference's operators use) or 32 rows of a
// 128-row Q block (per-warp granularity: quant_per_block.py:102-148 with WARPQ = 32, one scale per 32 query rows, which
// are the rows of one wavefront of the attention kernel).  Pooling and the similarity flag stay per block.
template <int BS, int D, int DT, bool HAS_MEAN, bool WITH_POOL, int QR = BS>
__global__ __launch_bounds__(256) void pool_sim_quant_kernel(const uint16_t *__restrict__ x, const Strides xs,
                                                             const uint16_t *__restrict__ km,
                                                             uint16_t *__restrict__ pool, uint8_t *__restrict__ sim,
                                                             int8_t *__restrict__ xq, float *__restrict__ scale,
                                                             const float *__restrict__ simthr, int H, int N, int nb) {
  constexpr int ROWS = 128;           // rows per workgroup
  constexpr int SUB = ROWS / BS;      // blocks per workgroup
  constexpr int TPR = D / 8;          // lanes per row (16 B each)
  constexpr int RPP = 256 / TPR;      // rows per pass of the workgroup
  constexpr int NPT = ROWS / RPP;     // passes (rows per thread)
  constexpr int NP = BS / RPP;        // passes per block
  constexpr int WPS = D / 64;         // wavefronts that hold one block's columns in the tail (thread = block * D + column)
  constexpr int NQG = ROWS / QR;      // quantisation groups per workgroup (1, 2 or 4)
  constexpr int GPB = BS / QR;        // ... per block
  constexpr int NPQ = QR / RPP;       // passes per quantisation group
  static_assert(BS == 64 || BS == 128, "block sizes of the operators");
  static_assert(QR == BS || (QR == 32 && BS == 128), "per-block, or 32-row groups of a Q block");
  static_assert(RPP <= QR, "a pass of the workgroup stays inside one quantisation group");
  static_assert(RPP <= BS && SUB * D <= 256, "thread <-> (block, column) mapping of the tail");
  // magnitude patterns (sign bit cleared) order like the magnitudes, for both 16-bit formats
  constexpr uint32_t ABS2 = 0x7fff7fffu;
  constexpr uint32_t INF16 = DT == 1 ? 0x7f80u : 0x7c00u;
  // "every element of the row is tiny": bfloat16 below 2^-63 (both top exponent bits clear), binary16 zero
  constexpr uint32_t TINY2 = DT == 1 ? 0x60006000u : 0x7fff7fffu;
  const int bh = blockIdx.y;
  const int tid = threadIdx.x, c = tid % TPR, r = tid / TPR;
  const int row_base = blockIdx.x * ROWS;
  const int rows_here = min(ROWS, N - row_base);          // >= 1
  const bool partial = rows_here < ROWS;                  // workgroup-uniform: only the last workgroup of a head
  const int blk0 = blockIdx.x * SUB;
  auto rows_valid_of = [&](int sb) { return max(0, min(BS, rows_here - sb * BS)); };
  const uint16_t *xb = x + (size_t)(bh / H) * xs.sb + (size_t)(bh % H) * xs.sh + (size_t)row_base * xs.sn + c * 8;

  float kmf[8];
  if constexpr (HAS_MEAN) {
    const uint4 v = *(const uint4 *)(km + (size_t)bh * D + c * 8);
    unpack2<DT>(v.x, kmf[0], kmf[1]);
    unpack2<DT>(v.y, kmf[2], kmf[3]);
    unpack2<DT>(v.z, kmf[4], kmf[5]);
    unpack2<DT>(v.w, kmf[6], kmf[7]);
  }

  // all loads of the thread are issued before the first use (rows beyond the end re-read the last row and are zeroed
  // afterwards: no load sits behind a branch)
  uint32_t w[NPT][4];
  {
    uint4 raw[NPT];
#pragma unroll
    for (int p = 0; p < NPT; p++) raw[p] = load_stream_u4(xb + (size_t)min(r + p * RPP, rows_here - 1) * xs.sn);
#pragma unroll
    for (int p = 0; p < NPT; p++) { w[p][0] = raw[p].x; w[p][1] = raw[p].y; w[p][2] = raw[p].z; w[p][3] = raw[p].w; }
  }
  if constexpr (HAS_MEAN) {
    // (k - km) rounded once to the input dtype (utils.py:184-188).  The binary32 difference of two 16-bit floats is
    // either exact or nowhere near a rounding tie of the 16-bit format, so rounding it to nearest even equals rounding
    // the exact difference.  The tile is kept as the rounded 16-bit patterns.
#pragma unroll
    for (int p = 0; p < NPT; p++)
#pragma unroll
      for (int j = 0; j < 4; j++) {
        float f0, f1;
        unpack2<DT>(w[p][j], f0, f1);
        w[p][j] = pack_round2<DT>(f0 - kmf[2 * j], f1 - kmf[2 * j + 1]);
      }
  }
  if (partial) {                                  // masked rows are zero (utils.py:188)
#pragma unroll
    for (int p = 0; p < NPT; p++)
      if (r + p * RPP >= rows_here) { w[p][0] = 0; w[p][1] = 0; w[p][2] = 0; w[p][3] = 0; }
  }

  // largest magnitude of the thread's elements per quantisation group (as 16-bit patterns: group g in half g % 2 of
  // word g / 2) and, per row, whether all of the thread's elements are tiny
  constexpr int MW = (NQG + 1) / 2;
  uint32_t m_thread[MW], tiny_rows = 0;
#pragma unroll
  for (int i = 0; i < MW; i++) m_thread[i] = 0;
#pragma unroll
  for (int g = 0; g < NQG; g++) {
    uint32_t m2 = 0;
#pragma unroll
    for (int p = g * NPQ; p < (g + 1) * NPQ; p++) {
      const uint32_t rm = pk_max_u16(pk_max_u16(w[p][0] & ABS2, w[p][1] & ABS2), pk_max_u16(w[p][2] & ABS2, w[p][3] & ABS2));
      m2 = pk_max_u16(m2, rm);
      if constexpr (WITH_POOL) tiny_rows |= ((rm & TINY2) == 0 ? 1u : 0u) << p;
    }
    m_thread[g / 2] |= max(m2 & 0xffffu, m2 >> 16) << (16 * (g % 2));
  }
  // A NaN pattern lies above the infinity pattern and wins the maxima above.  The similarity flag wants exactly that
  // (a block with a NaN is never "similar"), the quantisation scale does not: the reference's block maximum ignores NaN
  // (tl.max lowers to a maxnum, utils.py:140 / 206), so only the NaN elements themselves are poisoned (they quantise to
  // 0).  m_raw keeps the maxima with NaN for the flag; a thread that met one recomputes m_thread without (rare).
  uint32_t m_raw[MW];
#pragma unroll
  for (int i = 0; i < MW; i++) m_raw[i] = m_thread[i];
  {
    bool nan_seen = false;
#pragma unroll
    for (int i = 0; i < MW; i++) nan_seen |= (m_thread[i] & 0xffffu) > INF16 || (m_thread[i] >> 16) > INF16;
    if (nan_seen) {
#pragma unroll
      for (int i = 0; i < MW; i++) m_thread[i] = 0;
#pragma unroll
      for (int g = 0; g < NQG; g++) {
        uint32_t m1 = 0;
#pragma unroll
        for (int p = g * NPQ; p < (g + 1) * NPQ; p++)
#pragma unroll
          for (int j = 0; j < 4; j++) {
            const uint32_t lo = w[p][j] & 0x7fffu, hi = (w[p][j] >> 16) & 0x7fffu;
            m1 = max(m1, max(lo > INF16 ? 0u : lo, hi > INF16 ? 0u : hi));
          }
        m_thread[g / 2] |= m1 << (16 * (g % 2));
      }
    }
  }
  // largest magnitude pattern of block sb as this thread (or, after the reduction, the workgroup) knows it
  auto block_max = [&](const uint32_t(&mm)[MW], int sb) -> uint32_t {
    uint32_t m = 0;
#pragma unroll
    for (int g = sb * GPB; g < (sb + 1) * GPB; g++) m = max(m, (mm[g / 2] >> (16 * (g % 2))) & 0xffffu);
    return m;
  };
  __shared__ uint32_t s_wmax[4][MW], s_wbad[4];
  __shared__ long long s_wg[4];
#pragma unroll
  for (int i = 0; i < MW; i++) {
    uint32_t mw = m_thread[i];                    // two groups' maxima reduced together
#pragma unroll
    for (int o = 32; o >= 1; o >>= 1) mw = pk_max_u16(mw, (uint32_t)__shfl_xor((int)mw, o, SPG_WAVE));
    if ((tid & 63) == 0) s_wmax[tid >> 6][i] = mw;
  }

  if constexpr (WITH_POOL) {
    // column sums of all blocks of the workgroup, one row group per line; used for the pooled mean first and, with a
    // non-negative similarity threshold, for the normalised rows afterwards
    __shared__ double s_red[SUB][RPP][D];
    // column sums for the pooled mean: binary64, exact
#pragma unroll
    for (int sb = 0; sb < SUB; sb++) {
      double colsum[8];
#pragma unroll
      for (int e = 0; e < 8; e++) colsum[e] = 0.0;
#pragma unroll
      for (int p = sb * NP; p < (sb + 1) * NP; p++)
#pragma unroll
        for (int j = 0; j < 4; j++) {
          float f0, f1;
          forget(w[p][j]);
          unpack2<DT>(w[p][j], f0, f1);
          colsum[2 * j] += (double)f0;
          colsum[2 * j + 1] += (double)f1;
        }
#pragma unroll
      for (int e = 0; e < 8; e++) s_red[sb][r][c * 8 + e] = colsum[e];
    }

    // row norms: the TPR lanes of a row group all need sqrt(sum of squares) and its reciprocal for each of their NPT
    // rows.  Both are computed ONCE per NPT rows - lane c of the group takes row c % NPT - and handed round with lane
    // reads, instead of NPT times in every lane.
    static_assert(NPT <= TPR, "one lane of the row group per row");
    // A NEGATIVE similarity threshold (the top-k operators' default, -0.1) decides the flag without the normalised rows:
    // the statistic is ||sum of x_hat||^2 / rows^2 >= 0 > threshold whenever every x_hat is finite.  x_hat = x / norm is
    // non-finite exactly for rows with norm == 0 (all-zero rows such as the padding of a partial block, or rows too
    // small for their squares) and for non-finite x; |x| <= norm (1 + 2^-23) keeps every other quotient within fp16.
    // Only two facts about the rows are needed then: is any element non-finite, and does any row have a zero norm.  A
    // row whose largest |x| is at least 2^-63 has a sum of squares of at least 2^-126, a positive binary32 number; rows
    // in which every element is smaller (all-zero rows, the padding of a partial block, bfloat16 values near the bottom
    // of the range) are decided by the exact sums below.
    const bool sim_trivial = simthr[bh % H] < 0.f;     // workgroup-uniform
    uint32_t bad = 0;                                  // bit sb: block sb holds a non-finite x_hat
    float ssf_mine = 0.f;
    bool need_norms = true;                            // wavefront-uniform
    if (sim_trivial) {
#pragma unroll
      for (int sb = 0; sb < SUB; sb++)                 // inf or NaN anywhere (overflowing squares of finite values are harmless: x / inf = 0)
        bad |= (block_max(m_raw, sb) >= INF16 ? 1u : 0u) << sb;
      tiny_rows = group_and_u32<TPR>(tiny_rows);      // rows tiny in every lane of their group
      need_norms = __any(tiny_rows != 0);             // rare
    }
    if (need_norms) {
      // sum of squares of every row (exact in binary64), rounded to binary32 like the reference's (utils.py:194)
#pragma unroll
      for (int p = 0; p < NPT; p++) {
        double ss = 0.0;
#pragma unroll
        for (int j = 0; j < 4; j++) {
          float f0, f1;
          forget(w[p][j]);
          unpack2<DT>(w[p][j], f0, f1);
          const double d0 = (double)f0, d1 = (double)f1;
          ss = __builtin_fma(d0, d0, ss);             // squares and their sum are exact in binary64
          ss = __builtin_fma(d1, d1, ss);
        }
        ss = group_sum_f64<TPR>(ss);                 // the TPR lanes of this row
        const float ssf = (float)ss;
        ssf_mine = (c % NPT == p) ? ssf : ssf_mine;
        if (sim_trivial) bad |= ((ssf == 0.f) ? 1u : 0u) << (p / NP);
      }
    }
    __syncthreads();
    // tail: thread = block * D + column
    const int t_sb = tid / D, t_col = tid % D;
    const bool t_on = tid < SUB * D;
    const int t_rows = rows_valid_of(t_sb);
    if (t_on && t_rows > 0) {
      double s = 0.0;
      for (int i = 0; i < RPP; i++) s += s_red[t_sb][i][t_col];
      // full blocks: the row count is a power of two, so the product with its reciprocal is the exact quotient
      const double mean = t_rows == BS ? s * (1.0 / BS) : s / (double)t_rows;
      pool[((size_t)bh * nb + blk0 + t_sb) * D + t_col] = f64_to_elem_fast<DT>(mean);
    }
    long long g = 0;
    if (!sim_trivial) {
      __syncthreads();                                // s_red is reused
      const float norm_mine = sqrtf(ssf_mine);
      const float rn_mine = rcp_safe(norm_mine) ? exact_rcp(norm_mine) : 0.f;
      const int group_lane0 = (tid & 63) & ~(TPR - 1);
#pragma unroll
      for (int sb = 0; sb < SUB; sb++) {
        double colxh[8];
#pragma unroll
        for (int e = 0; e < 8; e++) colxh[e] = 0.0;
#pragma unroll
        for (int p = sb * NP; p < (sb + 1) * NP; p++) {
          const float norm = __shfl(norm_mine, group_lane0 + p, SPG_WAVE);
          const float rn = __shfl(rn_mine, group_lane0 + p, SPG_WAVE);
          const bool fast = rcp_safe(norm);
#pragma unroll
          for (int j = 0; j < 4; j++) {
            float f0, f1;
            forget(w[p][j]);
            unpack2<DT>(w[p][j], f0, f1);
            // the slow branch gives 0/0 = NaN for all-zero (masked) rows
            const _Float16 h0 = (_Float16)(fast ? div_by(f0, norm, rn) : f0 / norm);
            const _Float16 h1 = (_Float16)(fast ? div_by(f1, norm, rn) : f1 / norm);
            colxh[2 * j] += (double)(float)h0;        // fp16 values: integer multiples of 2^-24, sums are exact
            colxh[2 * j + 1] += (double)(float)h1;
          }
        }
#pragma unroll
        for (int e = 0; e < 8; e++) s_red[sb][r][c * 8 + e] = colxh[e];
      }
      __syncthreads();
      if (t_on) {
        double sx = 0.0;
        for (int i = 0; i < RPP; i++) sx += s_red[t_sb][i][t_col];
        if (__builtin_isfinite(sx)) {
          const long long si = (long long)(sx * 16777216.0);   // exact integer
          g = si * si;
        } else {
          bad |= 1u << t_sb;                          // a NaN/inf x_hat anywhere in the column
        }
      }
#pragma unroll
      for (int o = 32; o >= 1; o >>= 1) g += shfl_xor_i64(g, o);
      if ((tid & 63) == 0) s_wg[tid >> 6] = g;
    }
    // bit sb of any_bad: some thread saw a non-finite x_hat in block sb (one flag word per wavefront, combined below)
    {
      uint32_t wb = 0;
#pragma unroll
      for (int sb = 0; sb < SUB; sb++) wb |= (__any((bad >> sb) & 1u) ? 1u : 0u) << sb;
      if ((tid & 63) == 0) s_wbad[tid >> 6] = wb;
    }
    __syncthreads();
    const uint32_t any_bad = s_wbad[0] | s_wbad[1] | s_wbad[2] | s_wbad[3];
    if (tid < SUB && rows_valid_of(tid) > 0) {
      const int rv = rows_valid_of(tid);
      bool similar = sim_trivial;
      if (!sim_trivial) {
        long long gt = 0;                             // = sum(gram) * 2^48, exact
        for (int i = 0; i < WPS; i++) gt += s_wg[tid * WPS + i];
        const double thr = (double)simthr[bh % H] * (double)(rv * rv) * 281474976710656.0;
        similar = (double)gt > thr;
      }
      sim[(size_t)bh * nb + blk0 + tid] = (!((any_bad >> tid) & 1u) && similar) ? 1 : 0;
    }
  } else {
    __syncthreads();
  }

  uint32_t m_all[MW];
#pragma unroll
  for (int i = 0; i < MW; i++)
    m_all[i] = pk_max_u16(pk_max_u16(s_wmax[0][i], s_wmax[1][i]), pk_max_u16(s_wmax[2][i], s_wmax[3][i]));
  int8_t *qb = xq + ((size_t)bh * N + row_base) * D + c * 8;
#pragma unroll
  for (int g = 0; g < NQG; g++) {
    // per-block scales exist for blocks with at least one row; the 32-row groups of the last Q block all get a scale
    // (1e-7 for a group without rows, what the reference's quantiser writes for an all-masked group)
    if (QR == BS && rows_here - g * QR <= 0) break;     // workgroup-uniform
    const float amax = elem_to_f32<DT>((uint16_t)(m_all[g / 2] >> (16 * (g % 2))));
    const float s = amax / 127.0f + 1e-7f;
    auto quantise = [&](auto divide, auto check_rows) {
#pragma unroll
      for (int p = g * NPQ; p < (g + 1) * NPQ; p++) {
        const int row = r + p * RPP;
        if (!decltype(check_rows)::value || row < rows_here) {
          float y[8];
#pragma unroll
          for (int j = 0; j < 4; j++) {
            float f[2];
            forget(w[p][j]);
            unpack2<DT>(w[p][j], f[0], f[1]);
#pragma unroll
            for (int h = 0; h < 2; h++) {
              const float t = divide(f[h]);
              y[2 * j + h] = t + __builtin_copysignf(0.5f, t);   // +0.5 for t >= 0 (a -0 quotient truncates to 0 either way)
            }
          }
          uint32_t pk0, pk1;                       // truncation toward zero, low 8 bits of element e into byte e % 4
          cvt_trunc_to_byte<0>(pk0, y[0]); cvt_trunc_to_byte<1>(pk0, y[1]); cvt_trunc_to_byte<2>(pk0, y[2]); cvt_trunc_to_byte<3>(pk0, y[3]);
          cvt_trunc_to_byte<0>(pk1, y[4]); cvt_trunc_to_byte<1>(pk1, y[5]); cvt_trunc_to_byte<2>(pk1, y[6]); cvt_trunc_to_byte<3>(pk1, y[7]);
          *(uint2 *)(qb + (size_t)row * D) = make_uint2(pk0, pk1);
        }
      }
    };
    if (rcp_safe(s) && !partial) {         // workgroup-uniform; the common case carries no row test
      const float rs = exact_rcp(s);
      quantise([&](float v) { return div_by(v, s, rs); }, std::false_type{});
    } else if (rcp_safe(s)) {
      const float rs = exact_rcp(s);
      quantise([&](float v) { return div_by(v, s, rs); }, std::true_type{});
    } else {
      quantise([&](float v) { return v / s; }, std::true_type{});
    }
    if (tid == 0) scale[((size_t)bh * nb + blk0) * GPB + g] = s;
  }
}

// =============================================================================================
// canonical exp: a fixed sequence of binary64 mul / add (no fma), t <= 0.
// =============================================================================================
__device__ __forceinline__ double cexp(double t) {
  if (!(t >= -700.0)) return 0.0;
  const double k = __builtin_rint(t * 1.4426950408889634);
  const double r = (t - k * 0.6931471803691238) - k * 1.9082149292705877e-10;
  double p = 1.0 / 6227020800.0;
  p = p * r; p = p + 1.0 / 479001600.0;
  p = p * r; p = p + 1.0 / 39916800.0;
  p = p * r; p = p + 1.0 / 3628800.0;
  p = p * r; p = p + 1.0 / 362880.0;
  p = p * r; p = p + 1.0 / 40320.0;
  p = p * r; p = p + 1.0 / 5040.0;
  p = p * r; p = p + 1.0 / 720.0;
  p = p * r; p = p + 1.0 / 120.0;
  p = p * r; p = p + 1.0 / 24.0;
  p = p * r; p = p + 1.0 / 6.0;
  p = p * r; p = p + 1.0 / 2.0;
  p = p * r; p = p + 1.0;
  p = p * r; p = p + 1.0;
  return __builtin_ldexp(p, (int)k);
}

// exclusive prefix of per-thread counts over the 256 threads of the workgroup; returns (offset, total)
__device__ __forceinline__ int2 block_exclusive_scan_i32(int v, int *s_tmp /* >= 4 ints */) {
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  int inc = v;
#pragma unroll
  for (int o = 1; o < 64; o <<= 1) {
    const int t = __shfl_up(inc, o, SPG_WAVE);
    if (lane >= o) inc += t;
  }
  __syncthreads();                       // s_tmp may still be read from a previous call
  if (lane == 63) s_tmp[wave] = inc;
  __syncthreads();
  const int w0 = s_tmp[0], w1 = s_tmp[1], w2 = s_tmp[2], w3 = s_tmp[3];
  const int base = (wave > 0 ? w0 : 0) + (wave > 1 ? w1 : 0) + (wave > 2 ? w2 : 0);
  return make_int2(base + inc - v, w0 + w1 + w2 + w3);
}

// flags (per column, via functor) -> ascending compact index list -> delta LUT, zero tail, valid count.
template <class FlagFn>
__device__ __forceinline__ void emit_lut(FlagFn flag, int nk, int nkp, int32_t *s_idx, int *s_tmp,
                                         int32_t *__restrict__ lut_row, int32_t *__restrict__ valid_out) {
  const int tid = threadIdx.x;
  const int seg = nkp / 256;
  const int j0 = tid * seg, j1 = min(nk, j0 + seg);
  int cnt = 0;
  for (int j = j0; j < j1; j++) cnt += flag(j) ? 1 : 0;
  const int2 st = block_exclusive_scan_i32(cnt, s_tmp);
  int pos = st.x;
  for (int j = j0; j < j1; j++)
    if (flag(j)) s_idx[pos++] = j;
  __syncthreads();
  for (int p = tid; p < nk; p += 256) {
    int v = 0;
    if (p < st.y) v = s_idx[p] - (p ? s_idx[p - 1] : 0);
    lut_row[p] = v;
  }
  if (tid == 0) *valid_out = st.y;
}

// =============================================================================================
// block_select: one workgroup per (R consecutive q block rows, b*h).
// Phase 1 computes the R x nk pooled scores with every pooled-K row read ONCE for the R rows (one lane per
// column, binary64 accumulation in the fixed order d = 0..D-1); phase 2 handles the rows one after the other:
// softmax, stable descending sort, top-k / CDF count, block-map row, delta LUT.
// dynamic LDS: R*D*8 (pooled Q as doubles) + R*nkp*4 (scores) + 12*nkp (per-row work area).
// =============================================================================================
template <int D, int DT, int R>
__global__ __launch_bounds__(256) void block_select_kernel(
    const uint16_t *__restrict__ pool_q, const uint8_t *__restrict__ sim_q, const uint16_t *__restrict__ pool_k,
    const uint8_t *__restrict__ sim_k, const float *__restrict__ topk, const float *__restrict__ cdfthr, int is_causal,
    int sink, int32_t *__restrict__ lut, int32_t *__restrict__ valid, uint8_t *__restrict__ bmap, int H, int Hkv, int nq,
    int nk, int nkp) {
  extern __shared__ __align__(16) unsigned char smem[];
  double *s_pq = (double *)smem;                                   // [R][D]
  float *s_scores = (float *)(smem + (size_t)R * D * 8);           // [R][nkp]
  unsigned char *work = smem + (size_t)R * D * 8 + (size_t)R * nkp * 4;
  double *e_buf = (double *)work;                      // [nkp] exp values        (step 1)
  uint32_t *skey = (uint32_t *)work;                   // [nkp] sorted keys       (step 2, aliases e_buf)
  int32_t *s_idx = (int32_t *)(work + 4 * (size_t)nkp);    // [nkp] compact indices (step 3, aliases e_buf)
  uint32_t *okey = (uint32_t *)(work + 8 * (size_t)nkp);   // [nkp] keys in column order
  __shared__ float s_wmax[4];
  __shared__ double s_wsum[4];
  __shared__ double s_tsum[256];
  __shared__ int s_tmp[256];
  __shared__ int s_n;

  const int i0 = blockIdx.x * R, bh = blockIdx.y, h = bh % H, tid = threadIdx.x;
  const int rows = min(R, nq - i0);
  for (int t = tid; t < R * D; t += 256) {
    const int row = t / D;
    s_pq[t] = row < rows ? (double)elem_to_f32<DT>(pool_q[((size_t)bh * nq + i0 + row) * D + (t % D)]) : 0.0;
  }
  __syncthreads();

  const float sm_scale = (D == 64) ? 0.125f : 0.088388347648318447f;  // fp32(D^-0.5)
  // grouped K/V heads: query head h is scored against the pooled blocks of K head h / (H / Hkv)
  const int bhk = (bh / H) * Hkv + h / (H / Hkv);
  const uint16_t *pk_base = pool_k + (size_t)bhk * nk * D;
  const uint8_t *simk = sim_k + (size_t)bhk * nk;

  // ---- phase 1: scores.  Products of two 16-bit floats are exact in binary64, so fma == multiply-then-add. ----
  for (int j = tid; j < nk; j += 256) {
    double acc[R];
#pragma unroll
    for (int row = 0; row < R; row++) acc[row] = 0.0;
    const uint4 *krow = (const uint4 *)(pk_base + (size_t)j * D);
#pragma unroll 2
    for (int cch = 0; cch < D / 8; cch++) {
      const uint4 v = krow[cch];
      const uint32_t w[4] = {v.x, v.y, v.z, v.w};
      double kd[8];
#pragma unroll
      for (int e = 0; e < 8; e++)
        kd[e] = (double)elem_to_f32<DT>((uint16_t)((e & 1) ? (w[e >> 1] >> 16) : (w[e >> 1] & 0xffffu)));
#pragma unroll
      for (int row = 0; row < R; row++) {
        const double *q = s_pq + row * D + cch * 8;
#pragma unroll
        for (int e = 0; e < 8; e++) acc[row] = __builtin_fma(q[e], kd[e], acc[row]);
      }
    }
    const bool dead_col = simk[j] == 0;
#pragma unroll
    for (int row = 0; row < R; row++) {
      const float s1 = elem_to_f32<DT>(f64_to_elem<DT>(acc[row]));
      float s2 = elem_to_f32<DT>(f64_to_elem<DT>((double)s1 * (double)sm_scale));
      if (dead_col || (is_causal && j >= 2 * (i0 + row + 1))) s2 = -INFINITY;
      s_scores[(size_t)row * nkp + j] = s2;
    }
  }
  __syncthreads();

  // ---- phase 2: one row at a time ------------------------------------------------------------------------
  for (int row = 0; row < rows; row++) {
    const int i = i0 + row;
    const int causal_lim = is_causal ? min(nk, 2 * (i + 1)) : nk;
    const float *s_score = s_scores + (size_t)row * nkp;

    float lmax = -INFINITY;
    for (int j = tid; j < nk; j += 256) lmax = fmaxf(lmax, s_score[j]);
    lmax = wave_max_f32(lmax);
    if ((tid & 63) == 0) s_wmax[tid >> 6] = lmax;
    __syncthreads();
    const float mx = fmaxf(fmaxf(s_wmax[0], s_wmax[1]), fmaxf(s_wmax[2], s_wmax[3]));

    // exp, then the fixed summation tree: lane l of ONE wavefront adds e[l], e[l+64], ... in order, followed by an
    // xor butterfly (32 .. 1)
    for (int j = tid; j < nk; j += 256) {
      const float s2 = s_score[j];
      e_buf[j] = (s2 == -INFINITY) ? 0.0 : cexp((double)s2 - (double)mx);
    }
    __syncthreads();
    if (tid < 64) {
      double part = 0.0;
      for (int j = tid; j < nk; j += 64) part = part + e_buf[j];
#pragma unroll
      for (int o = 32; o >= 1; o >>= 1) part = part + shfl_xor_f64(part, o);
      if (tid == 0) s_wsum[0] = part;
    }
    __syncthreads();
    const double total = s_wsum[0];

    // probabilities -> sortable keys (value bits, then lower index first)
    for (int j = tid; j < nk; j += 256) {
      double p = e_buf[j] / total;
      if (!__builtin_isfinite(p)) p = 0.0;
      const uint32_t bits = f64_to_elem<DT>(p);
      okey[j] = (bits << 16) | (0xffffu - (uint32_t)j);
    }
    __syncthreads();
    for (int j = tid; j < nkp; j += 256) skey[j] = (j < nk) ? okey[j] : 0u;
    __syncthreads();

    // bitonic sort, descending
    for (int k = 2; k <= nkp; k <<= 1) {
      for (int lj = __builtin_ctz(k) - 1; lj >= 0; lj--) {     // compare distance j = 2^lj
        const int j = 1 << lj;
        for (int t = tid; t < nkp / 2; t += 256) {
          const int lo = ((t >> lj) << (lj + 1)) | (t & (j - 1));
          const int hi = lo | j;
          const bool desc = (lo & k) == 0;
          const uint32_t a = skey[lo], b = skey[hi];
          if ((a < b) == desc) { skey[lo] = b; skey[hi] = a; }
        }
        __syncthreads();
      }
    }

    // how many to keep
    long long n;
    if (topk != nullptr) {
      const float t = topk[h] * (float)nk;     // binary32 product, truncated (utils.py:405)
      n = (long long)t;
    } else {
      // cdf[i] = T(sum_{u<=i} p_sorted[u]);  n = #{i < nk : cdf[i] <= threshold}  (utils.py:398-403)
      const int seg = nkp / 256;
      const int p0 = tid * seg;
      double lsum = 0.0;
      for (int u = 0; u < seg; u++) lsum += (double)elem_to_f32<DT>((uint16_t)(skey[p0 + u] >> 16));
      s_tsum[tid] = lsum;
      __syncthreads();
      double run = 0.0;
      for (int u = 0; u < tid; u++) run += s_tsum[u];
      const double thr = (double)cdfthr[h];
      int cnt = 0;
      for (int u = 0; u < seg; u++) {
        run += (double)elem_to_f32<DT>((uint16_t)(skey[p0 + u] >> 16));
        const float cdfv = elem_to_f32<DT>(f64_to_elem<DT>(run));
        if (p0 + u < nk && (double)cdfv <= thr) cnt++;
      }
      cnt = wave_sum_i32(cnt);
      if (tid == 0) s_n = 0;
      __syncthreads();
      if ((tid & 63) == 0) atomicAdd(&s_n, cnt);
      __syncthreads();
      n = s_n;
    }
    if (n <= 0) n = 1;                              // utils.py:289
    const uint32_t kth = (n >= nk) ? 0u : skey[n - 1];
    __syncthreads();                                // skey is dead from here

    // block map row and LUT
    const bool row_forced = sim_q[(size_t)bh * nq + i] == 0;
    auto flag = [&](int j) -> bool {
      bool f = row_forced || (okey[j] >= kth) || (simk[j] == 0);
      if (j >= causal_lim) f = false;
      if (sink && j == 0) f = true;
      return f;
    };
    const size_t row_off = ((size_t)bh * nq + i) * nk;
    if (bmap != nullptr)
      for (int j = tid; j < nk; j += 256) bmap[row_off + j] = flag(j) ? 1 : 0;
    emit_lut(flag, nk, nkp, s_idx, s_tmp, lut + row_off, valid + (size_t)bh * nq + i);
    __syncthreads();                                // the work area is reused by the next row
  }
}

// =============================================================================================
// block_select, wavefront-per-row variant (nk <= 2048).
// Phase 1 computes the scores of 16 pooled-Q rows against all pooled-K rows on the matrix unit in binary64
// (v_mfma_f64_16x16x4_f64: operands are delivered once per 1024 multiply-adds instead of once per multiply-add) and
// leaves them in LDS as 16-bit patterns.  Phase 2 gives each of the four wavefronts its own rows and keeps a whole row
// in registers (EPL = nkp / 64 columns per lane): no workgroup barrier, the stable descending sort is a bitonic network
// whose short-distance steps are register-local and whose long-distance steps are lane exchanges.
// dynamic LDS: 16*nkp*2 (scores) + 4*nkp*4 (per-wave index list) + 4*64*8 (lane sums).
// =============================================================================================
template <int EPL, int K, int J>
__device__ __forceinline__ void bitonic_step(uint32_t (&key)[EPL], int lane) {
  constexpr int NKP = 64 * EPL;
  // element v = lane * EPL + t; a step compares v with v ^ J inside blocks of size K (descending where (v & K) == 0)
  if constexpr (J >= EPL) {
    constexpr int DL = J / EPL;                                     // partner lane = lane ^ DL
    const bool lower = (lane & DL) == 0;
    const bool desc = (K >= NKP) ? true : ((lane & (K / EPL)) == 0);
    const bool want_max = lower == desc;
#pragma unroll
    for (int t = 0; t < EPL; t++) {
      const uint32_t o = (uint32_t)__shfl_xor((int)key[t], DL, SPG_WAVE);
      const uint32_t mx = key[t] > o ? key[t] : o, mn = key[t] > o ? o : key[t];
      key[t] = want_max ? mx : mn;
    }
  } else {
#pragma unroll
    for (int t = 0; t < EPL; t++) {
      if ((t & J) == 0) {
        const uint32_t a = key[t], b = key[t | J];
        const uint32_t mx = a > b ? a : b, mn = a > b ? b : a;
        if constexpr (K < EPL) {
          const bool desc = (t & K) == 0;                           // compile-time
          key[t] = desc ? mx : mn;
          key[t | J] = desc ? mn : mx;
        } else {
          const bool desc = (K >= NKP) ? true : ((lane & (K / EPL)) == 0);
          key[t] = desc ? mx : mn;
          key[t | J] = desc ? mn : mx;
        }
      }
    }
  }
}
template <int EPL, int K, int J>
__device__ __forceinline__ void bitonic_inner(uint32_t (&key)[EPL], int lane) {
  bitonic_step<EPL, K, J>(key, lane);
  if constexpr (J > 1) bitonic_inner<EPL, K, J / 2>(key, lane);
}
template <int EPL, int K>
__device__ __forceinline__ void bitonic_sort_desc(uint32_t (&key)[EPL], int lane) {
  bitonic_inner<EPL, K, K / 2>(key, lane);
  if constexpr (K < 64 * EPL) bitonic_sort_desc<EPL, K * 2>(key, lane);
}

template <int D, int DT, int NW, int EPL, bool DUAL>
__global__ __launch_bounds__(64 * NW, (!DUAL && NW == 8) ? 2 : 1) void block_select_wave_kernel(
    const uint16_t *__restrict__ pool_q, const uint8_t *__restrict__ sim_q, const uint16_t *__restrict__ pool_k,
    const uint8_t *__restrict__ sim_k, const float *__restrict__ topk, const float *__restrict__ cdfthr, int is_causal,
    int sink, int32_t *__restrict__ lut, int32_t *__restrict__ valid, uint8_t *__restrict__ bmap, int H, int Hkv, int nq,
    int nk) {
  constexpr int R = 16;             // rows per workgroup: phase 1 computes 16 x 16 score tiles on the matrix unit
  constexpr int NKP = 64 * EPL;
  static_assert(NW == 8 || NW == 16, "wavefronts per workgroup");
  extern __shared__ __align__(16) unsigned char smem[];
  uint16_t *s_scores = (uint16_t *)smem;                                      // [R][NKP] scores as 16-bit patterns
  uint16_t *s_idx_all = (uint16_t *)(smem + (size_t)R * NKP * 2);             // [NW][NKP] (column indices are below 2048)
  double *s_lsum_all = (double *)(smem + (size_t)R * NKP * 2 + NW * (size_t)NKP * 2);   // [NW][64]

  // Causal rows get heavier with the row index.  Workgroups that differ by 8 in blockIdx.y tend to share a CU (ids are
  // dealt round-robin over 8 XCDs, then over the CUs of an XCD), so the row-group index is rotated by a quarter of
  // the grid per such step: a CU then holds a mix of light and heavy row groups.
  const int bx = (int)((blockIdx.x + (blockIdx.y >> 3) * (gridDim.x >> 2)) % gridDim.x);
  const int i0 = bx * R, bh = blockIdx.y, h = bh % H, tid = threadIdx.x;
  const int rows = min(R, nq - i0);
  const int lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);

  const float sm_scale = (D == 64) ? 0.125f : 0.088388347648318447f;  // fp32(D^-0.5)
  // grouped K/V heads: query head h is scored against the pooled blocks of K head h / (H / Hkv)
  const int bhk = (bh / H) * Hkv + h / (H / Hkv);
  const uint16_t *pk_base = pool_k + (size_t)bhk * nk * D;
  const uint8_t *simk = sim_k + (size_t)bhk * nk;

  // ---- phase 1: the 16 x nk pooled scores in binary64 on the matrix unit (v_mfma_f64_16x16x4_f64) --------------------
  // Products of two 16-bit floats are exact in binary64 and so are their partial sums (the contract's domain), so the
  // sum does not depend on the order of the terms: a tile of 16 rows x 16 columns accumulates the D dimensions four at a
  // time.  Lane l = 16 g + c supplies A[c][g] (pooled Q row c) and B[g][c] (pooled K column c) of each step and receives
  // rows g, g + 4, g + 8, g + 12 of column c.  Step s pairs lane group g with dimension 32 (s / 8) + 8 g + (s % 8): every lane
  // then consumes the eight values of one 16-byte load in eight consecutive steps.
  {
    typedef double d4_t __attribute__((ext_vector_type(4)));
    constexpr int NL = D / 32;                    // 16-byte loads per row and lane
    const int c = lane & 15, g = lane >> 4;
    double qa[D / 4];
    {
      const bool row_ok = c < rows;
      const uint16_t *qrow = pool_q + ((size_t)bh * nq + i0 + (row_ok ? c : 0)) * D + 8 * g;
#pragma unroll
      for (int t = 0; t < NL; t++) {
        const uint4 v = row_ok ? *(const uint4 *)(qrow + 32 * t) : make_uint4(0, 0, 0, 0);
        const uint32_t w[4] = {v.x, v.y, v.z, v.w};
#pragma unroll
        for (int e = 0; e < 8; e++)
          qa[8 * t + e] = (double)elem_to_f32<DT>((uint16_t)((e & 1) ? (w[e >> 1] >> 16) : (w[e >> 1] & 0xffffu)));
      }
    }
    // columns at or beyond j_live are masked for every row of this workgroup: they get -inf without any arithmetic
    const int j_live = is_causal ? min(nk, 2 * (i0 + rows)) : nk;
    constexpr uint16_t NEG_INF = DT == 1 ? 0xff80u : 0xfc00u;
    const int n_tiles = NKP / 16, live_tiles = (j_live + 15) / 16;
    auto load_k = [&](int ct, uint4 (&raw)[NL]) __attribute__((always_inline)) {
      const int j = min(16 * ct + c, nk - 1);    // columns beyond nk re-read the last one and are masked below
      const uint16_t *krow = pk_base + (size_t)j * D + 8 * g;
#pragma unroll
      for (int t = 0; t < NL; t++) raw[t] = *(const uint4 *)(krow + 32 * t);
    };
    auto finish = [&](int ct, const d4_t &acc) __attribute__((always_inline)) {
      const int j = 16 * ct + c;
      const bool dead = j >= nk || simk[min(j, nk - 1)] == 0;
#pragma unroll
      for (int v = 0; v < 4; v++) {
        const int row = g + 4 * v;
        const float a1 = elem_to_f32<DT>(f64_to_elem_fast<DT>(acc[v]));
        uint16_t a2 = f64_to_elem_fast<DT>((double)a1 * (double)sm_scale);
        if (dead || (is_causal && j >= 2 * (i0 + row + 1))) a2 = NEG_INF;
        s_scores[(size_t)row * NKP + j] = a2;
      }
    };
    // DUAL: two column tiles per trip (two independent accumulator chains), for the long rows that leave a SIMD only two
    // wavefronts; otherwise one (128 registers per lane, four wavefronts per SIMD keep the matrix unit busy instead).
    // The next trip's pooled-K rows are in flight meanwhile.
    constexpr int STEP = DUAL ? 2 * NW : NW;
    uint4 ra[NL], rb[DUAL ? NL : 1];
    int ct = wave;
    if (ct < live_tiles) {
      load_k(ct, ra);
      if constexpr (DUAL) load_k(min(ct + NW, live_tiles - 1), rb);
    }
#pragma unroll 1
    for (; ct < live_tiles; ct += STEP) {
      uint4 ka[NL], kb[DUAL ? NL : 1];
#pragma unroll
      for (int t = 0; t < NL; t++) { ka[t] = ra[t]; if constexpr (DUAL) kb[t] = rb[t]; }
      const bool two = DUAL && ct + NW < live_tiles;         // wavefront-uniform
      if (ct + STEP < live_tiles) {
        load_k(ct + STEP, ra);
        if constexpr (DUAL) load_k(min(ct + STEP + NW, live_tiles - 1), rb);
      }
      d4_t acc_a = {0.0, 0.0, 0.0, 0.0}, acc_b = {0.0, 0.0, 0.0, 0.0};
#pragma unroll
      for (int t = 0; t < NL; t++) {
        const uint32_t wa[4] = {ka[t].x, ka[t].y, ka[t].z, ka[t].w};
#pragma unroll
        for (int e = 0; e < 8; e++) {
          const double xa = (double)elem_to_f32<DT>((uint16_t)((e & 1) ? (wa[e >> 1] >> 16) : (wa[e >> 1] & 0xffffu)));
          acc_a = __builtin_amdgcn_mfma_f64_16x16x4f64(qa[8 * t + e], xa, acc_a, 0, 0, 0);
          if constexpr (DUAL) {
            const uint32_t wb[4] = {kb[t].x, kb[t].y, kb[t].z, kb[t].w};
            const double xb = (double)elem_to_f32<DT>((uint16_t)((e & 1) ? (wb[e >> 1] >> 16) : (wb[e >> 1] & 0xffffu)));
            acc_b = __builtin_amdgcn_mfma_f64_16x16x4f64(qa[8 * t + e], xb, acc_b, 0, 0, 0);
          }
        }
      }
      finish(ct, acc_a);
      if (two) finish(ct + NW, acc_b);
    }
    // dead column tiles
    for (int t2 = live_tiles + wave; t2 < n_tiles; t2 += NW) {
      const int j = 16 * t2 + c;
#pragma unroll
      for (int v = 0; v < 4; v++) s_scores[(size_t)(g + 4 * v) * NKP + j] = NEG_INF;
    }
  }
  __syncthreads();

  // ---- phase 2: wavefront `wave` owns rows wave, wave + NW, ...; lane l holds columns l, l + 64, ... ---------------
  uint16_t *s_idx = s_idx_all + wave * NKP;
  double *s_lsum = s_lsum_all + wave * 64;
  for (int row = wave; row < rows; row += NW) {
    const int i = i0 + row;
    const int causal_lim = is_causal ? min(nk, 2 * (i + 1)) : nk;
    const uint16_t *s_score = s_scores + (size_t)row * NKP;

    float sc[EPL];
    float lmax = -INFINITY;
#pragma unroll
    for (int t = 0; t < EPL; t++) {
      sc[t] = elem_to_f32<DT>(s_score[t * 64 + lane]);   // columns >= nk were written as -inf by phase 1
      lmax = fmaxf(lmax, sc[t]);
    }
    const float mx = wave_max_f32(lmax);

    // exp and the fixed summation tree: lane l adds e[l], e[l+64], ... in order, then an xor butterfly (32 .. 1)
    double ev[EPL];
    double part = 0.0;
#pragma unroll
    for (int t = 0; t < EPL; t++) {
      ev[t] = (sc[t] == -INFINITY) ? 0.0 : cexp((double)sc[t] - (double)mx);
      part = part + ev[t];
    }
#pragma unroll
    for (int o = 32; o >= 1; o >>= 1) part = part + shfl_xor_f64(part, o);
    const double total = part;

    // probabilities -> sortable keys (value bits, then lower column first).  The 16-bit pattern of e / total is taken
    // from e * (1 / total), which is within two units in the last place of the quotient: through binary32, the two
    // agree unless the product lands exactly on a rounding tie of the 16-bit format or outside its normal range, and
    // those elements take the division and the exact conversion.
    const double rtotal = total > 0.0 ? 1.0 / total : 0.0;     // a row without a live column has e = 0 everywhere
    uint32_t okey[EPL], key[EPL];
#pragma unroll
    for (int t = 0; t < EPL; t++) {
      const int j = t * 64 + lane;
      const float pr = (float)(ev[t] * rtotal);
      const uint32_t pb = __builtin_bit_cast(uint32_t, pr);    // probabilities are non-negative
      constexpr uint32_t DROP = DT == 1 ? 16u : 13u, LOWM = (1u << DROP) - 1u, TIE = 1u << (DROP - 1u);
      constexpr uint32_t LO = DT == 1 ? 0x00800000u : 0x38800000u;     // smallest normal of the format
      const bool safe = pb == 0u || (pb >= LO && pb <= 0x3f800000u && (pb & LOWM) != TIE);
      uint32_t bits;
      if (safe) {
        bits = f32_to_elem<DT>(pr);
      } else {
        double p = ev[t] / total;
        if (!__builtin_isfinite(p)) p = 0.0;
        bits = f64_to_elem<DT>(p);
      }
      okey[t] = j < nk ? ((bits << 16) | (0xffffu - (uint32_t)j)) : 0u;
      key[t] = okey[t];
    }
    // how many to keep, and the key of the last one kept
    long long n;
    uint32_t kth = 0u;
    if (topk != nullptr) {
      const float t = topk[h] * (float)nk;            // binary32 product, truncated (utils.py:405)
      n = (long long)t;
      if (n <= 0) n = 1;                              // utils.py:289
      if (n < nk) {
        // top-k needs the n-th largest key only, not the order: build it bit by bit, the largest T with
        // #{key >= T} >= n.  Keys are distinct, probabilities are <= 1 (bits 31 and 30 of a key are clear) and
        // bits 15 .. log2(NKP) are set in every real key (they hold 0xFFFF - column).  A candidate that exactly n keys
        // reach selects the same set as the n-th largest key itself, so the search stops there.
        constexpr int LOW = 31 - __builtin_clz((unsigned)NKP);   // log2(NKP)
        uint32_t T = 0u;
        bool exact = false;                                      // wavefront-uniform
        auto try_bit = [&](int bit) {
          const uint32_t cand = T | (1u << bit);
          int cnt = 0;
#pragma unroll
          for (int tt = 0; tt < EPL; tt++) cnt += __builtin_popcountll(__ballot(okey[tt] >= cand));
          if (cnt >= (int)n) T = cand;
          exact = cnt == (int)n;
        };
#pragma unroll 1
        for (int bit = 29; bit >= 16 && !exact; bit--) try_bit(bit);
        if (!exact) {
          T |= 0xffffu & ~((1u << LOW) - 1u);
#pragma unroll 1
          for (int bit = LOW - 1; bit >= 0 && !exact; bit--) try_bit(bit);
        }
        kth = T;
      }
    } else {
      bitonic_sort_desc<EPL, 2>(key, lane);           // sorted position of key[t] is lane * EPL + t
      // cdf[v] = T(sum_{u<=v} p_sorted[u]);  n = #{v < nk : cdf[v] <= threshold}  (utils.py:398-403)
      double lsum = 0.0;
#pragma unroll
      for (int t = 0; t < EPL; t++) lsum += (double)elem_to_f32<DT>((uint16_t)(key[t] >> 16));
      s_lsum[lane] = lsum;
      __builtin_amdgcn_fence(__ATOMIC_ACQ_REL, "wavefront");
      __builtin_amdgcn_wave_barrier();
      double run = 0.0;
      for (int u = 0; u < lane; u++) run += s_lsum[u];
      const double thr = (double)cdfthr[h];
      int cnt = 0;
#pragma unroll
      for (int t = 0; t < EPL; t++) {
        run += (double)elem_to_f32<DT>((uint16_t)(key[t] >> 16));
        const float cdfv = elem_to_f32<DT>(f64_to_elem<DT>(run));
        if (lane * EPL + t < nk && (double)cdfv <= thr) cnt++;
      }
      n = wave_sum_i32(cnt);
      __builtin_amdgcn_wave_barrier();
      if (n <= 0) n = 1;                              // utils.py:289
      if (n < nk) {                                   // wavefront-uniform
        const int pos = (int)n - 1, src = pos / EPL, tt = pos % EPL;
        uint32_t mine = key[0];
#pragma unroll
        for (int t = 1; t < EPL; t++) mine = (tt == t) ? key[t] : mine;
        kth = (uint32_t)__shfl((int)mine, src, SPG_WAVE);
      }
    }

    // block map row, ascending index list, delta LUT
    const bool row_forced = sim_q[(size_t)bh * nq + i] == 0;
    const size_t row_off = ((size_t)bh * nq + i) * nk;
    int base = 0;
#pragma unroll
    for (int t = 0; t < EPL; t++) {
      const int j = t * 64 + lane;
      bool f = false;
      if (j < nk) {
        f = row_forced || (okey[t] >= kth) || (simk[j] == 0);
        if (j >= causal_lim) f = false;
        if (sink && j == 0) f = true;
        if (bmap != nullptr) bmap[row_off + j] = f ? 1 : 0;
      }
      const unsigned long long m = __ballot(f);
      const int below = __builtin_amdgcn_mbcnt_hi((uint32_t)(m >> 32), __builtin_amdgcn_mbcnt_lo((uint32_t)m, 0));
      if (f) s_idx[base + below] = (uint16_t)j;
      base += __builtin_popcountll(m);
    }
    __builtin_amdgcn_fence(__ATOMIC_ACQ_REL, "wavefront");
    __builtin_amdgcn_wave_barrier();
#pragma unroll
    for (int t = 0; t < EPL; t++) {
      const int pidx = t * 64 + lane;
      if (pidx < nk) {
        int v = 0;
        if (pidx < base) v = (int)s_idx[pidx] - (pidx ? (int)s_idx[pidx - 1] : 0);
        lut[row_off + pidx] = v;
      }
    }
    if (lane == 0) valid[(size_t)bh * nq + i] = base;
    __builtin_amdgcn_fence(__ATOMIC_ACQ_REL, "wavefront");
    __builtin_amdgcn_wave_barrier();                  // the index list is reused by this wavefront's next row
  }
}

// =============================================================================================
// user mask -> LUT
// =============================================================================================
template <int KIND>
__device__ __forceinline__ bool mask_nonzero(const void *row, int j) {
  if constexpr (KIND == 0) return ((const uint8_t *)row)[j] != 0;
  if constexpr (KIND == 1) return ((const uint16_t *)row)[j] != 0;
  if constexpr (KIND == 2) return ((const uint32_t *)row)[j] != 0;
  if constexpr (KIND == 3) return ((const uint64_t *)row)[j] != 0;
  if constexpr (KIND == 4) return (((const uint16_t *)row)[j] & 0x7fffu) != 0;            // +-0.0 is zero
  if constexpr (KIND == 5) return (((const uint32_t *)row)[j] & 0x7fffffffu) != 0;
  if constexpr (KIND == 6) return (((const uint64_t *)row)[j] & 0x7fffffffffffffffull) != 0;
  return false;
}
constexpr int mask_elem_size(int kind) { return kind == 0 ? 1 : (kind == 1 || kind == 4) ? 2 : (kind == 2 || kind == 5) ? 4 : 8; }

template <int KIND>
__global__ __launch_bounds__(256) void map_to_lut_kernel(const void *__restrict__ mask, int32_t *__restrict__ lut,
                                                         int32_t *__restrict__ valid, int nq, int nk, int nkp) {
  extern __shared__ __align__(16) unsigned char smem[];
  int32_t *s_idx = (int32_t *)smem;
  __shared__ int s_tmp[256];
  const int i = blockIdx.x, bh = blockIdx.y;
  const size_t row_off = ((size_t)bh * nq + i) * nk;
  const void *row = (const unsigned char *)mask + row_off * mask_elem_size(KIND);
  auto flag = [&](int j) -> bool { return mask_nonzero<KIND>(row, j); };
  emit_lut(flag, nk, nkp, s_idx, s_tmp, lut + row_off, valid + (size_t)bh * nq + i);
}

// =============================================================================================
// host launchers
// =============================================================================================
static int next_pow2_ge(int v, int lo) {
  int p = lo;
  while (p < v) p <<= 1;
  return p;
}

static int km_chunks(int B, int H, int N) {
  // enough workgroups to fill 256 CUs several times over, at least 256 rows each
  int want = (4096 + B * H - 1) / (B * H);
  int maxc = (N + 255) / 256;
  int c = want < maxc ? want : maxc;
  return c < 1 ? 1 : c;
}

size_t km_mean_workspace_bytes(int B, int H, int N, int D) {
  return (size_t)B * H * km_chunks(B, H, N) * D * sizeof(double);
}

template <int D, int DT>
static void launch_km(const void *k, Strides ks, void *km, void *ws, int B, int H, int N, hipStream_t st) {
  const int nchunk = km_chunks(B, H, N);
  const int rpc = (N + nchunk - 1) / nchunk;
  km_partial_kernel<D, DT><<<dim3(nchunk, B * H), 256, 0, st>>>((const uint16_t *)k, ks, H, (double *)ws, N, rpc);
  km_final_kernel<DT><<<B * H, dim3(D, 8), 0, st>>>((const double *)ws, (uint16_t *)km, nchunk, D, N);
}

void launch_km_mean(const void *k, Strides ks, void *km, void *ws, int B, int H, int N, int D, int dtype, hipStream_t st) {
  if (D == 64) { if (dtype == 0) launch_km<64, 0>(k, ks, km, ws, B, H, N, st); else launch_km<64, 1>(k, ks, km, ws, B, H, N, st); }
  else         { if (dtype == 0) launch_km<128, 0>(k, ks, km, ws, B, H, N, st); else launch_km<128, 1>(k, ks, km, ws, B, H, N, st); }
}

// ---- K column mean without a caller-provided workspace ---------------------------------------------------------
// The per-chunk partial sums go to a fixed array in device memory that the library owns (one copy per GPU, alive
// until the process ends).  In host code the array's NAME is only a handle: its device address is asked for once per
// device with hipGetSymbolAddress and that pointer is what the kernels receive.  Every call on a GPU shares the
// array, so two calls that overlap in time on one GPU (different streams or threads) race; calls on one stream are
// ordered.  Nothing needs clearing between calls: km_partial writes every partial sum km_final reads.
static __device__ __align__(256) unsigned char km_static_scratch[SPG_KM_STATIC_SCRATCH_BYTES];

size_t km_mean_static_capacity() { return SPG_KM_STATIC_SCRATCH_BYTES; }

hipError_t launch_km_mean_static(const void *k, Strides ks, void *km, int B, int H, int N, int D, int dtype, hipStream_t st) {
  constexpr int MAX_DEV = 64;
  static std::atomic<void *> scratch_of_device[MAX_DEV];
  int dev = -1;
  hipError_t e = hipGetDevice(&dev);
  if (e != hipSuccess) return e;
  if (dev < 0 || dev >= MAX_DEV) return hipErrorInvalidDevice;
  // The array's address is looked up for, and only valid on, the CURRENT device: a stream that belongs to another GPU
  // would run the kernels there with this GPU's address.  (The null stream always belongs to the current device.)
  if (st != nullptr) {
    hipDevice_t sdev = -1;
    e = hipStreamGetDevice(st, &sdev);
    if (e != hipSuccess) return e;
    if ((int)sdev != dev) return hipErrorInvalidDevice;
  }
  void *ptr = scratch_of_device[dev].load(std::memory_order_acquire);
  if (ptr == nullptr) {
    // first call on this device (the device is current): resolve this GPU's copy of the array
    e = hipGetSymbolAddress(&ptr, HIP_SYMBOL(km_static_scratch));
    if (e != hipSuccess) return e;
    if (ptr == nullptr) return hipErrorInvalidSymbol;
    scratch_of_device[dev].store(ptr, std::memory_order_release);
  }
  launch_km_mean(k, ks, km, ptr, B, H, N, D, dtype, st);
  return hipSuccess;
}

template <int BS, int D, int DT>
static void launch_psq3(const void *x, Strides xs, const void *km, void *pool, uint8_t *sim, int8_t *xq, float *scale,
                        const float *thr, int B, int H, int N, int quant_rows, hipStream_t st) {
  const int nb = (N + BS - 1) / BS;
  const dim3 grid((N + 127) / 128, B * H);      // one workgroup per 128 rows: one or two blocks
  const uint16_t *xp = (const uint16_t *)x, *kp = (const uint16_t *)km;
  uint16_t *pp = (uint16_t *)pool;
  if constexpr (BS == 128) {
    if (quant_rows == 32) {                     // per-warp granularity of Q (no mean: the C ABI refuses the combination)
      if (pool != nullptr) pool_sim_quant_kernel<BS, D, DT, false, true, 32><<<grid, 256, 0, st>>>(xp, xs, kp, pp, sim, xq, scale, thr, H, N, nb);
      else                 pool_sim_quant_kernel<BS, D, DT, false, false, 32><<<grid, 256, 0, st>>>(xp, xs, kp, pp, sim, xq, scale, thr, H, N, nb);
      return;
    }
  }
  if (pool != nullptr) {
    if (km) pool_sim_quant_kernel<BS, D, DT, true, true><<<grid, 256, 0, st>>>(xp, xs, kp, pp, sim, xq, scale, thr, H, N, nb);
    else    pool_sim_quant_kernel<BS, D, DT, false, true><<<grid, 256, 0, st>>>(xp, xs, kp, pp, sim, xq, scale, thr, H, N, nb);
  } else {
    if (km) pool_sim_quant_kernel<BS, D, DT, true, false><<<grid, 256, 0, st>>>(xp, xs, kp, pp, sim, xq, scale, thr, H, N, nb);
    else    pool_sim_quant_kernel<BS, D, DT, false, false><<<grid, 256, 0, st>>>(xp, xs, kp, pp, sim, xq, scale, thr, H, N, nb);
  }
}

void launch_pool_sim_quant(const void *x, Strides xs, const void *km, void *pool, uint8_t *sim, int8_t *xq, float *scale,
                           const float *thr, int B, int H, int N, int D, int block, int quant_rows, int dtype,
                           hipStream_t st) {
#define SPG_PSQ(BS_, D_, DT_) launch_psq3<BS_, D_, DT_>(x, xs, km, pool, sim, xq, scale, thr, B, H, N, quant_rows, st)
  if (block == 128) {
    if (D == 64) { if (dtype == 0) SPG_PSQ(128, 64, 0); else SPG_PSQ(128, 64, 1); }
    else         { if (dtype == 0) SPG_PSQ(128, 128, 0); else SPG_PSQ(128, 128, 1); }
  } else {
    if (D == 64) { if (dtype == 0) SPG_PSQ(64, 64, 0); else SPG_PSQ(64, 64, 1); }
    else         { if (dtype == 0) SPG_PSQ(64, 128, 0); else SPG_PSQ(64, 128, 1); }
  }
#undef SPG_PSQ
}

int block_select_max_nk() { return 8192; }

// Kernels that need more than 48 KiB of dynamic LDS must be told so once (per device); the size granted last is
// remembered per kernel and device, so the attribute call is not repeated on every launch.  gfx950 has 160 KiB of LDS
// per workgroup; a request beyond it (including the kernel's static arrays, at most 4 KiB here) is refused up front.
template <auto Kern>
static hipError_t allow_dynamic_lds(size_t lds) {
  if (lds + 4096 > 160 * 1024) return hipErrorInvalidConfiguration;
  if (lds <= 48 * 1024) return hipSuccess;
  static std::atomic<size_t> granted[32];
  int dev = 0;
  hipError_t e = hipGetDevice(&dev);
  if (e != hipSuccess) return e;
  const bool tracked = dev >= 0 && dev < 32;
  if (tracked && granted[dev].load(std::memory_order_relaxed) >= lds) return hipSuccess;
  e = hipFuncSetAttribute((const void *)Kern, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
  if (e == hipSuccess && tracked) granted[dev].store(lds, std::memory_order_relaxed);
  return e;
}

void launch_div_selftest(unsigned long long *counts, int n_div, uint32_t seed, hipStream_t st) {
  div_selftest_kernel<<<(n_div + 255) / 256, 256, 0, st>>>(counts, n_div, seed);
}

template <int D, int DT, int R>
static hipError_t launch_bs3(const void *pq, const uint8_t *sq, const void *pk, const uint8_t *sk, const float *topk,
                             const float *cdf, int causal, int sink, int32_t *lut, int32_t *valid, uint8_t *bmap, int B,
                             int H, int Hkv, int nq, int nk, int nkp, hipStream_t st) {
  const size_t lds = (size_t)R * D * 8 + (size_t)R * nkp * 4 + 12 * (size_t)nkp;
  auto kern = block_select_kernel<D, DT, R>;
  {
    hipError_t e = allow_dynamic_lds<block_select_kernel<D, DT, R>>(lds);
    if (e != hipSuccess) return e;
  }
  kern<<<dim3((nq + R - 1) / R, B * H), 256, lds, st>>>((const uint16_t *)pq, sq, (const uint16_t *)pk, sk, topk, cdf,
                                                        causal, sink, lut, valid, bmap, H, Hkv, nq, nk, nkp);
  return hipSuccess;
}

template <int D, int DT>
static hipError_t launch_bs2(const void *pq, const uint8_t *sq, const void *pk, const uint8_t *sk, const float *topk,
                             const float *cdf, int causal, int sink, int32_t *lut, int32_t *valid, uint8_t *bmap, int B,
                             int H, int Hkv, int nq, int nk, hipStream_t st) {
  const int nkp = next_pow2_ge(nk, 256);
  if (nkp <= 2048) {
    // a whole row fits the registers of one wavefront
#define SPG_BSW(NW_, EPL_, DUAL_)                                                                                    \
    {                                                                                                           \
      const size_t lds = (size_t)16 * nkp * 2 + (size_t)NW_ * nkp * 2 + NW_ * 64 * 8;                           \
      auto kern = block_select_wave_kernel<D, DT, NW_, EPL_, DUAL_>;                                                   \
      {                                                                                                         \
        hipError_t e = allow_dynamic_lds<block_select_wave_kernel<D, DT, NW_, EPL_, DUAL_>>(lds);                      \
        if (e != hipSuccess) return e;                                                                          \
      }                                                                                                         \
      kern<<<dim3((nq + 15) / 16, B * H), 64 * NW_, lds, st>>>((const uint16_t *)pq, sq, (const uint16_t *)pk, sk, topk, \
                                                               cdf, causal, sink, lut, valid, bmap, H, Hkv, nq, nk); \
      return hipSuccess;                                                                                        \
    }
    // one wavefront per row (16 per workgroup) where a row's registers fit the 128 a 1024-thread workgroup leaves each
    // lane, two rows per wavefront beyond
    if (nkp == 256) SPG_BSW(8, 4, false)
    if (nkp == 512) SPG_BSW(8, 8, false)
    if (nkp == 1024) SPG_BSW(8, 16, false)
    SPG_BSW(8, 32, true)
#undef SPG_BSW
  }
  // rows per workgroup: reuse of the pooled-K reads against LDS footprint (scores are R*nkp floats)
  if (nkp <= 1024) return launch_bs3<D, DT, 8>(pq, sq, pk, sk, topk, cdf, causal, sink, lut, valid, bmap, B, H, Hkv, nq, nk, nkp, st);
  if (nkp <= 4096) return launch_bs3<D, DT, 4>(pq, sq, pk, sk, topk, cdf, causal, sink, lut, valid, bmap, B, H, Hkv, nq, nk, nkp, st);
  // nkp = 8192: one row per workgroup (D*8 + 16*nkp = 129 KiB; two rows would need 162 KiB, more than the 160 KiB a
  // workgroup can have)
  return launch_bs3<D, DT, 1>(pq, sq, pk, sk, topk, cdf, causal, sink, lut, valid, bmap, B, H, Hkv, nq, nk, nkp, st);
}

hipError_t launch_block_select(const void *pq, const uint8_t *sq, const void *pk, const uint8_t *sk, const float *topk,
                               const float *cdf, int causal, int sink, int32_t *lut, int32_t *valid, uint8_t *bmap,
                               int B, int H, int Hkv, int nq, int nk, int D, int dtype, hipStream_t st) {
#define SPG_BS(D_, DT_) return launch_bs2<D_, DT_>(pq, sq, pk, sk, topk, cdf, causal, sink, lut, valid, bmap, B, H, Hkv, nq, nk, st)
  if (D == 64) { if (dtype == 0) SPG_BS(64, 0); else SPG_BS(64, 1); }
  else         { if (dtype == 0) SPG_BS(128, 0); else SPG_BS(128, 1); }
#undef SPG_BS
}

hipError_t launch_map_to_lut(const void *mask, int kind, int32_t *lut, int32_t *valid, int B, int H, int nq, int nk,
                             hipStream_t st) {
  const int nkp = next_pow2_ge(nk, 256);
  const size_t lds = 4 * (size_t)nkp;
  const dim3 grid(nq, B * H);
#define SPG_M2L(K_)                                                                                      \
  case K_: {                                                                                             \
    auto kern = map_to_lut_kernel<K_>;                                                                   \
    {                                                                                                    \
      hipError_t e = allow_dynamic_lds<map_to_lut_kernel<K_>>(lds);                                      \
      if (e != hipSuccess) return e;                                                                     \
    }                                                                                                    \
    kern<<<grid, 256, lds, st>>>(mask, lut, valid, nq, nk, nkp);                                         \
    break;                                                                                               \
  }
  switch (kind) {
    SPG_M2L(0) SPG_M2L(1) SPG_M2L(2) SPG_M2L(3) SPG_M2L(4) SPG_M2L(5) SPG_M2L(6)
    default: return hipErrorInvalidValue;
  }
#undef SPG_M2L
  return hipSuccess;
}

}  // namespace spg
