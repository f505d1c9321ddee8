// Dense FP16 flash attention on gfx950 MFMA: the comparator the sparse path's speed-up is quoted against.
// Same skeleton as attn.hip (transposed products, one query column per lane, double-buffered LDS tiles, XCD-aware
// workgroup order) with v_mfma_f32_32x32x16_f16 for both products and fp16 P.  Not part of the reference.
#include "common.h"
#include "launch.h"

namespace spg {

typedef _Float16 v8h __attribute__((ext_vector_type(8)));
typedef float v16f __attribute__((ext_vector_type(16)));

struct DenseParams {
  const uint16_t *q, *k, *vt;
  uint16_t *out;
  int B, H, N, nq, nk;
  float sm_scale_log2;
  int is_causal;
  int total_wg, wg_per_xcd;
};

template <int D>
__global__ __launch_bounds__(256, 2) void dense_attn_f16_kernel(const DenseParams p) {
  constexpr int KS = D / 16;          // k-steps of QK^T
  constexpr int NDT = D / 32;         // output channel tiles
  constexpr int KSTR = D * 2 + 16;    // bytes per K row in LDS
  constexpr int VSTR = 64 * 2 + 16;   // bytes per V^T row in LDS
  constexpr int CH = D / 32;          // 16-byte chunks per thread per tile (64*D*2/16/256)
  extern __shared__ __align__(16) unsigned char smem[];
  auto sKp = [&](int b) -> unsigned char * { return smem + b * (64 * KSTR); };
  auto sVp = [&](int b) -> unsigned char * { return smem + 2 * 64 * KSTR + b * (D * VSTR); };

  const int w = blockIdx.x;
  const int L = (w & 7) * p.wg_per_xcd + (w >> 3);
  if (L >= p.total_wg) return;
  const int bh = L / p.nq;
  const int qb = p.nq - 1 - (L % p.nq);
  const int tid = threadIdx.x, wave = tid >> 6, lane = tid & 63, r = lane & 31, hh = lane >> 5;
  const int N = p.N;
  const int q_row = qb * 128 + wave * 32 + r;
  const int nblk = p.is_causal ? min(p.nk, 2 * (qb + 1)) : p.nk;

  v8h qreg[KS];
#pragma unroll
  for (int ks = 0; ks < KS; ks++) {
    uint4 t = make_uint4(0, 0, 0, 0);
    if (q_row < N) t = *(const uint4 *)(p.q + ((size_t)bh * N + q_row) * D + 16 * ks + 8 * hh);
    qreg[ks] = __builtin_bit_cast(v8h, t);
  }
  const uint16_t *kbase = p.k + (size_t)bh * N * D;
  const uint16_t *vbase = p.vt + (size_t)bh * p.nk * (size_t)(D * 64);
  const float c = p.sm_scale_log2;

  // staging registers for the next block's tiles (named scalars: an indexed array ends up in scratch memory)
  uint4 kr0, kr1, kr2, kr3, vr0, vr1, vr2, vr3;
  kr0 = kr1 = kr2 = kr3 = vr0 = vr1 = vr2 = vr3 = make_uint4(0, 0, 0, 0);
#define SPG_FETCH1(U, KR, VR, BLK)                                                                       \
  if constexpr (CH > U) {                                                                                \
    const int ci = tid + 256 * U;                                                                        \
    const int row = ci / (D / 8), col = ci % (D / 8);                                                    \
    /* rows beyond N (last block only) are clamped to a valid row: their scores are masked below */      \
    const int grow = min((BLK) * 64 + row, N - 1);                                                       \
    KR = *(const uint4 *)(kbase + (size_t)grow * D + col * 8);                                           \
    VR = *(const uint4 *)(vbase + (size_t)(BLK) * (D * 64) + (size_t)ci * 8);                            \
  }
#define SPG_FETCH(BLK)                                                                                   \
  { SPG_FETCH1(0, kr0, vr0, BLK) SPG_FETCH1(1, kr1, vr1, BLK) SPG_FETCH1(2, kr2, vr2, BLK) SPG_FETCH1(3, kr3, vr3, BLK) }
#define SPG_STASH1(U, KR, VR, BUF)                                                                       \
  if constexpr (CH > U) {                                                                                \
    const int ci = tid + 256 * U;                                                                        \
    *(uint4 *)(sKp(BUF) + (ci / (D / 8)) * KSTR + (ci % (D / 8)) * 16) = KR;                             \
    *(uint4 *)(sVp(BUF) + (ci >> 3) * VSTR + (ci & 7) * 16) = VR;                                        \
  }
#define SPG_STASH(BUF)                                                                                   \
  { SPG_STASH1(0, kr0, vr0, BUF) SPG_STASH1(1, kr1, vr1, BUF) SPG_STASH1(2, kr2, vr2, BUF) SPG_STASH1(3, kr3, vr3, BUF) }

  // MFMA row i of key tile kt carries key 32*kt + 16*(i>>4) + 8*((i>>2)&1) + 4*((i>>3)&1) + (i&3):
  // after S^T, the 8 registers [8n', 8n'+8) of a lane hold 8 consecutive keys 16*(2kt+n') + 8*half + (0..7).
  const int krow0 = 16 * (r >> 4) + 8 * ((r >> 2) & 1) + 4 * ((r >> 3) & 1) + (r & 3);

  float m = -INFINITY, dsum = 0.f;
  v16f O[NDT];
#pragma unroll
  for (int dt = 0; dt < NDT; dt++)
#pragma unroll
    for (int e = 0; e < 16; e++) O[dt][e] = 0.f;

  SPG_FETCH(0);
  SPG_STASH(0);
  int buf = 0;
  for (int blk = 0; blk < nblk; blk++) {
    __syncthreads();
    v16f S[2];
#pragma unroll
    for (int e = 0; e < 16; e++) { S[0][e] = 0.f; S[1][e] = 0.f; }
#pragma unroll
    for (int ks = 0; ks < KS; ks++) {
#pragma unroll
      for (int kt = 0; kt < 2; kt++) {
        const uint4 t = *(const uint4 *)(sKp(buf) + (krow0 + 32 * kt) * KSTR + (16 * ks + 8 * hh) * 2);
        S[kt] = __builtin_amdgcn_mfma_f32_32x32x16_f16(__builtin_bit_cast(v8h, t), qreg[ks], S[kt], 0, 0, 0);
      }
    }
    const bool more = blk + 1 < nblk;
    SPG_FETCH(more ? blk + 1 : blk);   // unconditional: keeps the staging registers out of scratch

    // register e of tile kt <-> key 64*blk + 32*kt + 16*(e>>3) + 8*hh + (e&7)
    const bool edge = (p.is_causal && blk >= 2 * qb) || (blk == p.nk - 1);
    float fm = -INFINITY;
#pragma unroll
    for (int kt = 0; kt < 2; kt++)
#pragma unroll
      for (int e = 0; e < 16; e++) {
        float v = S[kt][e];
        if (edge) {
          const int key = 64 * blk + 32 * kt + 16 * (e >> 3) + 8 * hh + (e & 7);
          if (key >= N || (p.is_causal && key > q_row)) v = -INFINITY;
          S[kt][e] = v;
        }
        fm = fmaxf(fm, v);
      }
    fm = half_swap_max_f32(fm) * c;
    const float m_new = fmaxf(m, fm);
    const float m_use = (m_new == -INFINITY) ? 0.f : m_new;
    const float osc = __builtin_amdgcn_exp2f(m - m_use);
    m = m_new;
    dsum *= osc;
    if (__any(osc != 1.0f)) {
#pragma unroll
      for (int dt = 0; dt < NDT; dt++)
#pragma unroll
        for (int e = 0; e < 16; e++) O[dt][e] *= osc;
    }
    v8h pb[4];
    float ps = 0.f;
#pragma unroll
    for (int kt = 0; kt < 2; kt++)
#pragma unroll
      for (int e = 0; e < 16; e += 2) {
        const float p0 = __builtin_amdgcn_exp2f(__builtin_fmaf(S[kt][e], c, -m_use));
        const float p1 = __builtin_amdgcn_exp2f(__builtin_fmaf(S[kt][e + 1], c, -m_use));
        ps += p0 + p1;
        const auto h2 = __builtin_amdgcn_cvt_pkrtz(p0, p1);      // two fp16 in one instruction
        pb[2 * kt + (e >> 3)][e & 7] = (_Float16)h2[0];
        pb[2 * kt + (e >> 3)][(e & 7) + 1] = (_Float16)h2[1];
      }
    dsum += ps;
#pragma unroll
    for (int n = 0; n < 4; n++) {
#pragma unroll
      for (int dt = 0; dt < NDT; dt++) {
        const uint4 t = *(const uint4 *)(sVp(buf) + (32 * dt + r) * VSTR + (16 * n + 8 * hh) * 2);
        O[dt] = __builtin_amdgcn_mfma_f32_32x32x16_f16(__builtin_bit_cast(v8h, t), pb[n], O[dt], 0, 0, 0);
      }
    }
    SPG_STASH(buf ^ 1);                // buf^1 was last read before this iteration's barrier
    buf ^= 1;
  }

#undef SPG_FETCH
#undef SPG_STASH
#undef SPG_FETCH1
#undef SPG_STASH1
  const float dtot = half_swap_sum_f32(dsum);
  const float inv = 1.0f / dtot;
  if (q_row < N) {
    uint16_t *orow = p.out + ((size_t)bh * N + q_row) * D;
#pragma unroll
    for (int dt = 0; dt < NDT; dt++)
#pragma unroll
      for (int g = 0; g < 4; g++) {
        const int d0 = 32 * dt + 8 * g + 4 * hh;
        const uint16_t o0 = f32_to_elem<0>(O[dt][4 * g + 0] * inv);
        const uint16_t o1 = f32_to_elem<0>(O[dt][4 * g + 1] * inv);
        const uint16_t o2 = f32_to_elem<0>(O[dt][4 * g + 2] * inv);
        const uint16_t o3 = f32_to_elem<0>(O[dt][4 * g + 3] * inv);
        *(uint2 *)(orow + d0) = make_uint2((uint32_t)o0 | ((uint32_t)o1 << 16), (uint32_t)o2 | ((uint32_t)o3 << 16));
      }
  }
}

template <int D>
static hipError_t launch_dense(const DenseParams &p, hipStream_t st) {
  constexpr size_t lds = 2 * 64 * (D * 2 + 16) + 2 * D * (64 * 2 + 16);
  auto kern = dense_attn_f16_kernel<D>;
  if (lds > 48 * 1024) {
    hipError_t e = hipFuncSetAttribute((const void *)kern, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
    if (e != hipSuccess) return e;
  }
  kern<<<p.wg_per_xcd * 8, 256, lds, st>>>(p);
  return hipGetLastError();
}

hipError_t launch_dense_attn_f16(const void *q, const void *k, const void *vt, void *out, int B, int H, int N, int D,
                                 float sm_scale, int is_causal, hipStream_t st) {
  DenseParams p;
  p.q = (const uint16_t *)q; p.k = (const uint16_t *)k; p.vt = (const uint16_t *)vt; p.out = (uint16_t *)out;
  p.B = B; p.H = H; p.N = N; p.nq = (N + 127) / 128; p.nk = (N + 63) / 64;
  p.sm_scale_log2 = sm_scale * 1.44269504088896340736f;
  p.is_causal = is_causal;
  p.total_wg = p.nq * H * B;
  p.wg_per_xcd = (p.total_wg + 7) / 8;
  return D == 64 ? launch_dense<64>(p, st) : launch_dense<128>(p, st);
}

}  // namespace spg
