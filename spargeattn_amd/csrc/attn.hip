// Block-sparse INT8-QK / FP8-PV attention for gfx950 (CDNA4), written for 64-lane wavefronts and MFMA.
//
// Replaces qk_int_sv_f8_block_sparse_attn_kernel (csrc/qattn/qk_int_sv_f8_cuda_sm89.cuh:42-755) as launched by
// qk_int8_sv_f8_accum_f32_block_sparse_attn_inst_buf_fuse_v_scale_with_pv_threshold
// (csrc/qattn/qk_int_sv_f8_cuda_sm89.cu:197-390): per-block INT8 scales, per-block PV threshold, fp32 PV
// accumulation, V scale fused into the epilogue.
//
// Design (not a translation of the mma.sync tiling):
//  * one workgroup = one 128-row Q block = 4 wavefronts x 32 queries;
//  * both products are computed TRANSPOSED so that a lane owns one query column throughout:
//        S^T (64 keys x 32 queries) = K . Q^T   v_mfma_i32_32x32x32_i8     (A = K rows from LDS, B = Q in VGPRs)
//        O^T (D x 32 queries)      += V^T . P^T v_mfma_f32_32x32x64_f8f6f4 (A = V^T rows from LDS, B = P in VGPRs)
//    lane l holds query l%32; lanes l and l^32 hold the two halves of that query's keys / output channels.
//    Row max / row sum are lane-local plus ONE cross-lane exchange; the O rescale is lane-local.
//  * the K rows are assigned to MFMA rows through a permutation chosen such that, after S^T is computed, the
//    32 scores a lane holds belong to 32 CONSECUTIVE keys (32*half .. 32*half+31): packing them to e4m3 gives the
//    B operand of the PV MFMA with no shuffle, and the matching A operand is 32 contiguous bytes of a V^T row;
//  * V lives in HBM as [nk][D][64] e4m3 tiles (one contiguous 64*D-byte read per block), K as (N,D) int8 rows;
//  * K/V tiles go through a 3-deep LDS ring: the tiles of block it+2 are in flight from HBM/L2 into VGPRs and the
//    tiles of block it+1 are written to LDS while block it is being computed, so that ONE workgroup barrier per
//    block covers both the tile hand-over and the workgroup-wide PV-skip vote;
//  * workgroup ids are remapped so that one XCD (one L2) works on one head at a time, heaviest rows first.
#include "common.h"
#include "launch.h"

namespace spg {

typedef int v4i __attribute__((ext_vector_type(4)));
typedef int v8i __attribute__((ext_vector_type(8)));
typedef int v16i __attribute__((ext_vector_type(16)));
typedef float v16f __attribute__((ext_vector_type(16)));

#define SPG_NEG_BIG (-5000000.0f)   // csrc/qattn/attn_utils.cuh:350, qk_int_sv_f8_cuda_sm89.cuh:171
#define SPG_FP8_OFFSET 8.807f       // csrc/qattn/attn_utils.cuh:28
#define SPG_LOG2E 1.44269504088896340736f

struct AttnParams {
  const int8_t *q8, *k8;
  const uint8_t *v8;
  void *out;
  const int32_t *lut, *valid;
  const float *pvthr, *q_scale, *k_scale, *v_scale;
  int32_t *pv_count;
  int B, H, N, nq, nk;
  float sm_scale_log2;
  int is_causal;
  int total_wg, wg_per_xcd;
};

template <int D, int ODT>
__global__ __launch_bounds__(256, 2) void block_sparse_attn_kernel(const AttnParams p) {
  constexpr int KS = D / 32;        // k-steps of the int8 MFMA
  constexpr int NDT = D / 32;       // 32-channel output tiles
  constexpr int KSTR = D + 16;      // LDS row stride of a K tile (bytes)
  constexpr int VSTR = 64 + 16;     // LDS row stride of a V^T tile (bytes)
  constexpr int CH = D / 64;        // 16-byte chunks per thread per tile (K: 64*D/16/256, V: D*64/16/256)
  constexpr int NBUF = 3;
  __shared__ __align__(16) int8_t sK[NBUF][64 * KSTR];
  __shared__ __align__(16) uint8_t sV[NBUF][D * VSTR];
  __shared__ float sRed[2][4];

  // ---- workgroup -> (batch*head, q block): one XCD per head at a time, heavy (late) rows first ----------
  const int w = blockIdx.x;
  const int L = (w & 7) * p.wg_per_xcd + (w >> 3);
  if (L >= p.total_wg) return;
  const int bh = L / p.nq;
  const int qb = p.nq - 1 - (L % p.nq);
  const int head = bh % p.H;
  const int nv = p.valid[(size_t)bh * p.nq + qb];
  if (nv == 0) return;                                       // output rows stay unwritten (sm89.cuh:232-235)
  const int32_t *lut_row = p.lut + ((size_t)bh * p.nq + qb) * p.nk;

  const int tid = threadIdx.x, wave = tid >> 6, lane = tid & 63, r = lane & 31, hh = lane >> 5;
  const int N = p.N;
  const int q_row = qb * 128 + wave * 32 + r;

  // ---- Q fragment: B operand of S^T = K.Q^T, resident for the whole loop -------------------------------
  v4i qreg[KS];
#pragma unroll
  for (int ks = 0; ks < KS; ks++) {
    qreg[ks] = (v4i){0, 0, 0, 0};
    if (q_row < N) qreg[ks] = *(const v4i *)(p.q8 + ((size_t)bh * N + q_row) * D + 32 * ks + 16 * hh);
  }

  const int8_t *kbase = p.k8 + (size_t)bh * N * D;
  const uint8_t *vbase = p.v8 + (size_t)bh * p.nk * (size_t)(D * 64);
  const float *kscale = p.k_scale + (size_t)bh * p.nk;
  const float qs = p.q_scale[(size_t)bh * p.nq + qb];
  const float c = p.sm_scale_log2;
  const float thr = p.pvthr[head];

  // per-thread 16-byte chunks of a tile: chunk ci = tid + 256*u
  uint4 kr[CH], vr[CH];
  int krow[CH], kcol[CH];
#pragma unroll
  for (int u = 0; u < CH; u++) {
    const int ci = tid + 256 * u;
    krow[u] = ci / (D / 16);
    kcol[u] = (ci % (D / 16)) * 16;
  }
#define SPG_FETCH(BLK)                                                                                    \
  {                                                                                                       \
    _Pragma("unroll") for (int u = 0; u < CH; u++) {                                                      \
      const int grow = (BLK) * 64 + krow[u];                                                              \
      const int crow = min(grow, N - 1); /* rows beyond N: read a valid row, then zero it */              \
      uint4 t = *(const uint4 *)(kbase + (size_t)crow * D + kcol[u]);                                     \
      const uint32_t keep = grow < N ? 0xffffffffu : 0u;                                                  \
      kr[u] = make_uint4(t.x & keep, t.y & keep, t.z & keep, t.w & keep);                                 \
      vr[u] = *(const uint4 *)(vbase + (size_t)(BLK) * (D * 64) + (size_t)(tid + 256 * u) * 16);          \
    }                                                                                                     \
  }
#define SPG_STASH(BUF)                                                                                    \
  {                                                                                                       \
    _Pragma("unroll") for (int u = 0; u < CH; u++) {                                                      \
      const int ci = tid + 256 * u;                                                                       \
      *(uint4 *)(sK[BUF] + krow[u] * KSTR + kcol[u]) = kr[u];                                             \
      *(uint4 *)(sV[BUF] + (ci >> 2) * VSTR + (ci & 3) * 16) = vr[u];                                     \
    }                                                                                                     \
  }

  // MFMA row i of key tile kt carries key 32*((i>>2)&1) + 16*kt + 4*(i>>3) + (i&3)
  const int krow0 = 32 * ((r >> 2) & 1) + 4 * (r >> 3) + (r & 3);

  float m = SPG_NEG_BIG;
  float dsum = hh == 0 ? 1.0f : 0.0f;     // the two half-lanes of a query share d = 1.0 (sm89.cuh:172)
  v16f O[NDT];
#pragma unroll
  for (int dt = 0; dt < NDT; dt++)
#pragma unroll
    for (int e = 0; e < 16; e++) O[dt][e] = 0.f;
  int cnt = 0;

  int blk = lut_row[0];        // block computed in the current iteration
  SPG_FETCH(blk);
  SPG_STASH(0);
  int blk_next = blk;          // block whose tiles sit in kr/vr
  if (nv > 1) {
    blk_next = blk + lut_row[1];
    SPG_FETCH(blk_next);
  }
  __syncthreads();
  int buf = 0;

  for (int it = 0; it < nv; it++) {
    // ---- S^T = K . Q^T ---------------------------------------------------------------------------------
    v16i S0, S1;
#pragma unroll
    for (int e = 0; e < 16; e++) { S0[e] = 0; S1[e] = 0; }
#pragma unroll
    for (int ks = 0; ks < KS; ks++) {
      const v4i a0 = *(const v4i *)(sK[buf] + krow0 * KSTR + 32 * ks + 16 * hh);
      const v4i a1 = *(const v4i *)(sK[buf] + (krow0 + 16) * KSTR + 32 * ks + 16 * hh);
      S0 = __builtin_amdgcn_mfma_i32_32x32x32_i8(a0, qreg[ks], S0, 0, 0, 0);
      S1 = __builtin_amdgcn_mfma_i32_32x32x32_i8(a1, qreg[ks], S1, 0, 0, 0);
    }

    // ---- ring: tiles of block it+1 (in VGPRs since the previous iteration) -> LDS; fetch block it+2 -------
    const int cur = blk;
    const int nbuf = buf == NBUF - 1 ? 0 : buf + 1;
    if (it + 1 < nv) {
      SPG_STASH(nbuf);
      blk = blk_next;
      if (it + 2 < nv) {
        blk_next = blk + lut_row[it + 2];
        SPG_FETCH(blk_next);
      }
    }

    const float dq = qs * kscale[cur];
    const bool tail = it >= nv - 2;   // last two blocks: masks, no PV skip (sm89.cuh:467-648)
    float x[32];
    float a, fm;
    if (!tail) {
      int imax = S0[0];
#pragma unroll
      for (int e = 1; e < 16; e++) imax = max(imax, S0[e]);
#pragma unroll
      for (int e = 0; e < 16; e++) imax = max(imax, S1[e]);
#pragma unroll
      for (int e = 0; e < 16; e++) { x[e] = (float)S0[e]; x[16 + e] = (float)S1[e]; }
      a = c * dq;
      fm = (float)imax * a;
    } else {
      // slot e of this lane is key 64*cur + 32*hh + e; keys beyond `lim` are masked
      const int key0 = cur * 64 + 32 * hh;
      int lim = 0x7fffffff;
      if (p.is_causal) lim = q_row - key0;                       // key > query (attn_utils.cuh:334-361)
      if (it == nv - 1) lim = min(lim, N - 1 - key0);            // key >= kv_len (attn_utils.cuh:363-389)
      fm = SPG_NEG_BIG;
#pragma unroll
      for (int e = 0; e < 32; e++) {
        float v = (float)(e < 16 ? S0[e] : S1[e - 16]) * dq;
        v = e > lim ? SPG_NEG_BIG : v;
        x[e] = v;
        fm = fmaxf(fm, v);
      }
      a = c;
      fm = fm * c;
    }
    fm = fmaxf(fm, __shfl_xor(fm, 32, SPG_WAVE));
    const float diff = fm - m;
    const float m_new = fmaxf(m, fm);
    const float osc = __builtin_amdgcn_exp2f(m - m_new);
    m = m_new;
    if (!tail) {
      const float wd = wave_max_f32(diff);
      if (lane == 0) sRed[it & 1][wave] = wd;
    }
    __syncthreads();   // block it+1's tiles are in LDS; sRed is visible; ring slot of block it-1 is free
    bool compute = true;
    if (!tail) {
      const float wg = fmaxf(fmaxf(sRed[it & 1][0], sRed[it & 1][1]), fmaxf(sRed[it & 1][2], sRed[it & 1][3]));
      compute = (wg + thr > 0.f);     // workgroup-uniform (PVThresholdMode::kPerBlock, sm89.cuh:318-353)
    }
    dsum *= osc;
    if (__any(osc != 1.0f)) {
#pragma unroll
      for (int dt = 0; dt < NDT; dt++)
#pragma unroll
        for (int e = 0; e < 16; e++) O[dt][e] *= osc;
    }
    if (compute) {
      cnt++;
      const float neg = -m + SPG_FP8_OFFSET;
      float ps = 0.f;
#pragma unroll
      for (int e = 0; e < 32; e++) {
        x[e] = __builtin_amdgcn_exp2f(__builtin_fmaf(x[e], a, neg));
        ps += x[e];
      }
      dsum += ps;
      v8i pb;
#pragma unroll
      for (int u = 0; u < 8; u++) {
        int wv = __builtin_amdgcn_cvt_pk_fp8_f32(x[4 * u], x[4 * u + 1], 0, false);
        wv = __builtin_amdgcn_cvt_pk_fp8_f32(x[4 * u + 2], x[4 * u + 3], wv, true);
        pb[u] = wv;
      }
#pragma unroll
      for (int dt = 0; dt < NDT; dt++) {
        const uint8_t *vrow = sV[buf] + (32 * dt + r) * VSTR + 32 * hh;
        const v4i lo = *(const v4i *)(vrow);
        const v4i hi = *(const v4i *)(vrow + 16);
        const v8i av = {lo[0], lo[1], lo[2], lo[3], hi[0], hi[1], hi[2], hi[3]};
        O[dt] = __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(av, pb, O[dt], 0, 0, 0, 0, 0, 0);
      }
    }
    buf = nbuf;
  }
#undef SPG_FETCH
#undef SPG_STASH

  if (p.pv_count != nullptr && tid == 0) p.pv_count[(size_t)bh * p.nq + qb] = cnt;

  // ---- epilogue: O / d * v_scale -> out dtype -----------------------------------------------------------
  const float dtot = dsum + __shfl_xor(dsum, 32, SPG_WAVE);
  const float inv = __builtin_amdgcn_rcpf(dtot);
  if (q_row < N) {
    uint16_t *orow = (uint16_t *)p.out + ((size_t)bh * N + q_row) * D;
    const float *vs = p.v_scale + (size_t)bh * D;
#pragma unroll
    for (int dt = 0; dt < NDT; dt++) {
#pragma unroll
      for (int g = 0; g < 4; g++) {
        const int d0 = 32 * dt + 8 * g + 4 * hh;
        const float4 sc = *(const float4 *)(vs + d0);
        const uint16_t o0 = f32_to_elem<ODT>(O[dt][4 * g + 0] * inv * sc.x);
        const uint16_t o1 = f32_to_elem<ODT>(O[dt][4 * g + 1] * inv * sc.y);
        const uint16_t o2 = f32_to_elem<ODT>(O[dt][4 * g + 2] * inv * sc.z);
        const uint16_t o3 = f32_to_elem<ODT>(O[dt][4 * g + 3] * inv * sc.w);
        *(uint2 *)(orow + d0) = make_uint2((uint32_t)o0 | ((uint32_t)o1 << 16), (uint32_t)o2 | ((uint32_t)o3 << 16));
      }
    }
  }
}

hipError_t launch_block_sparse_attn(const int8_t *q8, const int8_t *k8, const uint8_t *v8, void *out, int out_dtype,
                                    const int32_t *lut, const int32_t *valid, const float *pvthreshd,
                                    const float *q_scale, const float *k_scale, const float *v_scale, int B, int H,
                                    int N, int D, float sm_scale, int is_causal, int32_t *pv_count, hipStream_t st) {
  AttnParams p;
  p.q8 = q8; p.k8 = k8; p.v8 = v8; p.out = out; p.lut = lut; p.valid = valid; p.pvthr = pvthreshd;
  p.q_scale = q_scale; p.k_scale = k_scale; p.v_scale = v_scale; p.pv_count = pv_count;
  p.B = B; p.H = H; p.N = N; p.nq = (N + 127) / 128; p.nk = (N + 63) / 64;
  p.sm_scale_log2 = sm_scale * SPG_LOG2E;
  p.is_causal = is_causal;
  p.total_wg = p.nq * H * B;
  p.wg_per_xcd = (p.total_wg + 7) / 8;
  const int grid = p.wg_per_xcd * 8;
  if (D == 64) {
    if (out_dtype == 0) block_sparse_attn_kernel<64, 0><<<grid, 256, 0, st>>>(p);
    else block_sparse_attn_kernel<64, 1><<<grid, 256, 0, st>>>(p);
  } else {
    if (out_dtype == 0) block_sparse_attn_kernel<128, 0><<<grid, 256, 0, st>>>(p);
    else block_sparse_attn_kernel<128, 1><<<grid, 256, 0, st>>>(p);
  }
  return hipGetLastError();
}

}  // namespace spg
