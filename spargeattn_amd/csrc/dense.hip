// Dense FP16 flash attention on gfx950 MFMA: the comparator the sparse path's speed-up is quoted against.
// Same skeleton as attn.hip: transposed products (one query column per lane), K rows permuted so that the 32 scores of
// a lane are 32 consecutive keys, K / V^T tiles brought from HBM/L2 straight into LDS (global_load_lds, no register
// staging) through a two-slot ring with ONE barrier per block, unpadded LDS tiles with XOR-swizzled 16-byte chunks, LDS
// operand reads through inline asm with their own waits, XCD-aware workgroup order; v_mfma_f32_32x32x16_f16 for both
// products and fp16 P.  Not part of the reference.
//
// V comes as the fp16 V^T tiles of spg_v_tiles_f16: [nk][D][64] fp16, the eight 8-key chunks of a 128-byte row stored
// at slot = chunk ^ ((d >> 1) & 7), zero beyond N.
#include "common.h"
#include "launch.h"
#include "lds_asm.h"

#include <type_traits>

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

// K tile row = key (2 D bytes = D/8 chunks of 16 bytes).  A half-wavefront reads the K operand from key rows
// {0..15} u {32..47} (+16 for the second key tile) at one chunk index; the swizzle spreads those 32 rows evenly over the
// sixteen 16-byte slots of a 256-byte LDS line (two lanes per slot).
template <int D>
__device__ __forceinline__ uint32_t dense_k_swz(uint32_t row) {
  if constexpr (D == 128) return row & 15u;          // one row per line: 16 chunks
  else return (row >> 1) & 7u;                       // two rows per line: bit 0 of the row is already a slot bit
}

template <int D, int NW>
__global__ __launch_bounds__(64 * NW, 2) void dense_attn_f16_kernel(const DenseParams p) {
  constexpr int KS = D / 16;          // k-steps of QK^T
  constexpr int NDT = D / 32;         // output channel tiles
  constexpr int TILE = 64 * D * 2;    // bytes of one K tile and of one V^T tile
  constexpr int CPR = D / 8;          // 16-byte chunks per K row
  constexpr int QROWS = 32 * NW;      // query rows per workgroup
  constexpr int BPQ = QROWS / 64;     // key blocks per query tile on the diagonal
  constexpr int PIECES = TILE / 1024; // 1 KiB pieces (one global_load_lds instruction each) per tile
  constexpr int WL = (PIECES + NW - 1) / NW;   // pieces per wavefront per tile, at most (the last wavefronts may take fewer)
  constexpr int NBUF = 2;
  __shared__ __align__(1024) unsigned char smem[NBUF * 2 * TILE];   // K ring | V^T ring
  const uint32_t lds_k0 = (uint32_t)(size_t)(__attribute__((address_space(3))) unsigned char *)smem;
  const uint32_t lds_v0 = lds_k0 + NBUF * TILE;

  const int w = blockIdx.x;
  const int L = (w & 7) * p.wg_per_xcd + (w >> 3);
  if (L >= p.total_wg) return;
  const int bh = L / p.nq;
  const int qb = p.nq - 1 - (L % p.nq);
  const int tid = threadIdx.x, lane = tid & 63, r = lane & 31, hh = lane >> 5;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int N = p.N;
  const int q_row = qb * QROWS + wave * 32 + r;
  const int nblk = p.is_causal ? min(p.nk, BPQ * (qb + 1)) : p.nk;

  v8h qreg[KS];
#pragma unroll
  for (int ks = 0; ks < KS; ks++) {
    uint4 t = make_uint4(0, 0, 0, 0);
    if (q_row < N) t = *(const uint4 *)(p.q + ((size_t)bh * N + q_row) * D + 16 * ks + 8 * hh);
    qreg[ks] = __builtin_bit_cast(v8h, t);
  }
  const unsigned char *kbase = (const unsigned char *)(p.k + (size_t)bh * N * D);
  const unsigned char *vbase = (const unsigned char *)(p.vt + (size_t)bh * p.nk * (size_t)(D * 64));
  const float c = p.sm_scale_log2;

  // ---- tile loader: wavefront w copies LDS bytes [1024 (WL w + u), +1024) of each tile, lane l the 16-byte chunk l.
  // K: LDS chunk position pos <-> (row = pos / CPR, slot = pos % CPR) holds global chunk slot ^ swz(row); V^T tiles are
  // stored swizzled in HBM and copied verbatim.  Rows beyond N (last block only) are clamped to row N - 1: their scores
  // are masked below and their V rows are zero.
  typedef __attribute__((address_space(3))) void *lds_ptr_t;
  typedef const __attribute__((address_space(1))) void *glb_ptr_t;
  // wavefront w takes pieces [first, first + npieces): the first PIECES % NW wavefronts take one piece more
  constexpr int BASE = PIECES / NW, EXTRA = PIECES % NW;
  const int npieces = BASE + (wave < EXTRA ? 1 : 0);
  const int first = BASE * wave + min(wave, EXTRA);
  uint32_t k_off[WL];
#pragma unroll
  for (int u = 0; u < WL; u++) {
    const uint32_t pos = (uint32_t)(64 * (first + u) + lane);
    const uint32_t row = pos / CPR, slot = pos % CPR;
    k_off[u] = row * (D * 2) + ((slot ^ dense_k_swz<D>(row)) * 16u);
  }
  const uint32_t v_off = (uint32_t)(1024 * first + 16 * lane);
  const int last_partial_blk = (N % 64) ? p.nk - 1 : -1;
  auto load_tiles = [&](int blk, int slot) __attribute__((always_inline)) {
    const unsigned char *kb = kbase + (size_t)blk * TILE;
    const unsigned char *vb = vbase + (size_t)blk * TILE;
    unsigned char *lk = smem + slot * TILE + first * 1024;
    unsigned char *lv = smem + (NBUF + slot) * TILE + first * 1024;
    if (blk != last_partial_blk) {
#pragma unroll
      for (int u = 0; u < WL; u++)
        if (u < npieces) __builtin_amdgcn_global_load_lds((glb_ptr_t)(kb + k_off[u]), (lds_ptr_t)(lk + u * 1024), 16, 0, 0);
    } else {
      const uint32_t rows_ok = (uint32_t)(N - blk * 64);
#pragma unroll
      for (int u = 0; u < WL; u++) {
        const uint32_t pos = (uint32_t)(64 * (first + u) + lane);
        const uint32_t row = min(pos / CPR, rows_ok - 1), slot_ = pos % CPR;
        const uint32_t ko = row * (D * 2) + ((slot_ ^ dense_k_swz<D>(pos / CPR)) * 16u);
        if (u < npieces) __builtin_amdgcn_global_load_lds((glb_ptr_t)(kb + ko), (lds_ptr_t)(lk + u * 1024), 16, 0, 0);
      }
    }
#pragma unroll
    for (int u = 0; u < WL; u++)
      if (u < npieces) __builtin_amdgcn_global_load_lds((glb_ptr_t)(vb + v_off + u * 1024), (lds_ptr_t)(lv + u * 1024), 16, 0, 0);
  };

  // MFMA row i of key tile kt carries key 32*((i>>2)&1) + 16*kt + 4*(i>>3) + (i&3): after S^T, register e of tile kt in
  // lane (r, hh) is key 32 hh + 16 kt + e, i.e. the lane's 32 scores are 32 consecutive keys.  Rows krow0 and krow0 + 16
  // have the same swizzle, so tile 1's operand sits 16 rows after tile 0's.
  const uint32_t krow0 = (uint32_t)(32 * ((r >> 2) & 1) + 4 * (r >> 3) + (r & 3));
  const uint32_t ksw = dense_k_swz<D>(krow0);
  // K operand of k-step ks: chunk (2 ks + hh) ^ ksw of row krow0, i.e. byte k_rd_base + ((32 ks) ^ k_rd_x)
  const uint32_t k_rd_base = lds_k0 + krow0 * (D * 2) + (((uint32_t)hh ^ ksw) & 1u) * 16u;
  const uint32_t k_rd_x = (ksw & ~1u) * 16u;
  // V^T operand of key step s: chunk (4 hh + s) ^ ((r >> 1) & 7) of the 128-byte row r (+ 32 dt): va ^ (16 s)
  const uint32_t va0 = lds_v0 + (uint32_t)(r * 128 + (((4 * hh) ^ ((r >> 1) & 7)) * 16));

  float m = -INFINITY, dsum = 0.f;
  v16f O[NDT];
#pragma unroll
  for (int dt = 0; dt < NDT; dt++)
#pragma unroll
    for (int e = 0; e < 16; e++) O[dt][e] = 0.f;

  load_tiles(0, 0);
  __builtin_amdgcn_s_waitcnt(0x0F70);     // vmcnt(0)
  __syncthreads();

  // One key block.  SLOT = blk & 1 is a compile-time constant (the loop below is unrolled twice), so every LDS address
  // of the step is a loop-invariant register plus an immediate offset.
  auto step = [&](auto slot_tag, const int blk) __attribute__((always_inline)) {
    constexpr int SLOT = decltype(slot_tag)::value;
    constexpr int SO = SLOT * TILE;
    // slot SLOT^1 was last read in iteration blk-1, which every wavefront has left (barrier at its end)
    if (blk + 1 < nblk) load_tiles(blk + 1, SLOT ^ 1);

    // ---- S^T = K . Q^T: the reads of the second half of the k-steps are in flight while the first half multiplies
    v16f S0, S1;
#pragma unroll
    for (int e = 0; e < 16; e++) { S0[e] = 0.f; S1[e] = 0.f; }
    {
      // one k-step (two reads) in flight while the previous one multiplies: two small operand buffers
      v4i a0[2], a1[2];
      lds_read_2x128<SO, SO + 16 * D * 2>(a0[0], a1[0], k_rd_base + k_rd_x);
#pragma unroll
      for (int ks = 0; ks < KS; ks++) {
        const int cur = ks & 1, nxt = cur ^ 1;
        if (ks + 1 < KS) {
          lds_read_2x128<SO, SO + 16 * D * 2>(a0[nxt], a1[nxt], k_rd_base + ((uint32_t)(32 * (ks + 1)) ^ k_rd_x));
          asm volatile("s_waitcnt lgkmcnt(2)" : "+v"(a0[cur]), "+v"(a1[cur]));   // all but the two reads just issued
        } else {
          lds_wait2(a0[cur], a1[cur]);
        }
        S0 = __builtin_amdgcn_mfma_f32_32x32x16_f16(__builtin_bit_cast(v8h, a0[cur]), qreg[ks], S0, 0, 0, 0);
        S1 = __builtin_amdgcn_mfma_f32_32x32x16_f16(__builtin_bit_cast(v8h, a1[cur]), qreg[ks], S1, 0, 0, 0);
      }
    }

    // slot e of this lane is key 64 blk + 32 hh + e (e < 16: S0[e], else S1[e - 16])
    const bool edge = (p.is_causal && blk >= BPQ * qb) || (blk == p.nk - 1);
    float x[32];
#pragma unroll
    for (int e = 0; e < 32; e++) x[e] = e < 16 ? S0[e] : S1[e - 16];
    if (edge) {
      const int key0 = 64 * blk + 32 * hh;
      int lim = N - 1 - key0;
      if (p.is_causal) lim = min(lim, q_row - key0);
#pragma unroll
      for (int e = 0; e < 32; e++) x[e] = e > lim ? -INFINITY : x[e];
    }
    float fm = x[0];
#pragma unroll
    for (int e = 1; e < 32; e++) fm = fmaxf(fm, x[e]);
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
#pragma unroll
    for (int e = 0; e < 32; e++) x[e] = __builtin_fmaf(x[e], c, -m_use);
#pragma unroll
    for (int e = 0; e < 32; e++) x[e] = __builtin_amdgcn_exp2f(x[e]);
    float ps = 0.f;
#pragma unroll
    for (int e = 0; e < 32; e++) ps += x[e];
    dsum += ps;
    v8h pb[4];
#pragma unroll
    for (int s4 = 0; s4 < 4; s4++)
#pragma unroll
      for (int j = 0; j < 8; j += 2) {
        const auto h2 = __builtin_amdgcn_cvt_pkrtz(x[8 * s4 + j], x[8 * s4 + j + 1]);   // two fp16 in one instruction
        pb[s4][j] = (_Float16)h2[0];
        pb[s4][j + 1] = (_Float16)h2[1];
      }

    // ---- O^T += V^T . P^T: the reads of key step s + 1 are in flight while step s multiplies
    {
      const uint32_t va = va0;
      v4i t[2][NDT];
      auto read_v = [&](int buf, int s4) __attribute__((always_inline)) {
        lds_read_2x128<SO, SO + 4096>(t[buf][0], t[buf][1], va ^ (uint32_t)(16 * s4));
        if constexpr (NDT == 4) lds_read_2x128<SO + 8192, SO + 12288>(t[buf][2], t[buf][3], va ^ (uint32_t)(16 * s4));
      };
      read_v(0, 0);
#pragma unroll
      for (int s4 = 0; s4 < 4; s4++) {
        const int cur = s4 & 1, nxt = cur ^ 1;
        if (s4 + 1 < 4) {
          read_v(nxt, s4 + 1);
          if constexpr (NDT == 4) asm volatile("s_waitcnt lgkmcnt(4)" : "+v"(t[cur][0]), "+v"(t[cur][1]), "+v"(t[cur][2]), "+v"(t[cur][3]));
          else asm volatile("s_waitcnt lgkmcnt(2)" : "+v"(t[cur][0]), "+v"(t[cur][1]));
        } else {
          if constexpr (NDT == 4) lds_wait4(t[cur][0], t[cur][1], t[cur][2], t[cur][3]);
          else lds_wait2(t[cur][0], t[cur][1]);
        }
#pragma unroll
        for (int dt = 0; dt < NDT; dt++)
          O[dt] = __builtin_amdgcn_mfma_f32_32x32x16_f16(__builtin_bit_cast(v8h, t[cur][dt]), pb[s4], O[dt], 0, 0, 0);
      }
    }
    __builtin_amdgcn_s_waitcnt(0x0F70);   // this wavefront's share of block blk+1's tiles has landed in LDS
    __syncthreads();                      // block blk+1's tiles are complete; every wavefront is done with block blk's
  };
  {
    int blk = 0;
#pragma unroll 1
    for (; blk + 2 <= nblk; blk += 2) {
      step(std::integral_constant<int, 0>{}, blk);
      step(std::integral_constant<int, 1>{}, blk + 1);
    }
    if (blk < nblk) step(std::integral_constant<int, 0>{}, blk);
  }

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

hipError_t launch_dense_attn_f16(const void *q, const void *k, const void *vt, void *out, int B, int H, int N, int D,
                                 float sm_scale, int is_causal, hipStream_t st) {
  DenseParams p;
  p.q = (const uint16_t *)q; p.k = (const uint16_t *)k; p.vt = (const uint16_t *)vt; p.out = (uint16_t *)out;
  // wavefronts (32 query rows each) per workgroup: 6 share a tile pair at D = 128 (two 64 KiB rings per CU, three
  // wavefronts per SIMD at 168 registers), 4 at D = 64
  const int NW = D == 64 ? 4 : 8;
  p.B = B; p.H = H; p.N = N; p.nq = (N + 32 * NW - 1) / (32 * NW); p.nk = (N + 63) / 64;
  p.sm_scale_log2 = sm_scale * 1.44269504088896340736f;
  p.is_causal = is_causal;
  p.total_wg = p.nq * H * B;
  p.wg_per_xcd = (p.total_wg + 7) / 8;
  if (D == 64) dense_attn_f16_kernel<64, 4><<<p.wg_per_xcd * 8, 256, 0, st>>>(p);
  else dense_attn_f16_kernel<128, 8><<<p.wg_per_xcd * 8, 512, 0, st>>>(p);
  return hipGetLastError();
}

}  // namespace spg
