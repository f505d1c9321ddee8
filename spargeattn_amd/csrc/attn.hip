// Block-sparse INT8-QK / FP8-PV attention for gfx950 (CDNA4), written for 64-lane wavefronts and MFMA.
//
// Replaces qk_int_sv_f8_block_sparse_attn_kernel (csrc/qattn/qk_int_sv_f8_cuda_sm89.cuh:42-755) as launched by
// qk_int8_sv_f8_accum_f32_block_sparse_attn_inst_buf_fuse_v_scale_with_pv_threshold
// (csrc/qattn/qk_int_sv_f8_cuda_sm89.cu:197-390): per-block or per-warp INT8 scales (qk_quant_gran 1 / 2), PV threshold
// per block (or per 32 rows, or none), fp32 PV accumulation, V scale fused into the epilogue.
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
//  * K/V tiles go HBM/L2 -> LDS directly (global_load_lds_dwordx4, no VGPR staging) through a 3-deep LDS ring:
//    the tiles of block it+2 are in flight while block it is computed, and ONE workgroup barrier per block covers
//    both the tile hand-over and the workgroup-wide PV-skip vote (the FP16-PV variant, whose V^T tiles are twice as
//    large, uses two-slot rings so that three workgroups still share a CU);
//  * the INT8 scale of Q is read per 128-row block or per wavefront of 32 rows (qk_quant_gran 1 / 2): a wavefront IS
//    the 32-row group, so the scale stays a scalar either way;
//  * LDS tiles are unpadded; bank conflicts are avoided by an XOR swizzle of the 16-byte chunks inside a row
//    (applied to the per-lane global address for K, baked into the HBM tile layout for V);
//  * the INT8 accumulators start at the bit pattern of the float 1/(2 pi), an inline constant of the instruction set (no
//    register or LDS read initialises them): read as a float the int32 result is 1/(2 pi) + dot * 2^-26, so the scores need
//    no int-to-float conversion; the constant is folded into the additive term of the fma that feeds exp2;
//  * only "skip" votes of the PV threshold reach LDS, and the rescale factor of O is computed only in iterations in which
//    a running maximum rose;
//  * workgroup ids are remapped so that one XCD (one L2) works on one head at a time, heaviest rows first.
#include "common.h"
#include "launch.h"
#include "lds_asm.h"

#include <type_traits>

namespace spg {

typedef int v8i __attribute__((ext_vector_type(8)));
typedef int v8i_a16 __attribute__((ext_vector_type(8), aligned(16)));
typedef int v16i __attribute__((ext_vector_type(16)));
typedef float v16f __attribute__((ext_vector_type(16)));

#define SPG_NEG_BIG (-5000000.0f)   // csrc/qattn/attn_utils.cuh:350, qk_int_sv_f8_cuda_sm89.cuh:171
#define SPG_FP8_OFFSET 8.807f       // csrc/qattn/attn_utils.cuh:28
#define SPG_ACC_C_BITS 0x3E22F983    // the float 1/(2 pi), an inline constant of the instruction set: initial accumulator
#define SPG_ACC_SCALE 67108864.0f    // 2^26: one unit of the integer dot product is 2^-26 in the binade [1/8, 1/4)
#define SPG_LOG2E 1.44269504088896340736f

struct AttnParams {
  const int8_t *q8, *k8;
  const uint8_t *v8;
  void *out;
  Strides os;      // element strides of out (B, H, N, D), last dimension contiguous
  const int32_t *lut, *valid;
  const float *pvthr, *q_scale, *k_scale, *v_scale;
  int32_t *pv_count;
  int B, H, Hkv, N, Nk, nq, nk;   // N query rows, Nk key/value rows per head (qo_len / kv_len of sm89.cu:256-300)
  float sm_scale_log2;
  int is_causal;
  int pv_mode;     // PVThresholdMode of the reference (attn_utils.cuh:58-62): 0 none, 1 per block, 2 per wavefront of 32 rows
  int q_per_warp;  // QuantGranularity of Q (sm89.cuh:106-121): 0 one scale per 128-row block, 1 one per 32 rows (B,H,nq*4)
  int total_wg, wg_per_xcd;
};

// v_max_f32 as one instruction: fmaxf() on a value the compiler cannot prove to be a quiet number (a loop-carried
// maximum, the output of a lane exchange) costs a canonicalising self-maximum per operand first.  The operands here are
// products and maxima of finite numbers.
__device__ __forceinline__ float max_raw(float a, float b) {
  float r;
  asm("v_max_f32 %0, %1, %2" : "=v"(r) : "v"(a), "v"(b));
  return r;
}
__device__ __forceinline__ float half_swap_max_raw(float v) {
  float lo, hi, r;
  half_swap(v, lo, hi);
  asm("s_nop 0\n\tv_max_f32 %0, %1, %2" : "=v"(r) : "v"(lo), "v"(hi));   // one idle state behind the lane exchange
  return r;
}
// e4m3 pack of the probabilities.  v_cvt_pk_fp8_f32 returns NaN (0x7f) for |x| > 464 unless MODE.FP16_OVFL is set, in
// which case finite values clamp to +-448 like the reference's cvt.rn.satfinite.e4m3x2.f32 (csrc/numeric_conversion.cuh:48-63);
// the bit is set once per wavefront, costs nothing per element and affects no other instruction this kernel depends on
// (the fp16 epilogue conversion cannot overflow: |O / d| <= max |V|).
__device__ __forceinline__ void fp8_saturation_on() {
  __builtin_amdgcn_s_setreg(1 | (23 << 6) | (0 << 11), 1);   // hwreg(HW_REG_MODE, offset 23, size 1) = FP16_OVFL
}
__device__ __forceinline__ int pack4_e4m3(float x0, float x1, float x2, float x3) {
  // both halves of the destination are written, so its initial content is irrelevant: start from a register that is
  // "defined" by an empty asm instead of a zeroed one
  int wv;
  asm volatile("" : "=v"(wv));
  wv = __builtin_amdgcn_cvt_pk_fp8_f32(x0, x1, wv, false);
  wv = __builtin_amdgcn_cvt_pk_fp8_f32(x2, x3, wv, true);
  return wv;
}

// Self test of the pack: codes[i] = e4m3(x[i]) exactly as the attention kernel produces it (saturate != 0) or as the bare
// instruction does (saturate == 0).  n is a multiple of 4.
__global__ __launch_bounds__(256) void fp8_pack_selftest_kernel(const float *__restrict__ x, uint32_t *__restrict__ codes,
                                                                int n4, int saturate) {
  if (saturate) fp8_saturation_on();
  const int i = blockIdx.x * 256 + threadIdx.x;
  if (i >= n4) return;
  const float4 v = ((const float4 *)x)[i];
  codes[i] = (uint32_t)pack4_e4m3(v.x, v.y, v.z, v.w);
}
void launch_fp8_pack_selftest(const float *x, uint8_t *codes, int n, int saturate, hipStream_t st) {
  const int n4 = n / 4;
  fp8_pack_selftest_kernel<<<(n4 + 255) / 256, 256, 0, st>>>(x, (uint32_t *)codes, n4, saturate);
}

// 16-byte-chunk swizzles.  K tile row = key (D bytes, D/16 chunks); V^T tile row = channel (64 bytes, 4 chunks).
// The LDS serves a ds_read_b128 one half-wavefront (32 lanes) at a time and needs two clocks for it when the 32
// addresses fall evenly on the sixteen 16-byte slots of a 256-byte line (two lanes per slot); a slot that is hit 2k
// times costs k times as much.  The slot of an address is (byte offset mod 256) / 16, so the low row bits already select
// part of it (one bit for 128-byte rows, two bits for 64-byte rows) and the swizzle must come from OTHER row bits that
// vary inside a half-wavefront: for the K operand lane r reads key row 32*((r>>2)&1) + 4*(r>>3) + (r&3) (+16 for the
// second tile), for the V^T operand lane r reads channel row r (+32 per output tile).
template <int D>
__device__ __forceinline__ uint32_t k_swz(uint32_t row) {
  if constexpr (D == 128) return ((row >> 1) & 3u) | (((row >> 5) & 1u) << 2);
  else return ((row >> 2) & 1u) | (((row >> 5) & 1u) << 1);
}
__device__ __forceinline__ int v_swz(int row) { return (row >> 2) & 3; }

// PV16 = false: V^T tiles are e4m3 (64 bytes per channel row), P is packed to e4m3 with the +8.807 exponent offset and
//               the denominator sums the un-rounded P (the SageAttention2 kernel, sm89.cuh).
// PV16 = true:  V^T tiles are fp16 (128 bytes per channel row, 16-byte chunks swizzled by slot = chunk ^ ((d >> 1) & 7)), P is
//               rounded to fp16 and the denominator sums the ROUNDED P in binary32 (what the SageAttention1 kernel's row
//               sum on the tensor cores computes, qk_int_sv_f16_cuda_sm80.cuh:339-368, attn_utils.cuh:599-626).  The PV product is
//               accumulated in fp32; the reference accumulates each 64-key block in fp16 before adding it to its fp32
//               accumulator (attn_utils.cuh:683-751), a rounding this kernel does not reproduce.
template <int D, int ODT, bool PV16>
__global__ __launch_bounds__(256, 3) void block_sparse_attn_kernel(const AttnParams p) {
  constexpr int KS = D / 32;        // k-steps of the int8 MFMA
  constexpr int NDT = D / 32;       // 32-channel output tiles
  constexpr int TILE = 64 * D;      // bytes of one K tile
  constexpr int VTILE = PV16 ? 2 * TILE : TILE;   // bytes of one V^T tile
  constexpr int CPR = D / 16;       // 16-byte chunks per K row
  constexpr int WL = D / 64;        // global_load_lds instructions per wave per K tile (TILE / 1024 / 4)
  constexpr int WLV = VTILE / 4096; // ... per V^T tile
  // Tile rings.  FP8 PV: three slots each, the tiles of block it+2 are requested while block it is computed.
  // FP16 PV (tiles twice as large): two slots each, so that three workgroups still share a CU (48 KiB): the K tile of
  // block it+2 goes to the slot block it's K tile just left, the V^T tile of block it+1 to the slot of block it-1.
  constexpr int NBUF = PV16 ? 2 : 3;
  // LDS: K ring [NBUF][TILE] | V^T ring [NBUF][VTILE] | votes
  __shared__ __align__(1024) unsigned char smem[NBUF * (TILE + VTILE)];
  // PV-skip vote of the per-block mode: a wavefront that votes "skip" stamps the iteration number into its slot; a slot
  // that does not hold the current iteration number means "compute".  Only "skip" votes are written (they are rare at the
  // thresholds in use), and only a wavefront that voted "skip" itself has to read the others' slots.  Two sets of slots,
  // used alternately: a wavefront can be at most one barrier ahead of the slowest one.
  __shared__ int sSkipAt[2][4];
  unsigned char *const sKr = smem;
  unsigned char *const sVr = smem + NBUF * TILE;
  const uint32_t lds_k0 = (uint32_t)(size_t)(__attribute__((address_space(3))) unsigned char *)smem;   // LDS byte address
  const uint32_t lds_v0 = lds_k0 + NBUF * TILE;

  // ---- workgroup -> (batch*head, q block): one XCD per head at a time, heavy (late) rows first ----------
  const int w = blockIdx.x;
  const int L = (w & 7) * p.wg_per_xcd + (w >> 3);
  if (L >= p.total_wg) return;
  const int bh = L / p.nq;
  const int qb = p.nq - 1 - (L % p.nq);
  const int head = bh % p.H;
  // grouped-query attention: H / Hkv consecutive query heads share one K/V head (sm89.cuh:118, head_id / num_kv_groups)
  const int bhk = (bh / p.H) * p.Hkv + head / (p.H / p.Hkv);
  const int nv = p.valid[(size_t)bh * p.nq + qb];
  if (nv == 0) return;                                       // output rows stay unwritten (sm89.cuh:232-235)
  const int32_t *lut_row = p.lut + ((size_t)bh * p.nq + qb) * p.nk;

  const int tid = threadIdx.x, lane = tid & 63, r = lane & 31, hh = lane >> 5;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);   // uniform: everything derived from it stays scalar
  const int N = p.N, Nk = p.Nk;
  const int q_row = qb * 128 + wave * 32 + r;
  if constexpr (!PV16) fp8_saturation_on();

  // ---- Q fragment: B operand of S^T = K.Q^T, resident for the whole loop -------------------------------
  v4i qreg[KS];
#pragma unroll
  for (int ks = 0; ks < KS; ks++) {
    qreg[ks] = (v4i){0, 0, 0, 0};
    if (q_row < N) qreg[ks] = *(const v4i *)(p.q8 + ((size_t)bh * N + q_row) * D + 32 * ks + 16 * hh);
  }

  const int8_t *kbase = p.k8 + (size_t)bhk * Nk * D;
  const uint8_t *vbase = p.v8 + (size_t)bhk * p.nk * (size_t)VTILE;
  // LUT and K scales are read through the constant address space: uniform addresses become scalar loads (SMEM),
  // which never touch the vector-memory counter the tile ring is synchronised with.
  typedef const __attribute__((address_space(4))) int32_t *c_i32_t;
  typedef const __attribute__((address_space(4))) float *c_f32_t;
  const c_i32_t lutc = (c_i32_t)(p.lut + ((size_t)bh * p.nq + qb) * p.nk);
  const c_f32_t kscale = (c_f32_t)(p.k_scale + (size_t)bhk * p.nk);
  // per-warp granularity: the 32 query rows of a wavefront are one quantisation group, so the scale stays a scalar
  const size_t qsi = (size_t)bh * p.nq + qb;
  const float qs = ((c_f32_t)p.q_scale)[p.q_per_warp ? qsi * 4 + wave : qsi];
  const float c = p.sm_scale_log2;
  const float thr = ((c_f32_t)p.pvthr)[head];

  // ---- tile loader: wave w copies LDS bytes [1024*(WL*w+u), +1024) of each tile, lane l the 16-byte chunk l ----
  // K: LDS chunk position pos <-> (row = pos / CPR, slot = pos % CPR) holds global chunk slot ^ k_swz(row).
  // A tile's global address is (uniform base of the block) + (per-lane 32-bit offset) + u*1024, and the same
  // u*1024 is the LDS offset: it rides in the instruction's immediate (applied to both addresses).
  // (the two per-lane offsets are recomputed from the thread id where they are used: cheaper than keeping them
  //  in registers across the loop, where the register file is the scarce resource)
  // Split into a part that depends on the lane only (recomputed with three or four vector instructions where it is
  // used) and a wavefront-uniform part that the compiler keeps in scalar registers: the K-row swizzle of chunk position
  // pos = WL*64*wave + lane takes its bits from lane bits 4-5 (D = 128) or 4 (D = 64) and from bit 1 of the wave index.
  static_assert(D == 64 || D == 128, "swizzle bit positions below");
  const uint32_t kswz_wave16 = (uint32_t)((wave >> 1) & 1) << (D == 128 ? 6 : 5);
  const uint32_t k_wave = (uint32_t)(WL * 1024 * wave), v_wave = (uint32_t)(WLV * 1024 * wave);
#define SPG_LANE_OFFSETS()                                                                                    \
  uint32_t lane_ = threadIdx.x & 63u;                                                                         \
  asm volatile("" : "+v"(lane_));                                                                             \
  const uint32_t pos0 = (uint32_t)(WL * 64 * wave) + lane_;                                                   \
  const uint32_t v_lane = v_wave + lane_ * 16u;                                                               \
  const uint32_t kswz_lane = D == 128 ? ((lane_ >> 4) & 3u) : ((lane_ >> 4) & 1u);                            \
  const uint32_t k_lane = k_wave + (((lane_ ^ kswz_lane) << 4) ^ kswz_wave16);   /* row * D + (slot ^ swz) * 16 */
  const int last_partial_blk = (Nk % 64) ? p.nk - 1 : -1;   // the only block with rows beyond Nk
  typedef __attribute__((address_space(3))) void *lds_ptr_t;
  typedef const __attribute__((address_space(1))) void *glb_ptr_t;
#define SPG_LOAD_K_(BLK, KOFF)   /* inside a scope that holds SPG_LANE_OFFSETS() */                            \
  {                                                                                                           \
    const int8_t *kb_ = kbase + (size_t)(BLK) * TILE;                                                         \
    unsigned char *lk_ = sKr + (KOFF) + WL * wave * 1024;                                                     \
    if ((BLK) != last_partial_blk) {                                                                          \
      /* the loads of one tile back to back: they share the LDS base register (M0) */                          \
      __builtin_amdgcn_global_load_lds((glb_ptr_t)(kb_ + k_lane), (lds_ptr_t)lk_, 16, 0, 0);                  \
      if constexpr (WL == 2)                                                                                  \
        __builtin_amdgcn_global_load_lds((glb_ptr_t)(kb_ + k_lane), (lds_ptr_t)lk_, 16, 1024, 0);             \
    } else {                                                                                                  \
      /* rows beyond Nk are clamped to row Nk-1: their scores are masked, their V rows are zero */              \
      const int rows_ok_ = Nk - (BLK) * 64;                                                                    \
      _Pragma("unroll") for (int u = 0; u < WL; u++) {                                                        \
        const uint32_t pos = pos0 + u * 64;                                                                   \
        const uint32_t row_ = min(pos / CPR, (uint32_t)(rows_ok_ - 1));                                       \
        const uint32_t ko_ = row_ * D + (((pos % CPR) ^ k_swz<D>(pos / CPR)) * 16u);                          \
        __builtin_amdgcn_global_load_lds((glb_ptr_t)(kb_ + ko_), (lds_ptr_t)(lk_ + u * 1024), 16, 0, 0);      \
      }                                                                                                       \
    }                                                                                                         \
  }
#define SPG_LOAD_V_(BLK, VOFF)                                                                                \
  {                                                                                                           \
    const uint8_t *vb_ = vbase + (size_t)(BLK) * VTILE;                                                       \
    unsigned char *lv_ = sVr + (VOFF) + WLV * wave * 1024;                                                    \
    __builtin_amdgcn_global_load_lds((glb_ptr_t)(vb_ + v_lane), (lds_ptr_t)lv_, 16, 0, 0);                    \
    if constexpr (WLV >= 2)                                                                                   \
      __builtin_amdgcn_global_load_lds((glb_ptr_t)(vb_ + v_lane), (lds_ptr_t)lv_, 16, 1024, 0);               \
    if constexpr (WLV == 4) {                                                                                 \
      __builtin_amdgcn_global_load_lds((glb_ptr_t)(vb_ + v_lane), (lds_ptr_t)lv_, 16, 2048, 0);               \
      __builtin_amdgcn_global_load_lds((glb_ptr_t)(vb_ + v_lane), (lds_ptr_t)lv_, 16, 3072, 0);               \
    }                                                                                                         \
  }
#define SPG_LOAD_K(BLK, KOFF) { SPG_LANE_OFFSETS() (void)v_lane; SPG_LOAD_K_(BLK, KOFF) }
#define SPG_LOAD_V(BLK, VOFF) { SPG_LANE_OFFSETS() (void)k_lane; (void)pos0; SPG_LOAD_V_(BLK, VOFF) }
// FP8 PV: both tiles of one block into ring slot offset BUFOFF (in K-tile units)
#define SPG_LOAD_TILES(BLK, BUFOFF) { SPG_LANE_OFFSETS() SPG_LOAD_K_(BLK, BUFOFF) SPG_LOAD_V_(BLK, BUFOFF) }

  // MFMA row i of key tile kt carries key 32*((i>>2)&1) + 16*kt + 4*(i>>3) + (i&3); rows krow0 and krow0+16 have
  // the same swizzle, so tile 1's operand sits 16 rows (16*D bytes) after tile 0's.
  const int krow0 = 32 * ((r >> 2) & 1) + 4 * (r >> 3) + (r & 3);
  const int ksw = k_swz<D>(krow0);
  // K operand of k-step ks (tile 0): chunk (2ks+hh) ^ ksw = ((2ks) ^ (ksw & 6)) | ((hh ^ ksw) & 1), i.e. the LDS
  // byte offset is k_rd_base + ((32*ks) ^ k_rd_x): one xor-add per read, two registers.
  const uint32_t k_rd_base = (uint32_t)(krow0 * D + ((hh ^ ksw) & 1) * 16);
  const uint32_t k_rd_x = (uint32_t)((ksw & 6) * 16);
  const int vsw = v_swz(r);                // v_swz(32*dt + r) does not depend on dt
  // V^T operand: key chunks 2hh and 2hh+1 of channel row r (+32*dt); the two swizzled slots differ in bit 4 only
  const uint32_t v_rd_lo = (uint32_t)(r * 64 + (((2 * hh) ^ vsw) * 16));
  // fp16 V^T operand of key step s: chunk (4hh + s) ^ ((r >> 1) & 7) of the 128-byte row r (+32*dt): v_rd16 ^ (16 * s)
  const uint32_t v_rd16 = (uint32_t)(r * 128 + (((4 * hh) ^ ((r >> 1) & 7)) * 16));

  float m = SPG_NEG_BIG;
  // d = 1.0 initially (sm89.cuh:172).  Each half-lane sums its own 32 keys, so only one of the two starts at 1.
  float dsum = hh == 0 ? 1.0f : 0.0f;
  v16f O[NDT];
#pragma unroll
  for (int dt = 0; dt < NDT; dt++)
#pragma unroll
    for (int e = 0; e < 16; e++) O[dt][e] = 0.f;
  int cnt = 0;

  // block ids: blk = block of iteration it, blk1 = it+1, blk2 = it+2 (tiles in flight); d3 = LUT delta of it+3.
  // K scales are fetched one iteration ahead as well.
  int blk = lutc[0];
  int blk1 = blk + (nv > 1 ? lutc[1] : 0);
  int blk2 = blk1 + (nv > 2 ? lutc[2] : 0);
  int d3 = nv > 3 ? lutc[3] : 0;
  float ksc = kscale[blk], ksc1 = kscale[blk1];
  if constexpr (PV16) {
    SPG_LOAD_K(blk, 0);
    SPG_LOAD_V(blk, 0);
    if (nv > 1) SPG_LOAD_K(blk1, TILE);           // the V^T tile of block 1 follows behind the first barrier
  } else {
    SPG_LOAD_TILES(blk, 0);
    if (nv > 1) SPG_LOAD_TILES(blk1, TILE);
  }
  uint32_t bufoff = 0;                     // LDS ring offset of block it

  // The INT8 accumulators do not start at zero but at the bit pattern 0x3E22F983 - the float 1/(2 pi), which the
  // instruction set offers as an INLINE CONSTANT, so the first product of each chain takes it as its C operand and no
  // register has to be initialised.  Its mantissa field is 2 292 099 and |dot| <= 128 * 128 * 128 = 2 097 152, so
  // the int32 sum stays inside the binade [1/8, 1/4): the accumulator READ AS A FLOAT is exactly
  // 1/(2 pi) + dot * 2^-26, and the scores need no int-to-float conversion - the 2^26 goes into the multiplier and the
  // constant into the additive term of the fma that feeds exp2.
  const float acc_c = __builtin_bit_cast(float, (int)SPG_ACC_C_BITS);
  if (tid < 8) (&sSkipAt[0][0])[tid] = -1;   // no slot may hold an iteration number by accident
  __builtin_amdgcn_s_waitcnt(0x0F70);     // vmcnt(0): Q fragment and the first tiles have arrived
  __syncthreads();

  // One K block.  TAIL = false: every block but the last two - PV-threshold test, no masks (sm89.cuh:283-391).
  // TAIL = true: the last two blocks - token-causal and out-of-bound masks where a score needs them, no skip
  // (sm89.cuh:467-648).  The two are
  // separate loops so that the common one carries none of the tail's predicates.
  // SLOT = 0, 1, 2: the ring slot of the block is a compile-time constant (the common loop is unrolled three times), so
  // every LDS address of the iteration is a loop-invariant register plus an immediate offset; SLOT = -1: the slot is the
  // run-time value `bufoff` (the up to two left-over blocks of the common loop and the two tail blocks).
  uint32_t kaddr_c[KS];
#pragma unroll
  for (int ks = 0; ks < KS; ks++) kaddr_c[ks] = lds_k0 + k_rd_base + ((uint32_t)(32 * ks) ^ k_rd_x);
  const uint32_t va_lo_c = lds_v0 + v_rd_lo, va_hi_c = lds_v0 + (v_rd_lo ^ 16u);
  const float cq26 = c * qs * SPG_ACC_SCALE;        // exponent multiplier a of a block = cq26 * k_scale * 2^-26
  // a 2^26 / (2 pi) >= 2^14  <=>  k_scale >= this bound; both are positive floats, so their bit patterns compare as integers
  const int kscale_precise_bits = __builtin_bit_cast(int, 16384.0f / (acc_c * cq26));
  auto step = [&](auto tail_tag, auto slot_tag, const int it) __attribute__((always_inline)) {
    constexpr bool TAIL = decltype(tail_tag)::value;
    constexpr int SLOT = decltype(slot_tag)::value;
    constexpr bool CS = SLOT >= 0 && !PV16;         // compile-time ring slot
    // ---- S^T = K . Q^T ---------------------------------------------------------------------------------
    v16i S0, S1;
    {
      // two groups of k-steps: the reads of the second group are in flight while the first group's MFMAs run
      constexpr int HK = KS / 2;
      v4i a0[KS], a1[KS];
      auto read_k = [&](int ks) __attribute__((always_inline)) {
        if constexpr (CS) lds_read_2x128<(SLOT < 0 ? 0 : SLOT) * TILE, (SLOT < 0 ? 0 : SLOT) * TILE + 16 * D>(a0[ks], a1[ks], kaddr_c[ks]);
        else lds_read_2x128<0, 16 * D>(a0[ks], a1[ks], kaddr_c[ks] + bufoff);
      };
      // first group: nothing to overlap with, the reads carry their wait
      {
        constexpr int SO = CS ? SLOT * TILE : 0;
        const uint32_t bo = CS ? 0u : bufoff;
        if constexpr (HK == 2) lds_read_4x128_wait<SO, SO + 16 * D>(a0[0], a1[0], a0[1], a1[1], kaddr_c[0] + bo, kaddr_c[1] + bo);
        else lds_read_2x128_wait<SO, SO + 16 * D>(a0[0], a1[0], kaddr_c[0] + bo, kaddr_c[0] + bo);
      }
      // second group: in flight under the first group's products (FP8 PV); the FP16-PV variant reads it afterwards, into
      // the first group's registers, which is what lets it keep three wavefronts per SIMD
      if constexpr (!PV16) {
#pragma unroll
        for (int ks = HK; ks < KS; ks++) read_k(ks);
      }
      // the first product of each chain, with the inline constant as its C operand (the compiler would otherwise keep
      // the constant in sixteen registers); the products that follow accumulate onto these and are ordinary builtins,
      // which the other chain's product always separates from their predecessor
      asm volatile("v_mfma_i32_32x32x32_i8 %0, %2, %4, 0.15915494\n\tv_mfma_i32_32x32x32_i8 %1, %3, %4, 0.15915494"
                   : "=&v"(S0), "=&v"(S1)
                   : "v"(a0[0]), "v"(a1[0]), "v"(qreg[0]));
#pragma unroll
      for (int ks = 1; ks < HK; ks++) {
        S0 = __builtin_amdgcn_mfma_i32_32x32x32_i8(a0[ks], qreg[ks], S0, 0, 0, 0);
        S1 = __builtin_amdgcn_mfma_i32_32x32x32_i8(a1[ks], qreg[ks], S1, 0, 0, 0);
      }
      if constexpr (PV16) {
        if constexpr (HK == 2) lds_read_4x128_wait<0, 16 * D>(a0[0], a1[0], a0[1], a1[1], kaddr_c[2] + bufoff, kaddr_c[3] + bufoff);
        else lds_read_2x128_wait<0, 16 * D>(a0[0], a1[0], kaddr_c[1] + bufoff, kaddr_c[1] + bufoff);
#pragma unroll
        for (int ks = HK; ks < KS; ks++) {
          S0 = __builtin_amdgcn_mfma_i32_32x32x32_i8(a0[ks - HK], qreg[ks], S0, 0, 0, 0);
          S1 = __builtin_amdgcn_mfma_i32_32x32x32_i8(a1[ks - HK], qreg[ks], S1, 0, 0, 0);
        }
      } else {
        if constexpr (HK == 2) lds_wait4(a0[2], a1[2], a0[3], a1[3]); else lds_wait2(a0[1], a1[1]);
#pragma unroll
        for (int ks = HK; ks < KS; ks++) {
          S0 = __builtin_amdgcn_mfma_i32_32x32x32_i8(a0[ks], qreg[ks], S0, 0, 0, 0);
          S1 = __builtin_amdgcn_mfma_i32_32x32x32_i8(a1[ks], qreg[ks], S1, 0, 0, 0);
        }
      }
    }

    // scalar prefetches for later iterations (SMEM).  Issued here, behind the last LDS wait of the products: scalar and
    // LDS loads share one counter, so a scalar load issued at the top of the loop would be waited for together with the
    // K operands; from here its latency runs under the MFMAs and the max reduction.
    __builtin_amdgcn_sched_barrier(0);
    float ksc2 = 0.f;
    int d4 = 0;
    if constexpr (!TAIL) {
      ksc2 = kscale[blk2];
      d4 = it + 4 < nv ? lutc[it + 4] : 0;
    }
    __builtin_amdgcn_sched_barrier(0);
    const float dq = qs * ksc;                     // used by the tail blocks only
    // S0/S1 are never rewritten (no copies at the join of the two paths): slot e < 16 is S0[e], slot e >= 16 is S1[e - 16]
    // multiplier of the accumulator read as a float: a * 2^26.  Wavefront-uniform, so it is moved to a scalar register:
    // the 32 multiply-adds below then read two vector registers each instead of three
    const float a26 = __builtin_bit_cast(float, __builtin_amdgcn_readfirstlane(__builtin_bit_cast(int, cq26 * ksc)));
    // The constant 1/(2 pi) leaves the exponent through ONE additive term, -(1/(2 pi) a 2^26 + m) (+ 8.807), whose rounding
    // error is half an ulp of 1.07e7 a.  Below 2^14 that is at most 2^-11 in the exponent (3e-4 relative in P, and the
    // row maximum's P stays below 448.2).  At or above it (large |q| |k| or a large softmax scale; uniform for the
    // wavefront) the scores are first taken relative to the lane's own maximum - an exact subtraction inside one binade -
    // so that no large constant is left to round: one more instruction per score, on such blocks only.
    const bool precise = __builtin_bit_cast(int, ksc) >= kscale_precise_bits;
    float fm, mloc = acc_c;
    int lim = 0x7fffffff;
    // The last two blocks take the masked arithmetic only if some score of the wavefront is masked at all (token-causal
    // kernels near the diagonal, a partial last K block); otherwise they run the arithmetic of the common loop, which
    // differs from the reference's masked branch (de-quantise, then scale) by the order of two binary32 roundings.
    bool masked = false;                             // wavefront-uniform
    if constexpr (TAIL) {
      // slot e of this lane is key 64*blk + 32*hh + e; keys beyond `lim` are masked
      const int key0 = blk * 64 + 32 * hh;
      if (p.is_causal) lim = q_row - key0;                       // key > query (attn_utils.cuh:334-361)
      if (it == nv - 1) lim = min(lim, Nk - 1 - key0);           // key >= kv_len (attn_utils.cuh:363-389)
      masked = __any(lim < 31);
    }
    if (!masked) {
      int imax = S0[0];
#pragma unroll
      for (int e = 1; e < 16; e++) imax = max(imax, S0[e]);
#pragma unroll
      for (int e = 0; e < 16; e++) imax = max(imax, S1[e]);
      mloc = __builtin_bit_cast(float, imax);   // 1/(2 pi) + 2^-26 * the largest of this lane's 32 dot products
      fm = (mloc - acc_c) * a26;                // the subtraction is exact (same binade)
    } else {
      fm = SPG_NEG_BIG;
      const float dq26 = dq * SPG_ACC_SCALE;
#pragma unroll
      for (int e = 0; e < 32; e++) {
        float v = (__builtin_bit_cast(float, e < 16 ? S0[e] : S1[e - 16]) - acc_c) * dq26;
        v = e > lim ? SPG_NEG_BIG : v;
        fm = fmaxf(fm, v);
      }
      fm = fm * c;
    }
    fm = half_swap_max_raw(fm);
    const float diff = fm - m;
    const float m_new = max_raw(m, fm);
    const float m_old = m;
    m = m_new;
    int vote = 1;
    if constexpr (!TAIL) {
      // max over rows of (diff) + thr > 0  <=>  some row has diff + thr > 0 (fp32 addition is monotonic)
      vote = __any(diff + thr > 0.f);
      if (vote == 0 && lane == 0) sSkipAt[it & 1][wave] = it;
    }
    __builtin_amdgcn_s_waitcnt(0x0F70);   // this wave's share of block it+1's tiles has landed in LDS
    __syncthreads();   // block it+1's tiles are complete; the votes are visible; ring slot of block it-1 is free
    bool compute = true;
    if constexpr (!TAIL) {   // workgroup-uniform in the per-block mode (sm89.cuh:318-353), wavefront-uniform otherwise
      compute = p.pv_mode == 0 || vote != 0;
      // per-block mode: a wavefront whose own vote is set knows the OR already; only one that voted "skip" has to read
      // what the others wrote (an LDS round trip that the common case does without)
      if (p.pv_mode == 1 && !compute)
        compute = !(sSkipAt[it & 1][0] == it && sSkipAt[it & 1][1] == it && sSkipAt[it & 1][2] == it &&
                    sSkipAt[it & 1][3] == it);
    }
    if constexpr (PV16) {
      // two-slot rings: every wavefront is past its reads of K slot it % 2 (this block's scores) and of V^T slot
      // (it + 1) % 2 (the previous block's P.V product)
      SPG_LANE_OFFSETS()
      (void)pos0;
      if (!TAIL || it + 2 < nv) SPG_LOAD_K_(blk2, bufoff);
      if (!TAIL || it + 1 < nv) SPG_LOAD_V_(blk1, 2 * (bufoff ^ (uint32_t)TILE));
    } else if (!TAIL || it + 2 < nv) {
      if constexpr (CS) {
        SPG_LOAD_TILES(blk2, ((SLOT + 2) % 3) * TILE);
      } else {
        const uint32_t b2 = bufoff == 0 ? 2 * TILE : bufoff - TILE;   // slot (it+2) % 3
        SPG_LOAD_TILES(blk2, b2);
      }
    }
    // the running maximum of some query rose: rescale (exp2(0) = 1 exactly, so the other iterations need neither the
    // exponential nor the products)
    if (__any(diff > 0.f)) {
      const float osc = __builtin_amdgcn_exp2f(m_old - m_new);
      dsum *= osc;
#pragma unroll
      for (int dt = 0; dt < NDT; dt++)
#pragma unroll
        for (int e = 0; e < 16; e++) O[dt][e] *= osc;
    }
    if (compute) {
      cnt++;
      const float neg0 = PV16 ? -m : -m + SPG_FP8_OFFSET;
      float ps;
      float x[32];
      if (!masked) {
        // three passes kept apart for the scheduler: a multiply-add feeding the exponential of the same element directly,
        // and the exponential feeding the running sum, would issue as one long chain of dependent instructions
        if (!precise) {
          const float neg = __builtin_fmaf(-acc_c, a26, neg0);   // takes the accumulator constant out: one rounding per row
#pragma unroll
          for (int e = 0; e < 32; e++) x[e] = __builtin_fmaf(__builtin_bit_cast(float, e < 16 ? S0[e] : S1[e - 16]), a26, neg);
        } else {
          // (S - S_max,lane) a + (S_max,lane a - m + offset): what the reference's fma(S, a, -m + offset) computes
          // (attn_utils.cuh:391-415), with the rounding of m as the only error
          const float c0 = __builtin_fmaf(mloc - acc_c, a26, neg0);
#pragma unroll
          for (int e = 0; e < 32; e++)
            x[e] = __builtin_fmaf(__builtin_bit_cast(float, e < 16 ? S0[e] : S1[e - 16]) - mloc, a26, c0);
        }
        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
        for (int e = 0; e < 32; e++) x[e] = __builtin_amdgcn_exp2f(x[e]);
        __builtin_amdgcn_sched_barrier(0);
        if constexpr (!PV16) {
          ps = x[0];
#pragma unroll
          for (int e = 1; e < 32; e++) ps += x[e];
        }
      } else {
        ps = 0.f;
        const float masked = __builtin_fmaf(SPG_NEG_BIG, c, neg0);   // what the sentinel score turns into
        const float dq26 = dq * SPG_ACC_SCALE;
#pragma unroll
        for (int e = 0; e < 32; e++) {
          // de-quantised score first, then the softmax scale, as the reference's masked branch does (sm89.cuh:467-648)
          const float sv = (__builtin_bit_cast(float, e < 16 ? S0[e] : S1[e - 16]) - acc_c) * dq26;
          const float t = __builtin_fmaf(sv, c, neg0);
          x[e] = __builtin_amdgcn_exp2f(e > lim ? masked : t);
          if constexpr (!PV16) ps += x[e];
        }
      }
      if constexpr (PV16) {
        typedef _Float16 h8 __attribute__((ext_vector_type(8)));
        typedef _Float16 h2 __attribute__((ext_vector_type(2)));
        typedef float f2 __attribute__((ext_vector_type(2)));
        h8 pb16[4];
#pragma unroll
        for (int s4 = 0; s4 < 4; s4++)
#pragma unroll
          for (int j = 0; j < 8; j += 2) {
            const f2 pr = {x[8 * s4 + j], x[8 * s4 + j + 1]};
            const h2 ph = __builtin_convertvector(pr, h2);          // v_cvt_pk_f16_f32, round to nearest even
            pb16[s4][j] = ph[0];
            pb16[s4][j + 1] = ph[1];
          }
        {
          // row sums of the ROUNDED P (the reference sums them on the tensor cores, rowsum_f16f16f32, attn_utils.cuh:614):
          // v_dot2_f32_f16 with a pair of ones adds two fp16 values to a binary32 accumulator per instruction, which
          // leaves the matrix unit to the two products.  Each half-lane sums its own 32 keys; the halves meet in the
          // epilogue.
          const h2 ones2 = {(_Float16)1, (_Float16)1};
          float rs = 0.f;
#pragma unroll
          for (int s4 = 0; s4 < 4; s4++)
#pragma unroll
            for (int j = 0; j < 8; j += 2) {
              const h2 pr = {pb16[s4][j], pb16[s4][j + 1]};
              rs = __builtin_amdgcn_fdot2(pr, ones2, rs, false);
            }
          dsum += rs;
        }
        // V^T operands in two halves of two 16-key steps each, through ONE set of registers (the budget of three
        // wavefronts per SIMD); every read carries its wait
        const uint32_t va = lds_v0 + 2 * bufoff + v_rd16;
#pragma unroll
        for (int half = 0; half < 2; half++) {
          v4i t[2][NDT];
          const uint32_t va0 = va ^ (uint32_t)(32 * half), va1 = va0 ^ 16u;
          if constexpr (NDT == 4)
            lds_read_8x128_wait<0, 4096, 8192, 12288>(t[0][0], t[0][1], t[0][2], t[0][3], t[1][0], t[1][1], t[1][2], t[1][3], va0, va1);
          else
            lds_read_4x128_wait<0, 4096>(t[0][0], t[0][1], t[1][0], t[1][1], va0, va1);
#pragma unroll
          for (int u = 0; u < 2; u++)
#pragma unroll
            for (int dt = 0; dt < NDT; dt++)
              O[dt] = __builtin_amdgcn_mfma_f32_32x32x16_f16(__builtin_bit_cast(h8, t[u][dt]), pb16[2 * half + u], O[dt], 0, 0, 0);
        }
      } else {
      dsum += ps;
      v8i pb;
#pragma unroll
      for (int u = 0; u < 8; u++) pb[u] = pack4_e4m3(x[4 * u], x[4 * u + 1], x[4 * u + 2], x[4 * u + 3]);
      {
        constexpr int HD = NDT / 2;
        constexpr int SB = CS ? SLOT * TILE : 0;     // ring slot as an immediate, or in the address registers
        const uint32_t va_lo = CS ? va_lo_c : va_lo_c + bufoff, va_hi = CS ? va_hi_c : va_hi_c + bufoff;
        v4i lo[NDT], hi[NDT];
        // group 0 (output tile dt reads channel rows 32 dt .. 32 dt + 31: 2048 bytes further on)
        if constexpr (HD == 2) lds_read_4x128_wait<SB, SB + 2048>(lo[0], lo[1], hi[0], hi[1], va_lo, va_hi);
        else lds_read_2x128_wait<SB, SB>(lo[0], hi[0], va_lo, va_hi);
        // group 1 in flight while group 0 multiplies
        if constexpr (HD == 2) {
          lds_read_pair<SB + 4096>(lo[2], hi[2], va_lo, va_hi);
          lds_read_pair<SB + 6144>(lo[3], hi[3], va_lo, va_hi);
        } else {
          lds_read_pair<SB + 2048>(lo[1], hi[1], va_lo, va_hi);
        }
#pragma unroll
        for (int dt = 0; dt < HD; dt++) {
          const v8i av = {lo[dt][0], lo[dt][1], lo[dt][2], lo[dt][3], hi[dt][0], hi[dt][1], hi[dt][2], hi[dt][3]};
          O[dt] = __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(av, pb, O[dt], 0, 0, 0, 0, 0, 0);
        }
        if constexpr (HD == 2) lds_wait4(lo[2], hi[2], lo[3], hi[3]); else lds_wait2(lo[1], hi[1]);
#pragma unroll
        for (int dt = HD; dt < NDT; dt++) {
          const v8i av = {lo[dt][0], lo[dt][1], lo[dt][2], lo[dt][3], hi[dt][0], hi[dt][1], hi[dt][2], hi[dt][3]};
          O[dt] = __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(av, pb, O[dt], 0, 0, 0, 0, 0, 0);
        }
      }
      }   // !PV16
    }
    // advance the block pipeline and the ring
    blk = blk1; blk1 = blk2; blk2 = blk2 + d3; d3 = d4;
    ksc = ksc1; ksc1 = ksc2;
    if constexpr (!CS) bufoff = bufoff == (NBUF - 1) * TILE ? 0 : bufoff + TILE;
  };
  {
    int it = 0;
    // the common loop, three blocks per trip (ring slots 0, 1, 2); `bufoff` stays 0 throughout where the slots are
    // compile-time constants, and three run-time steps bring it back to 0 where they are not
#pragma unroll 1
    for (; it + 3 <= nv - 2; it += 3) {
      step(std::false_type{}, std::integral_constant<int, 0>{}, it);
      step(std::false_type{}, std::integral_constant<int, 1>{}, it + 1);
      step(std::false_type{}, std::integral_constant<int, 2>{}, it + 2);
    }
#pragma unroll 1
    for (; it < nv - 2; it++) step(std::false_type{}, std::integral_constant<int, -1>{}, it);
#pragma unroll 1
    for (; it < nv; it++) step(std::true_type{}, std::integral_constant<int, -1>{}, it);
  }
#undef SPG_LOAD_TILES
#undef SPG_LOAD_K
#undef SPG_LOAD_V
#undef SPG_LOAD_K_
#undef SPG_LOAD_V_
#undef SPG_LANE_OFFSETS

  // one count per wavefront of 32 query rows, the layout of the reference's PV_Count (sm89.cuh:650-659); the four
  // counts of a Q block are equal because the skip decision is taken per block
  if (p.pv_count != nullptr && lane == 0) p.pv_count[((size_t)bh * p.nq + qb) * 4 + wave] = cnt;

  // ---- epilogue: O / d * v_scale -> out dtype -----------------------------------------------------------
  const float dtot = half_swap_sum_f32(dsum);
  const float inv = __builtin_amdgcn_rcpf(dtot);
  if (q_row < N) {
    uint16_t *orow = (uint16_t *)p.out + (size_t)(bh / p.H) * p.os.sb + (size_t)head * p.os.sh + (size_t)q_row * p.os.sn;
    const float *vs = p.v_scale + (size_t)bhk * D;
#pragma unroll
    for (int dt = 0; dt < NDT; dt++) {
#pragma unroll
      for (int g = 0; g < 4; g++) {
        const int d0 = 32 * dt + 8 * g + 4 * hh;
        float4 sc = make_float4(1.f, 1.f, 1.f, 1.f);
        if constexpr (!PV16) sc = *(const float4 *)(vs + d0);
        const uint16_t o0 = f32_to_elem<ODT>(O[dt][4 * g + 0] * inv * sc.x);
        const uint16_t o1 = f32_to_elem<ODT>(O[dt][4 * g + 1] * inv * sc.y);
        const uint16_t o2 = f32_to_elem<ODT>(O[dt][4 * g + 2] * inv * sc.z);
        const uint16_t o3 = f32_to_elem<ODT>(O[dt][4 * g + 3] * inv * sc.w);
        *(uint2 *)(orow + d0) = make_uint2((uint32_t)o0 | ((uint32_t)o1 << 16), (uint32_t)o2 | ((uint32_t)o3 << 16));
      }
    }
  }
}

hipError_t launch_block_sparse_attn(const int8_t *q8, const int8_t *k8, const uint8_t *v8, void *out, Strides os,
                                    int out_dtype, const int32_t *lut, const int32_t *valid, const float *pvthreshd,
                                    const float *q_scale, const float *k_scale, const float *v_scale, int B, int H,
                                    int Hkv, int N, int Nk, int D, float sm_scale, int is_causal, int q_per_warp,
                                    int pv_mode, int32_t *pv_count, hipStream_t st) {
  AttnParams p;
  p.q8 = q8; p.k8 = k8; p.v8 = v8; p.out = out; p.os = os; p.lut = lut; p.valid = valid; p.pvthr = pvthreshd;
  p.q_scale = q_scale; p.k_scale = k_scale; p.v_scale = v_scale; p.pv_count = pv_count;
  p.B = B; p.H = H; p.Hkv = Hkv; p.N = N; p.Nk = Nk; p.nq = (N + 127) / 128; p.nk = (Nk + 63) / 64;
  p.sm_scale_log2 = sm_scale * SPG_LOG2E;
  p.is_causal = is_causal;
  p.pv_mode = pv_mode;
  p.q_per_warp = q_per_warp;
  p.total_wg = p.nq * H * B;
  p.wg_per_xcd = (p.total_wg + 7) / 8;
  const int grid = p.wg_per_xcd * 8;
  if (v_scale != nullptr) {
    if (D == 64) {
      if (out_dtype == 0) block_sparse_attn_kernel<64, 0, false><<<grid, 256, 0, st>>>(p);
      else block_sparse_attn_kernel<64, 1, false><<<grid, 256, 0, st>>>(p);
    } else {
      if (out_dtype == 0) block_sparse_attn_kernel<128, 0, false><<<grid, 256, 0, st>>>(p);
      else block_sparse_attn_kernel<128, 1, false><<<grid, 256, 0, st>>>(p);
    }
  } else {   // fp16 V^T tiles, no V scale
    if (D == 64) {
      if (out_dtype == 0) block_sparse_attn_kernel<64, 0, true><<<grid, 256, 0, st>>>(p);
      else block_sparse_attn_kernel<64, 1, true><<<grid, 256, 0, st>>>(p);
    } else {
      if (out_dtype == 0) block_sparse_attn_kernel<128, 0, true><<<grid, 256, 0, st>>>(p);
      else block_sparse_attn_kernel<128, 1, true><<<grid, 256, 0, st>>>(p);
    }
  }
  return hipGetLastError();
}

}  // namespace spg
