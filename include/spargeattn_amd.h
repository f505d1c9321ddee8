/*
 * spargeattn_amd.h - C ABI of the MI355X (gfx950) SpargeAttn hot path.
 *
 * One function per stage of
 *   spas_sage2_attn_meansim_topk_cuda   (spas_sage_attn/core.py:105-169)
 *   block_sparse_sage2_attn_cuda        (spas_sage_attn/core.py:171-233)
 * of thu-ml/SpargeAttn.  Every function takes raw DEVICE pointers, explicit
 * sizes, enum ints and a HIP stream (hipStream_t passed as void*); it launches
 * asynchronously on that stream, allocates nothing, synchronises nothing and
 * keeps no state - with one exception, spg_km_mean_static, which owns an 8 MiB
 * device array per GPU and remembers its address (see there).  Tensors the
 * library produces are contiguous (B,H,N,D) ("HND"); the caller's own q, k, v
 * and output may be strided (see "Strides" below).
 * Return value: SPG_OK or an error code; spg_last_error() gives the message of
 * the last failure on the calling thread.
 *
 * Block geometry (fixed, as on the reference's non-Hopper path, core.py:128):
 *   Q block = 128 rows, K/V block = 64 rows; nq = ceil(N/128), nk = ceil(N/64).
 */
#ifndef SPARGEATTN_AMD_H
#define SPARGEATTN_AMD_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

enum spg_status {
  SPG_OK = 0,
  SPG_ERR_INVALID = 1,      /* bad argument (maps to ValueError / RuntimeError on the Python side) */
  SPG_ERR_UNSUPPORTED = 2,  /* valid but outside what the kernels cover (e.g. head_dim not in {64,128}) */
  SPG_ERR_HIP = 3           /* a HIP runtime call failed */
};

enum spg_dtype { SPG_F16 = 0, SPG_BF16 = 1 };

/* PVThresholdMode of the reference (csrc/qattn/attn_utils.cuh:58-62): whether the P.V product of a K block is skipped
 * when no row's running maximum came within pvthreshd of being raised by it - never, decided for the whole 128-row
 * Q block (the mode every Python entry point of the reference uses), or for each 32 query rows on their own. */
enum spg_pv_threshold_mode { SPG_PV_NONE = 0, SPG_PV_PER_BLOCK = 1, SPG_PV_PER_WARP = 2 };

/* qk_quant_gran of the reference's kernel entry points (csrc/qattn/attn_cuda.h:61-76, dispatched in
 * csrc/pytorch_extensions_utils.cuh:71-85; QuantGranularity in csrc/qattn/attn_utils.cuh:44-50), same integer values:
 * 1 = one INT8 scale per 128-row Q block and per 64-row K block (what every Python operator of the reference passes),
 * 2 = one scale per warp: 32 query rows (q_scale (B,H,nq*4), index 4*qblock + row/32, csrc/qattn/qk_int_sv_f8_cuda_sm89.cuh:111-115)
 *     and 64 key rows, i.e. K scales stay per block (WARP_K = CTA_K = 64);
 * 3 = per thread: tied to the lane layout of mma.sync fragments, refused with SPG_ERR_UNSUPPORTED. */
enum spg_qk_quant_gran { SPG_QUANT_PER_BLOCK = 1, SPG_QUANT_PER_WARP = 2 };

/* element kinds accepted for a user block mask ("non-zero = keep", spas_sage_attn/utils.py:68-69) */
enum spg_mask_kind {
  SPG_MASK_I8 = 0, SPG_MASK_I16 = 1, SPG_MASK_I32 = 2, SPG_MASK_I64 = 3,
  SPG_MASK_F16 = 4, SPG_MASK_F32 = 5, SPG_MASK_F64 = 6   /* bf16 uses SPG_MASK_F16: both test (bits & 0x7fff) != 0 */
};

int spg_version(void);
const char *spg_last_error(void);

/* Strides.  The tensors the CALLER owns in its own layout - q, k, v going in, the attention output coming out - are
 * described by a pointer plus `const int64_t *strides`: NULL for a contiguous (B,H,N,D) tensor ("HND"), or a HOST array
 * {batch, head, row} of element strides with the last dimension contiguous, e.g. {N*H*D, D, H*D} for a contiguous
 * (B,N,H,D) tensor ("NHD").  This is what tensor_layout and the stride arguments of the reference's kernels carry
 * (csrc/qattn/qk_int_sv_f8_cuda_sm89.cu:256-300; the Python API copies NHD inputs to HND first, core.py:109-117, which
 * a caller of this library need not do).  Rows move in 16-byte pieces: every stride is a positive multiple of 8
 * elements and the pointer is 16-byte aligned.  Everything the library produces for itself (int8 tensors, scales,
 * pooled blocks, LUT, FP8 tiles) is contiguous HND. */

/* ---- A2: km = k.mean(dim=-2)  (spas_sage_attn/core.py:119-120) -------------------------------
 * k (B,H,N,D) dtype, strided -> km (B,H,D) dtype.  Column sums are accumulated in binary64 and rounded once.
 * workspace: spg_km_mean_workspace_bytes() bytes of device scratch (per-chunk partial sums). */
size_t spg_km_mean_workspace_bytes(int B, int H, int N, int D);
int spg_km_mean(const void *k, const int64_t *k_strides, void *km, void *workspace, int B, int H, int N, int D, int dtype,
                void *stream);

/* ---- A2 for callers that cannot allocate (no counterpart in the reference).
 * Same result as spg_km_mean, bit for bit, without a workspace argument: the partial sums go to an 8 MiB array in
 * device memory that the library owns (one per GPU, held until the process ends), so the call performs no allocation of
 * any kind - it is meant for code under HIP graph capture, tight serving loops and harnesses that forbid hipMalloc.
 * Limit: spg_km_mean_workspace_bytes(B,H,N,D) <= 8 MiB (any shape with B*H <= 8192 at D = 128 or B*H <= 16384 at D = 64);
 * larger shapes return SPG_ERR_UNSUPPORTED.  All calls on one GPU share the array: calls that overlap in time on one
 * GPU (two streams, two threads) race and must be ordered by the caller; calls on one stream are ordered already.
 * The first call on a device looks the array's address up (no allocation, but make it outside a graph capture).
 * `stream` must belong to the current device (SPG_ERR_INVALID otherwise): each GPU has its own copy of the array. */
int spg_km_mean_static(const void *k, const int64_t *k_strides, void *km, int B, int H, int N, int D, int dtype,
                       void *stream);

/* ---- A3/A4: fused pool + self-similarity + per-block INT8 quantisation ------------------------
 * replaces triton_bmm_pool_sim_simmean_fuse_quant (spas_sage_attn/utils.py:161-214, wrapper 270-280).
 * x (B,H,N,D) dtype, strided; km (B,H,D) dtype or NULL (Q: NULL, K: the column mean, subtracted in dtype);
 * block = 128 (Q) or 64 (K); simthreshd1 (H,) float32.
 * quant_rows = rows that share one INT8 scale: `block` for per-block scales (the reference's operators), or 32 with
 * block = 128 and km == NULL for the per-warp granularity of Q (per_warp_int8 with WARPQ = 32,
 * spas_sage_attn/quant_per_block.py:102-148, same arithmetic as the fused kernel): nb * block / quant_rows scales per
 * head, a 32-row group without rows (past N in the last block) gets the scale of an all-zero group, 1e-7.
 * out: pool (B,H,nb,D) dtype; sim (B,H,nb) uint8 0/1; xq (B,H,N,D) int8; scale (B,H,nb*block/quant_rows) float32.
 * ---- A13: with pool == NULL and sim == NULL this is qk_quantize (utils.py:89-159): xq and scale only. */
int spg_pool_sim_quant(const void *x, const int64_t *x_strides, const void *km, void *pool, uint8_t *sim, int8_t *xq,
                       float *scale, const float *simthreshd1, int B, int H, int N, int D, int block, int quant_rows,
                       int dtype, void *stream);

/* ---- A5-A8: compressed attention, top-k / CDF selection, block map, LUT ------------------------
 * replaces the torch glue of get_block_map_meansim_fuse_quant (spas_sage_attn/utils.py:386-420),
 * triton_fill_causal_mask (304-316), triton_fill_block_map_kernel (282-302) and
 * triton_block_map_to_lut_kernel (54-87) with one kernel; the score matrix never reaches HBM.
 * Exactly one of topk / cdfthreshd ((H,) float32 device pointers) is non-NULL.
 * pool_q (B,H,nq,D), sim_q (B,H,nq); pool_k (B,Hkv,nk,D), sim_k (B,Hkv,nk) with Hkv dividing H: query head h is scored
 * against K head h / (H / Hkv).  Hkv = H is the reference's case; fewer K heads (grouped-query attention) is an
 * extension - the reference's pooled-score matmul needs equal head counts (utils.py:388).
 * out: lut (B,H,nq,nk) int32 delta-encoded ascending block indices, zero tail;
 *      valid_block_num (B,H,nq) int32; block_map (B,H,nq,nk) uint8 0/1 or NULL. */
int spg_block_select(const void *pool_q, const uint8_t *sim_q, const void *pool_k, const uint8_t *sim_k,
                     const float *topk, const float *cdfthreshd, int is_causal, int attention_sink,
                     int32_t *lut, int32_t *valid_block_num, uint8_t *block_map,
                     int B, int H, int Hkv, int nq, int nk, int D, int dtype, void *stream);

/* ---- A8 alone: user block mask -> LUT  (block_map_lut_triton, spas_sage_attn/utils.py:76-87) ---- */
int spg_map_to_lut(const void *mask, int mask_kind, int32_t *lut, int32_t *valid_block_num,
                   int B, int H, int nq, int nk, void *stream);

/* ---- A9+A10: V -> fp16 -> per-channel FP8 e4m3 ---------------------------------------------------
 * replaces transpose_pad_permute_cuda + scale_fuse_quant_cuda(..., scale_max = 2.25)
 * (csrc/fused/fused.cu:193-267, 269-344; called at core.py:147,151).
 * v (B,H,N,D) dtype, strided (bf16 input is first rounded to fp16, core.py:117).
 * out: v8 e4m3fn codes in TILE layout [B][H][nk][D][64] (key index fastest inside a 64-key tile, rows
 *      beyond N are zero; inside a 64-byte row the four 16-key chunks are XOR-swizzled: key chunk kc is
 *      stored at slot kc ^ ((d >> 2) & 3)) - the layout the attention kernel copies to LDS verbatim;
 *      v_scale (B,H,D) float32 = amax/2.25.  v_scale doubles as the amax scratch between the passes. */
int spg_v_quant_fp8(const void *v, const int64_t *v_strides, uint8_t *v8, float *v_scale, int B, int H, int N, int D,
                    int dtype, void *stream);

/* ---- A11: block-sparse INT8-QK / FP8-PV attention ------------------------------------------------
 * replaces qk_int8_sv_f8_accum_f32_block_sparse_attn_inst_buf_fuse_v_scale_with_pv_threshold
 * (csrc/qattn/attn_cuda.h:61-76, csrc/qattn/qk_int_sv_f8_cuda_sm89.cu:197-390) with
 * tensor_layout = HND; qk_quant_gran as that entry point takes it (1 per block, 2 per warp; 3 is refused);
 * pv_threshold_mode = SPG_PV_PER_BLOCK is what that entry point compiles in (sm89.cu:365), the other two modes are the
 * kernel template's (sm89.cuh:283-391).
 * q8 int8 (B,H,N,D); k8 int8 (B,Hkv,N_kv,D); v8 as produced by spg_v_quant_fp8 for Hkv heads of N_kv rows; out (B,H,N,D)
 * out_dtype, strided.  N (qo_len) and N_kv (kv_len) are independent as in the reference (sm89.cu:256-300):
 * nq = ceil(N/128), nk = ceil(N_kv/64); keys >= N_kv of the last block are masked.
 * lut (B,H,nq,nk) / valid_block_num as above; pvthreshd (H,) float32; q_scale (B,H,nq) for qk_quant_gran = 1 or
 * (B,H,nq*4) for qk_quant_gran = 2, k_scale (B,Hkv,nk),
 * v_scale (B,Hkv,D) float32; Hkv divides H: query head h reads K/V head h / (H / Hkv) (grouped-query attention,
 * sm89.cu:310-314, sm89.cuh:118); Hkv = H is plain multi-head attention; pv_count (B,H,nq*4) int32 or NULL: number of K blocks
 * whose PV was computed, one entry per 32 query rows as in the reference (sm89.cu:331-334); entries of Q blocks with
 * valid_block_num == 0 are left untouched.
 * Row blocks with valid_block_num == 0 are left unwritten, as in the reference (sm89.cuh:232-235). */
int spg_block_sparse_attn(const int8_t *q8, const int8_t *k8, const uint8_t *v8, void *out, const int64_t *out_strides,
                          int out_dtype, const int32_t *lut, const int32_t *valid_block_num, const float *pvthreshd,
                          const float *q_scale, const float *k_scale, const float *v_scale,
                          int B, int H, int Hkv, int N, int N_kv, int D, float sm_scale, int is_causal,
                          int qk_quant_gran, int pv_threshold_mode, int32_t *pv_count, void *stream);

/* ---- SageAttention1-style variant: INT8 QK^T, FP16 PV.
 * Replaces qk_int8_sv_f16_accum_f16_block_sparse_attn_inst_buf_with_pv_threshold (csrc/qattn/attn_cuda.h:32-45,
 * kernel csrc/qattn/qk_int_sv_f16_cuda_sm80.cuh:42-671) as called by spas_sage_attn_meansim[_topk]_cuda
 * (spas_sage_attn/core.py:235-319): P is rounded to fp16, the denominator sums the rounded P, the output is O / d
 * with no V scale, is_causal masks at token level.  PV is accumulated in fp32 throughout (the reference rounds each
 * 64-key partial product to fp16 first).
 * spg_v_tiles_f16 prepares the V operand: v (B,H,N,D) fp16|bf16 -> vt (B,H,ceil(N/64),D,64) fp16, the V^T of each
 * 64-key block (bf16 is rounded to fp16 as core.py:247 does), 8-key chunks of a row stored at slot chunk ^ ((d >> 1) & 7),
 * zero beyond N.  It takes the place of the kernel's transposing shared-memory reads (ldmatrix.trans). */
int spg_v_tiles_f16(const void *v, const int64_t *v_strides, void *vt, int B, int H, int N, int D, int dtype, void *stream);
int spg_block_sparse_attn_f16v(const int8_t *q8, const int8_t *k8, const void *vt, void *out, const int64_t *out_strides,
                               int out_dtype, const int32_t *lut, const int32_t *valid_block_num, const float *pvthreshd,
                               const float *q_scale, const float *k_scale,
                               int B, int H, int Hkv, int N, int N_kv, int D, float sm_scale, int is_causal,
                               int qk_quant_gran, int pv_threshold_mode, int32_t *pv_count, void *stream);

/* ---- measurement comparator: dense FP16 flash attention on MFMA (no counterpart in the reference;
 * the "dense FP16 attention kernel built in the same run" the speed-up is quoted against).
 * q,k,out (B,H,N,D) fp16; vt = the fp16 V^T tiles spg_v_tiles_f16 writes, (B,H,ceil(N/64),D,64), chunk-swizzled,
 * zero beyond N. */
int spg_dense_attn_f16(const void *q, const void *k, const void *vt, void *out, int B, int H, int N, int D,
                       float sm_scale, int is_causal, void *stream);

/* ---- self test (no counterpart in the reference): the INT8 quantisation and the cosine normalisation divide by
 * a per-block / per-row value through a shared reciprocal; this entry point compares that division with the
 * hardware's correctly rounded one for every finite fp16 and bf16 numerator against n_divisors pseudo-random
 * divisors.  counts (device, 2 x uint64, zeroed by the caller): [0] += comparisons, [1] += mismatches. */
int spg_selftest_division(unsigned long long *counts, int n_divisors, unsigned int seed, void *stream);

/* ---- self test (no counterpart in the reference): the fp32 -> e4m3 pack of the probabilities.
 * x (n,) float32 device, n a multiple of 4 -> codes (n,) uint8.  saturate != 0: exactly what spg_block_sparse_attn does
 * (round to nearest even, finite |x| > 448 clamps to +-448 like cvt.rn.satfinite.e4m3x2.f32,
 * csrc/numeric_conversion.cuh:48-63; NaN and +-inf give NaN - the reference maps +-inf to +-448, a case the kernel
 * cannot reach because P = 2^x with x <= 8.807);
 * saturate == 0: the bare v_cvt_pk_fp8_f32 instruction (NaN for |x| > 464), for documentation of the hardware. */
int spg_selftest_fp8_pack(const float *x, uint8_t *codes, int n, int saturate, void *stream);

#ifdef __cplusplus
}
#endif
#endif /* SPARGEATTN_AMD_H */
