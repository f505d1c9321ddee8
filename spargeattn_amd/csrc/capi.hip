// extern "C" entry points declared in include/spargeattn_amd.h: argument checks, then a launch on the caller's
// stream.  No allocation, no synchronisation; the only state is the thread-local error string and, behind
// spg_km_mean_static, a library-owned device array per GPU with its cached address.
#include "../../include/spargeattn_amd.h"
#include "launch.h"

#include <cstdarg>
#include <cstdio>

namespace {
thread_local char g_err[512] = "";

int fail(int code, const char *fmt, ...) {
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(g_err, sizeof(g_err), fmt, ap);
  va_end(ap);
  return code;
}

int check_launch(const char *what, hipError_t e) {
  if (e == hipSuccess) e = hipGetLastError();
  if (e != hipSuccess) return fail(SPG_ERR_HIP, "%s: %s", what, hipGetErrorString(e));
  return SPG_OK;
}

int check_shape(const char *fn, int B, int H, int N, int D) {
  if (B <= 0 || H <= 0 || N <= 0) return fail(SPG_ERR_INVALID, "%s: B, H, N must be positive (got %d, %d, %d)", fn, B, H, N);
  if (D != 64 && D != 128) return fail(SPG_ERR_UNSUPPORTED, "%s: head_dim must be 64 or 128 (got %d)", fn, D);
  if ((double)B * H * (double)N * D >= 4294967296.0 * 4)
    return fail(SPG_ERR_UNSUPPORTED, "%s: tensor too large (B*H*N*D = %.0f)", fn, (double)B * H * (double)N * D);
  return SPG_OK;
}

int check_kv_heads(const char *fn, int H, int Hkv) {
  // the message of the reference (qk_int_sv_f8_cuda_sm89.cu:310-314)
  if (Hkv <= 0 || H % Hkv != 0)
    return fail(SPG_ERR_INVALID, "%s: num_qo_heads (%d) must be divisible by num_kv_heads (%d)", fn, H, Hkv);
  return SPG_OK;
}

int check_pv_mode(const char *fn, int mode) {
  if (mode < SPG_PV_NONE || mode > SPG_PV_PER_WARP)
    return fail(SPG_ERR_INVALID, "%s: pv_threshold_mode must be 0 (none), 1 (per block) or 2 (per 32 query rows), got %d", fn, mode);
  return SPG_OK;
}

// qk_quant_gran of the reference's kernel entry (csrc/pytorch_extensions_utils.cuh:71-85): 1 per block, 2 per warp,
// 3 per thread.  Per-thread scales follow the lane layout of mma.sync fragments and have no counterpart here.
int check_quant_gran(const char *fn, int gran) {
  if (gran == SPG_QUANT_PER_BLOCK || gran == SPG_QUANT_PER_WARP) return SPG_OK;
  if (gran == 3) return fail(SPG_ERR_UNSUPPORTED, "%s: qk_quant_gran 3 (per thread) is not supported on gfx950", fn);
  return fail(SPG_ERR_INVALID, "%s: Unsupported qk_quant_gran: %d", fn, gran);
}

int check_dtype(const char *fn, int dtype) {
  if (dtype != SPG_F16 && dtype != SPG_BF16) return fail(SPG_ERR_INVALID, "%s: dtype must be SPG_F16 or SPG_BF16 (got %d)", fn, dtype);
  return SPG_OK;
}

// strides == NULL: HND-contiguous.  Otherwise {batch, head, row} strides in elements; rows are read and written in
// 16-byte pieces, so every stride must be a multiple of 8 elements and a row must not overlap the next one.
int get_strides(const char *fn, const char *what, const int64_t *strides, int H, int N, int D, spg::Strides *out) {
  if (strides == nullptr) {
    out->sb = (long long)H * N * D; out->sh = (long long)N * D; out->sn = D;
    return SPG_OK;
  }
  for (int i = 0; i < 3; i++)
    if (strides[i] <= 0 || strides[i] % 8 != 0)
      return fail(SPG_ERR_INVALID, "%s: %s[%d] = %lld must be a positive multiple of 8 elements", fn, what, i, (long long)strides[i]);
  if (strides[2] < D) return fail(SPG_ERR_INVALID, "%s: %s[2] = %lld is smaller than head_dim %d", fn, what, (long long)strides[2], D);
  out->sb = strides[0]; out->sh = strides[1]; out->sn = strides[2];
  return SPG_OK;
}

#define SPG_TRY(expr) do { int rc_ = (expr); if (rc_ != SPG_OK) return rc_; } while (0)
#define SPG_NONNULL(fn, ptr) do { if ((ptr) == nullptr) return fail(SPG_ERR_INVALID, "%s: %s is NULL", fn, #ptr); } while (0)
}  // namespace

extern "C" {

int spg_version(void) { return 100; }

const char *spg_last_error(void) { return g_err; }

size_t spg_km_mean_workspace_bytes(int B, int H, int N, int D) {
  if (B <= 0 || H <= 0 || N <= 0 || D <= 0) return 0;
  return spg::km_mean_workspace_bytes(B, H, N, D);
}

int spg_km_mean(const void *k, const int64_t *k_strides, void *km, void *workspace, int B, int H, int N, int D, int dtype, void *stream) {
  const char *fn = "spg_km_mean";
  SPG_TRY(check_shape(fn, B, H, N, D));
  SPG_TRY(check_dtype(fn, dtype));
  SPG_NONNULL(fn, k); SPG_NONNULL(fn, km); SPG_NONNULL(fn, workspace);
  spg::Strides ks;
  SPG_TRY(get_strides(fn, "k_strides", k_strides, H, N, D, &ks));
  spg::launch_km_mean(k, ks, km, workspace, B, H, N, D, dtype, (hipStream_t)stream);
  return check_launch(fn, hipSuccess);
}

int spg_km_mean_static(const void *k, const int64_t *k_strides, void *km, int B, int H, int N, int D, int dtype, void *stream) {
  const char *fn = "spg_km_mean_static";
  SPG_TRY(check_shape(fn, B, H, N, D));
  SPG_TRY(check_dtype(fn, dtype));
  SPG_NONNULL(fn, k); SPG_NONNULL(fn, km);
  const size_t need = spg::km_mean_workspace_bytes(B, H, N, D);
  if (need > spg::km_mean_static_capacity())
    return fail(SPG_ERR_UNSUPPORTED, "%s: B=%d H=%d N=%d D=%d needs %zu bytes of scratch, the built-in array holds %zu "
                "(use spg_km_mean with a workspace of your own)", fn, B, H, N, D, need, spg::km_mean_static_capacity());
  spg::Strides ks;
  SPG_TRY(get_strides(fn, "k_strides", k_strides, H, N, D, &ks));
  const hipError_t e = spg::launch_km_mean_static(k, ks, km, B, H, N, D, dtype, (hipStream_t)stream);
  if (e == hipErrorInvalidDevice)
    return fail(SPG_ERR_INVALID, "%s: the stream's device must be the current device (the built-in array is per GPU)", fn);
  return check_launch(fn, e);
}

int spg_pool_sim_quant(const void *x, const int64_t *x_strides, const void *km, void *pool, uint8_t *sim, int8_t *xq, float *scale,
                       const float *simthreshd1, int B, int H, int N, int D, int block, int quant_rows, int dtype, void *stream) {
  const char *fn = "spg_pool_sim_quant";
  SPG_TRY(check_shape(fn, B, H, N, D));
  SPG_TRY(check_dtype(fn, dtype));
  if (block != 64 && block != 128) return fail(SPG_ERR_UNSUPPORTED, "%s: block must be 64 or 128 (got %d)", fn, block);
  if (quant_rows != block && !(quant_rows == 32 && block == 128 && km == nullptr))
    return fail(SPG_ERR_UNSUPPORTED, "%s: quant_rows must equal block (per-block scales), or be 32 with block = 128 and no "
                "mean (per-warp scales of Q); got quant_rows = %d, block = %d, km %s", fn, quant_rows, block,
                km == nullptr ? "NULL" : "given");
  SPG_NONNULL(fn, x); SPG_NONNULL(fn, xq); SPG_NONNULL(fn, scale);
  if ((pool == nullptr) != (sim == nullptr)) return fail(SPG_ERR_INVALID, "%s: pool and sim must both be given or both be NULL", fn);
  if (pool != nullptr) SPG_NONNULL(fn, simthreshd1);
  spg::Strides xs;
  SPG_TRY(get_strides(fn, "x_strides", x_strides, H, N, D, &xs));
  spg::launch_pool_sim_quant(x, xs, km, pool, sim, xq, scale, simthreshd1, B, H, N, D, block, quant_rows, dtype,
                             (hipStream_t)stream);
  return check_launch(fn, hipSuccess);
}

int spg_block_select(const void *pool_q, const uint8_t *sim_q, const void *pool_k, const uint8_t *sim_k,
                     const float *topk, const float *cdfthreshd, int is_causal, int attention_sink, int32_t *lut,
                     int32_t *valid_block_num, uint8_t *block_map, int B, int H, int Hkv, int nq, int nk, int D, int dtype,
                     void *stream) {
  const char *fn = "spg_block_select";
  if (B <= 0 || H <= 0 || nq <= 0 || nk <= 0) return fail(SPG_ERR_INVALID, "%s: B, H, nq, nk must be positive", fn);
  SPG_TRY(check_kv_heads(fn, H, Hkv));
  if (D != 64 && D != 128) return fail(SPG_ERR_UNSUPPORTED, "%s: head_dim must be 64 or 128 (got %d)", fn, D);
  SPG_TRY(check_dtype(fn, dtype));
  if ((topk == nullptr) == (cdfthreshd == nullptr))
    return fail(SPG_ERR_INVALID, "%s: Only one of cdfthreshd and topk can be set.", fn);
  if (nk > spg::block_select_max_nk())
    return fail(SPG_ERR_UNSUPPORTED, "%s: nk = %d exceeds the supported maximum %d", fn, nk, spg::block_select_max_nk());
  SPG_NONNULL(fn, pool_q); SPG_NONNULL(fn, sim_q); SPG_NONNULL(fn, pool_k); SPG_NONNULL(fn, sim_k);
  SPG_NONNULL(fn, lut); SPG_NONNULL(fn, valid_block_num);
  return check_launch(fn, spg::launch_block_select(pool_q, sim_q, pool_k, sim_k, topk, cdfthreshd, is_causal ? 1 : 0,
                                                   attention_sink ? 1 : 0, lut, valid_block_num, block_map, B, H, Hkv,
                                                   nq, nk, D, dtype, (hipStream_t)stream));
}

int spg_map_to_lut(const void *mask, int mask_kind, int32_t *lut, int32_t *valid_block_num, int B, int H, int nq,
                   int nk, void *stream) {
  const char *fn = "spg_map_to_lut";
  if (B <= 0 || H <= 0 || nq <= 0 || nk <= 0) return fail(SPG_ERR_INVALID, "%s: B, H, nq, nk must be positive", fn);
  if (mask_kind < SPG_MASK_I8 || mask_kind > SPG_MASK_F64) return fail(SPG_ERR_INVALID, "%s: bad mask_kind %d", fn, mask_kind);
  if (nk > 32768) return fail(SPG_ERR_UNSUPPORTED, "%s: nk = %d exceeds the supported maximum 32768", fn, nk);
  SPG_NONNULL(fn, mask); SPG_NONNULL(fn, lut); SPG_NONNULL(fn, valid_block_num);
  return check_launch(fn, spg::launch_map_to_lut(mask, mask_kind, lut, valid_block_num, B, H, nq, nk, (hipStream_t)stream));
}

int spg_selftest_division(unsigned long long *counts, int n_divisors, unsigned int seed, void *stream) {
  const char *fn = "spg_selftest_division";
  if (n_divisors <= 0 || n_divisors > (1 << 22)) return fail(SPG_ERR_INVALID, "%s: n_divisors must be in [1, 2^22]", fn);
  SPG_NONNULL(fn, counts);
  spg::launch_div_selftest(counts, n_divisors, seed, (hipStream_t)stream);
  return check_launch(fn, hipSuccess);
}

int spg_selftest_fp8_pack(const float *x, uint8_t *codes, int n, int saturate, void *stream) {
  const char *fn = "spg_selftest_fp8_pack";
  if (n <= 0 || n % 4 != 0) return fail(SPG_ERR_INVALID, "%s: n must be a positive multiple of 4 (got %d)", fn, n);
  SPG_NONNULL(fn, x); SPG_NONNULL(fn, codes);
  spg::launch_fp8_pack_selftest(x, codes, n, saturate ? 1 : 0, (hipStream_t)stream);
  return check_launch(fn, hipSuccess);
}

int spg_v_quant_fp8(const void *v, const int64_t *v_strides, uint8_t *v8, float *v_scale, int B, int H, int N, int D, int dtype, void *stream) {
  const char *fn = "spg_v_quant_fp8";
  SPG_TRY(check_shape(fn, B, H, N, D));
  SPG_TRY(check_dtype(fn, dtype));
  SPG_NONNULL(fn, v); SPG_NONNULL(fn, v8); SPG_NONNULL(fn, v_scale);
  spg::Strides vs;
  SPG_TRY(get_strides(fn, "v_strides", v_strides, H, N, D, &vs));
  spg::launch_v_quant_fp8(v, vs, v8, v_scale, B, H, N, D, dtype, (hipStream_t)stream);
  return check_launch(fn, hipSuccess);
}

int spg_block_sparse_attn(const int8_t *q8, const int8_t *k8, const uint8_t *v8, void *out, const int64_t *out_strides,
                          int out_dtype,
                          const int32_t *lut, const int32_t *valid_block_num, const float *pvthreshd,
                          const float *q_scale, const float *k_scale, const float *v_scale, int B, int H, int Hkv, int N,
                          int N_kv, int D, float sm_scale, int is_causal, int qk_quant_gran, int pv_threshold_mode,
                          int32_t *pv_count, void *stream) {
  const char *fn = "spg_block_sparse_attn";
  SPG_TRY(check_shape(fn, B, H, N, D));
  SPG_TRY(check_shape(fn, B, Hkv > 0 ? Hkv : 1, N_kv, D));
  SPG_TRY(check_kv_heads(fn, H, Hkv));
  SPG_TRY(check_quant_gran(fn, qk_quant_gran));
  SPG_TRY(check_pv_mode(fn, pv_threshold_mode));
  SPG_TRY(check_dtype(fn, out_dtype));
  SPG_NONNULL(fn, q8); SPG_NONNULL(fn, k8); SPG_NONNULL(fn, v8); SPG_NONNULL(fn, out); SPG_NONNULL(fn, lut);
  SPG_NONNULL(fn, valid_block_num); SPG_NONNULL(fn, pvthreshd); SPG_NONNULL(fn, q_scale); SPG_NONNULL(fn, k_scale);
  SPG_NONNULL(fn, v_scale);
  spg::Strides os;
  SPG_TRY(get_strides(fn, "out_strides", out_strides, H, N, D, &os));
  return check_launch(fn, spg::launch_block_sparse_attn(q8, k8, v8, out, os, out_dtype, lut, valid_block_num, pvthreshd,
                                                        q_scale, k_scale, v_scale, B, H, Hkv, N, N_kv, D, sm_scale,
                                                        is_causal ? 1 : 0, qk_quant_gran == SPG_QUANT_PER_WARP ? 1 : 0,
                                                        pv_threshold_mode, pv_count, (hipStream_t)stream));
}

int spg_v_tiles_f16(const void *v, const int64_t *v_strides, void *vt, int B, int H, int N, int D, int dtype, void *stream) {
  const char *fn = "spg_v_tiles_f16";
  SPG_TRY(check_shape(fn, B, H, N, D));
  SPG_TRY(check_dtype(fn, dtype));
  SPG_NONNULL(fn, v); SPG_NONNULL(fn, vt);
  spg::Strides vs;
  SPG_TRY(get_strides(fn, "v_strides", v_strides, H, N, D, &vs));
  spg::launch_v_tiles_f16(v, vs, vt, B, H, N, D, dtype, (hipStream_t)stream);
  return check_launch(fn, hipSuccess);
}

int spg_block_sparse_attn_f16v(const int8_t *q8, const int8_t *k8, const void *vt, void *out, const int64_t *out_strides,
                               int out_dtype,
                               const int32_t *lut, const int32_t *valid_block_num, const float *pvthreshd,
                               const float *q_scale, const float *k_scale, int B, int H, int Hkv, int N, int N_kv, int D,
                               float sm_scale, int is_causal, int qk_quant_gran, int pv_threshold_mode, int32_t *pv_count,
                               void *stream) {
  const char *fn = "spg_block_sparse_attn_f16v";
  SPG_TRY(check_shape(fn, B, H, N, D));
  SPG_TRY(check_shape(fn, B, Hkv > 0 ? Hkv : 1, N_kv, D));
  SPG_TRY(check_kv_heads(fn, H, Hkv));
  SPG_TRY(check_quant_gran(fn, qk_quant_gran));
  SPG_TRY(check_pv_mode(fn, pv_threshold_mode));
  SPG_TRY(check_dtype(fn, out_dtype));
  SPG_NONNULL(fn, q8); SPG_NONNULL(fn, k8); SPG_NONNULL(fn, vt); SPG_NONNULL(fn, out); SPG_NONNULL(fn, lut);
  SPG_NONNULL(fn, valid_block_num); SPG_NONNULL(fn, pvthreshd); SPG_NONNULL(fn, q_scale); SPG_NONNULL(fn, k_scale);
  spg::Strides os;
  SPG_TRY(get_strides(fn, "out_strides", out_strides, H, N, D, &os));
  return check_launch(fn, spg::launch_block_sparse_attn(q8, k8, (const uint8_t *)vt, out, os, out_dtype, lut, valid_block_num,
                                                        pvthreshd, q_scale, k_scale, nullptr, B, H, Hkv, N, N_kv, D, sm_scale,
                                                        is_causal ? 1 : 0, qk_quant_gran == SPG_QUANT_PER_WARP ? 1 : 0,
                                                        pv_threshold_mode, pv_count, (hipStream_t)stream));
}

int spg_dense_attn_f16(const void *q, const void *k, const void *v, void *out, int B, int H, int N, int D,
                       float sm_scale, int is_causal, void *stream) {
  const char *fn = "spg_dense_attn_f16";
  SPG_TRY(check_shape(fn, B, H, N, D));
  SPG_NONNULL(fn, q); SPG_NONNULL(fn, k); SPG_NONNULL(fn, v); SPG_NONNULL(fn, out);
  return check_launch(fn, spg::launch_dense_attn_f16(q, k, v, out, B, H, N, D, sm_scale, is_causal ? 1 : 0,
                                                     (hipStream_t)stream));
}

}  // extern "C"
