// Host-side launch functions shared between the kernel translation units and the C ABI (capi.hip).
#pragma once
#include <hip/hip_runtime.h>
#include <stddef.h>
#include <stdint.h>

namespace spg {

// Element strides of a (B, H, N, D) tensor whose last dimension is contiguous: element (b, h, n, d) sits at
// b*sb + h*sh + n*sn + d.  HND-contiguous: {H*N*D, N*D, D}; NHD-contiguous (B, N, H, D in memory): {N*H*D, D, H*D}.
struct Strides {
  long long sb, sh, sn;
};

size_t km_mean_workspace_bytes(int B, int H, int N, int D);
void launch_km_mean(const void *k, Strides ks, void *km, void *ws, int B, int H, int N, int D, int dtype, hipStream_t st);
// size of the library-owned scratch array behind launch_km_mean_static (bytes); a shape whose
// km_mean_workspace_bytes() exceeds it is refused by the caller
#define SPG_KM_STATIC_SCRATCH_BYTES (8u << 20)
size_t km_mean_static_capacity();
hipError_t launch_km_mean_static(const void *k, Strides ks, void *km, int B, int H, int N, int D, int dtype, hipStream_t st);
void launch_pool_sim_quant(const void *x, Strides xs, const void *km, void *pool, uint8_t *sim, int8_t *xq, float *scale,
                           const float *thr, int B, int H, int N, int D, int block, int quant_rows, int dtype,
                           hipStream_t st);
int block_select_max_nk();
hipError_t launch_block_select(const void *pq, const uint8_t *sq, const void *pk, const uint8_t *sk, const float *topk,
                               const float *cdf, int causal, int sink, int32_t *lut, int32_t *valid, uint8_t *bmap,
                               int B, int H, int Hkv, int nq, int nk, int D, int dtype, hipStream_t st);
void launch_div_selftest(unsigned long long *counts, int n_div, uint32_t seed, hipStream_t st);
hipError_t launch_map_to_lut(const void *mask, int kind, int32_t *lut, int32_t *valid, int B, int H, int nq, int nk,
                             hipStream_t st);

void launch_v_quant_fp8(const void *v, Strides vs, uint8_t *v8, float *v_scale, int B, int H, int N, int D, int dtype,
                        hipStream_t st);

void launch_v_tiles_f16(const void *v, Strides vs, void *vt, int B, int H, int N, int D, int dtype, hipStream_t st);

hipError_t launch_block_sparse_attn(const int8_t *q8, const int8_t *k8, const uint8_t *v8, void *out, Strides os,
                                    int out_dtype,
                                    const int32_t *lut, const int32_t *valid, const float *pvthreshd,
                                    const float *q_scale, const float *k_scale, const float *v_scale, int B, int H,
                                    int Hkv, int N, int Nk, int D, float sm_scale, int is_causal, int q_per_warp,
                                    int pv_mode, int32_t *pv_count, hipStream_t st);
void launch_fp8_pack_selftest(const float *x, uint8_t *codes, int n, int saturate, hipStream_t st);

hipError_t launch_dense_attn_f16(const void *q, const void *k, const void *v, void *out, int B, int H, int N, int D,
                                 float sm_scale, int is_causal, hipStream_t st);

}  // namespace spg
