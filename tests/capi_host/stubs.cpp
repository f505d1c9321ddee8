// Host-only stand-ins for the kernel launchers declared in spargeattn_amd/csrc/launch.h, so that the argument
// validation of capi.hip can be linked and run under AddressSanitizer / UBSan on a machine without a GPU.
// Every function records that it was reached: the checks in check.cpp only make calls that must be refused before.
#include "launch.h"

namespace spg {
int g_launches = 0;
size_t km_mean_workspace_bytes(int B, int H, int N, int D) { return (size_t)B * H * ((N + 255) / 256) * D * 8; }
void launch_km_mean(const void *, Strides, void *, void *, int, int, int, int, int, hipStream_t) { g_launches++; }
size_t km_mean_static_capacity() { return SPG_KM_STATIC_SCRATCH_BYTES; }
hipError_t launch_km_mean_static(const void *, Strides, void *, int, int, int, int, int, hipStream_t) { g_launches++; return hipSuccess; }
void launch_pool_sim_quant(const void *, Strides, const void *, void *, uint8_t *, int8_t *, float *, const float *, int,
                           int, int, int, int, int, int, hipStream_t) { g_launches++; }
int block_select_max_nk() { return 8192; }
hipError_t launch_block_select(const void *, const uint8_t *, const void *, const uint8_t *, const float *, const float *,
                               int, int, int32_t *, int32_t *, uint8_t *, int, int, int, int, int, int, int, hipStream_t) { g_launches++; return hipSuccess; }
void launch_div_selftest(unsigned long long *, int, uint32_t, hipStream_t) { g_launches++; }
hipError_t launch_map_to_lut(const void *, int, int32_t *, int32_t *, int, int, int, int, hipStream_t) { g_launches++; return hipSuccess; }
void launch_v_quant_fp8(const void *, Strides, uint8_t *, float *, int, int, int, int, int, hipStream_t) { g_launches++; }
void launch_v_tiles_f16(const void *, Strides, void *, int, int, int, int, int, hipStream_t) { g_launches++; }
hipError_t launch_block_sparse_attn(const int8_t *, const int8_t *, const uint8_t *, void *, Strides, int, const int32_t *,
                                    const int32_t *, const float *, const float *, const float *, const float *, int, int,
                                    int, int, int, int, float, int, int, int, int32_t *, hipStream_t) { g_launches++; return hipSuccess; }
void launch_fp8_pack_selftest(const float *, uint8_t *, int, int, hipStream_t) { g_launches++; }
hipError_t launch_dense_attn_f16(const void *, const void *, const void *, void *, int, int, int, int, float, int,
                                 hipStream_t) { g_launches++; return hipSuccess; }
}  // namespace spg
