// Runs the host-side argument validation of the C ABI (spargeattn_amd/csrc/capi.hip) with bad arguments of every kind.
// Built with -fsanitize=address,undefined by tests/test_capi_sanitized.py: a validation path that reads a stride array
// out of bounds, formats a message past its buffer or overflows a size computation fails the run.  No GPU is touched:
// every call here must be refused before a launch (spg::g_launches stays 0).
#include "../../include/spargeattn_amd.h"

#include <cstdio>
#include <cstring>

namespace spg { extern int g_launches; }

static int failures = 0;
#define EXPECT(rc, code, needle)                                                                         \
  do {                                                                                                   \
    const int rc_ = (rc);                                                                                \
    if (rc_ != (code) || std::strstr(spg_last_error(), (needle)) == nullptr) {                           \
      std::printf("line %d: rc %d (want %d), message '%s' (want '%s')\n", __LINE__, rc_, (int)(code), spg_last_error(), (needle)); \
      failures++;                                                                                        \
    }                                                                                                    \
  } while (0)

int main() {
  void *p = (void *)0x1000;                 // never dereferenced: every call below is refused on its arguments
  const float *fp = (const float *)p;
  int8_t *i8 = (int8_t *)p;
  uint8_t *u8 = (uint8_t *)p;
  int32_t *i32 = (int32_t *)p;
  int64_t bad_mult[3] = {128 * 64, 64, 60}, bad_small[3] = {128 * 64, 128 * 64, 32}, neg[3] = {-8, 64, 64};
  int64_t huge[3] = {INT64_MAX - 7, 8, 64};

  EXPECT(spg_km_mean(nullptr, nullptr, nullptr, nullptr, 1, 1, 128, 96, 0, nullptr), SPG_ERR_UNSUPPORTED, "head_dim");
  EXPECT(spg_km_mean(p, nullptr, p, p, 0, 1, 128, 64, 0, nullptr), SPG_ERR_INVALID, "must be positive");
  EXPECT(spg_km_mean(p, nullptr, p, p, 65536, 65536, 1 << 30, 128, 0, nullptr), SPG_ERR_UNSUPPORTED, "too large");
  EXPECT(spg_km_mean(p, nullptr, p, nullptr, 1, 1, 128, 64, 0, nullptr), SPG_ERR_INVALID, "NULL");
  EXPECT(spg_km_mean(p, bad_mult, p, p, 1, 1, 128, 64, 0, nullptr), SPG_ERR_INVALID, "multiple of 8");
  EXPECT(spg_km_mean(p, bad_small, p, p, 1, 1, 128, 64, 0, nullptr), SPG_ERR_INVALID, "smaller than head_dim");
  EXPECT(spg_km_mean(p, neg, p, p, 1, 1, 128, 64, 0, nullptr), SPG_ERR_INVALID, "positive multiple");
  EXPECT(spg_km_mean(p, huge, p, p, 1, 1, 128, 64, 7, nullptr), SPG_ERR_INVALID, "dtype");
  EXPECT(spg_km_mean_static(p, nullptr, p, 1, 8193, 128, 128, 0, nullptr), SPG_ERR_UNSUPPORTED, "scratch");
  if (spg_km_mean_workspace_bytes(-1, 1, 1, 1) != 0 || spg_km_mean_workspace_bytes(1, 32, 32768, 128) == 0) failures++;

  EXPECT(spg_pool_sim_quant(nullptr, nullptr, nullptr, nullptr, nullptr, nullptr, nullptr, nullptr, 1, 1, 128, 64, 128, 128, 1, nullptr),
         SPG_ERR_INVALID, "NULL");
  EXPECT(spg_pool_sim_quant(p, nullptr, nullptr, p, nullptr, i8, (float *)p, fp, 1, 1, 128, 64, 128, 128, 1, nullptr),
         SPG_ERR_INVALID, "both be given");
  EXPECT(spg_pool_sim_quant(p, nullptr, nullptr, nullptr, nullptr, i8, (float *)p, nullptr, 1, 1, 128, 64, 96, 96, 1, nullptr),
         SPG_ERR_UNSUPPORTED, "block must be");
  EXPECT(spg_pool_sim_quant(p, nullptr, nullptr, nullptr, nullptr, i8, (float *)p, nullptr, 1, 1, 128, 64, 64, 32, 1, nullptr),
         SPG_ERR_UNSUPPORTED, "quant_rows");
  EXPECT(spg_pool_sim_quant(p, nullptr, p, nullptr, nullptr, i8, (float *)p, nullptr, 1, 1, 128, 64, 128, 32, 1, nullptr),
         SPG_ERR_UNSUPPORTED, "quant_rows");

  EXPECT(spg_block_select(p, u8, p, u8, nullptr, nullptr, 0, 0, i32, i32, nullptr, 1, 1, 1, 1, 2, 64, 0, nullptr), SPG_ERR_INVALID,
         "Only one of cdfthreshd and topk");
  EXPECT(spg_block_select(p, u8, p, u8, fp, fp, 0, 0, i32, i32, nullptr, 1, 1, 1, 1, 2, 64, 0, nullptr), SPG_ERR_INVALID,
         "Only one of cdfthreshd and topk");
  EXPECT(spg_block_select(p, u8, p, u8, fp, nullptr, 0, 0, i32, i32, nullptr, 1, 6, 4, 1, 2, 64, 0, nullptr), SPG_ERR_INVALID,
         "must be divisible by num_kv_heads");
  EXPECT(spg_block_select(p, u8, p, u8, fp, nullptr, 0, 0, i32, i32, nullptr, 1, 6, 0, 1, 2, 64, 0, nullptr), SPG_ERR_INVALID,
         "must be divisible by num_kv_heads");
  EXPECT(spg_block_select(p, u8, p, u8, fp, nullptr, 0, 0, i32, i32, nullptr, 1, 4, 4, 1, 8193, 64, 0, nullptr), SPG_ERR_UNSUPPORTED,
         "exceeds the supported maximum");
  EXPECT(spg_map_to_lut(p, 9, i32, i32, 1, 1, 1, 1, nullptr), SPG_ERR_INVALID, "bad mask_kind");
  EXPECT(spg_map_to_lut(p, 0, i32, i32, 1, 1, 1, 40000, nullptr), SPG_ERR_UNSUPPORTED, "exceeds the supported maximum");

  EXPECT(spg_v_quant_fp8(p, nullptr, u8, (float *)p, 1, 1, 128, 64, 7, nullptr), SPG_ERR_INVALID, "dtype");
  EXPECT(spg_v_quant_fp8(p, bad_mult, u8, (float *)p, 1, 1, 128, 64, 0, nullptr), SPG_ERR_INVALID, "multiple of 8");
  EXPECT(spg_v_tiles_f16(p, bad_small, p, 1, 1, 128, 64, 0, nullptr), SPG_ERR_INVALID, "smaller than head_dim");

  for (int f16v = 0; f16v < 2; f16v++) {
    auto attn = [&](int H, int Hkv, int N, int Nkv, int D, int gran, int pv) {
      return f16v ? spg_block_sparse_attn_f16v(i8, i8, p, p, nullptr, 0, i32, i32, fp, fp, fp, 1, H, Hkv, N, Nkv, D, 0.125f, 0,
                                                gran, pv, nullptr, nullptr)
                  : spg_block_sparse_attn(i8, i8, u8, p, nullptr, 0, i32, i32, fp, fp, fp, fp, 1, H, Hkv, N, Nkv, D, 0.125f, 0, gran,
                                          pv, nullptr, nullptr);
    };
    EXPECT(attn(6, 4, 128, 128, 64, 1, 1), SPG_ERR_INVALID, "must be divisible by num_kv_heads");
    EXPECT(attn(4, 4, 128, 128, 64, 1, 3), SPG_ERR_INVALID, "pv_threshold_mode");
    EXPECT(attn(4, 4, 128, 0, 64, 1, 1), SPG_ERR_INVALID, "must be positive");
    EXPECT(attn(4, 4, 128, 128, 80, 1, 1), SPG_ERR_UNSUPPORTED, "head_dim");
    EXPECT(attn(4, 4, 128, 128, 64, 3, 1), SPG_ERR_UNSUPPORTED, "per thread");
    EXPECT(attn(4, 4, 128, 128, 64, 0, 1), SPG_ERR_INVALID, "Unsupported qk_quant_gran: 0");
    EXPECT(attn(4, 4, 128, 128, 64, -7, 1), SPG_ERR_INVALID, "Unsupported qk_quant_gran: -7");
  }
  EXPECT(spg_block_sparse_attn(i8, i8, u8, p, neg, 0, i32, i32, fp, fp, fp, fp, 1, 4, 4, 128, 128, 64, 0.125f, 0, 1, 1, nullptr, nullptr),
         SPG_ERR_INVALID, "positive multiple");
  EXPECT(spg_dense_attn_f16(p, p, nullptr, p, 1, 1, 128, 64, 0.125f, 0, nullptr), SPG_ERR_INVALID, "NULL");
  EXPECT(spg_selftest_fp8_pack(fp, u8, 6, 1, nullptr), SPG_ERR_INVALID, "multiple of 4");
  EXPECT(spg_selftest_division(nullptr, 16, 1, nullptr), SPG_ERR_INVALID, "NULL");
  EXPECT(spg_selftest_division((unsigned long long *)p, 0, 1, nullptr), SPG_ERR_INVALID, "n_divisors");

  if (spg::g_launches != 0) { std::printf("a refused call reached a launcher (%d)\n", spg::g_launches); failures++; }
  if (spg_version() < 100) failures++;
  std::printf(failures ? "FAILED (%d)\n" : "capi host checks ok\n", failures);
  return failures ? 1 : 0;
}
