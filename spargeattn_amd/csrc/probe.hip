// Measurement aids (no counterpart in the reference): what this machine delivers for the access shapes of the streaming
// kernels, and how matrix and vector instructions share a SIMD.  The figures the design notes quote for both come from
// these kernels (bench.py --stream-calibration, --issue-calibration).
#include "common.h"
#include "launch.h"

namespace spg {

// Streaming probe: nothing but the loads and stores of the streaming kernels' access shapes.  mode 0: read 16 B per lane with the non-temporal hint; mode 1: the same with plain loads; mode 2:
// read 16 B (non-temporal) and write 8 B per lane (the 2-bytes-in, 1-byte-out shape of the quantisation kernels).  One
// workgroup per 32 KiB of input.
template <int MODE>
__global__ __launch_bounds__(256) void stream_probe_kernel(const uint4 *__restrict__ src, uint2 *__restrict__ dst,
                                                           uint32_t *__restrict__ sink) {
  const size_t base = (size_t)blockIdx.x * 2048;
  uint4 v[8];
#pragma unroll
  for (int u = 0; u < 8; u++) {
    const uint4 *a = src + base + threadIdx.x + u * 256;
    v[u] = MODE == 1 ? *a : load_stream_u4(a);
  }
  uint32_t acc = 0;
#pragma unroll
  for (int u = 0; u < 8; u++) {
    if constexpr (MODE == 2) dst[base + threadIdx.x + u * 256] = make_uint2(v[u].x ^ v[u].y, v[u].z ^ v[u].w);
    else acc ^= v[u].x ^ v[u].y ^ v[u].z ^ v[u].w;
  }
  if (MODE != 2 && acc == 0x9e3779b9u) sink[0] = acc;      // keeps the loads alive; practically never true
}
void launch_stream_probe(const void *src, void *dst, void *sink, size_t bytes, int mode, hipStream_t st) {
  const int grid = (int)(bytes / 32768);
  if (mode == 0) stream_probe_kernel<0><<<grid, 256, 0, st>>>((const uint4 *)src, (uint2 *)dst, (uint32_t *)sink);
  else if (mode == 1) stream_probe_kernel<1><<<grid, 256, 0, st>>>((const uint4 *)src, (uint2 *)dst, (uint32_t *)sink);
  else stream_probe_kernel<2><<<grid, 256, 0, st>>>((const uint4 *)src, (uint2 *)dst, (uint32_t *)sink);
}


// Issue probe: every wavefront repeats "one MFMA, then NV independent v_add_f32" (two accumulator chains, so that
// consecutive MFMAs do not wait for each other).  With the vector adds hidden behind the matrix pipe the time per
// repetition would be max(MFMA, adds); what is measured is close to their sum.
// KIND 0: v_mfma_i32_32x32x32_i8, 1: v_mfma_f32_32x32x64_f8f6f4 (fp8 operands), 2: v_mfma_f32_32x32x16_f16.
typedef int pv4i __attribute__((ext_vector_type(4)));
typedef int pv8i __attribute__((ext_vector_type(8)));
typedef int pv16i __attribute__((ext_vector_type(16)));
typedef float pv16f __attribute__((ext_vector_type(16)));
typedef _Float16 pv8h __attribute__((ext_vector_type(8)));
template <int KIND, int NV>
__global__ __launch_bounds__(256) void issue_probe_kernel(float *__restrict__ out, float seed, int reps) {
  const pv4i a = {1, 2, 3, (int)threadIdx.x}, b = {4, 5, 6, 7};
  const pv8i a8 = {1, 2, 3, 4, 5, 6, 7, (int)threadIdx.x}, b8 = {1, 1, 1, 1, 1, 1, 1, 1};
  const pv8h ah = {(_Float16)1, (_Float16)2, (_Float16)3, (_Float16)4, (_Float16)5, (_Float16)6, (_Float16)7, (_Float16)(int)(threadIdx.x & 7)};
  const pv8h bh = {(_Float16)1, (_Float16)1, (_Float16)1, (_Float16)1, (_Float16)1, (_Float16)1, (_Float16)1, (_Float16)1};
  pv16i c0 = {0}, c1 = {0};
  pv16f f0 = {0}, f1 = {0};
  float x[8];
#pragma unroll
  for (int i = 0; i < 8; i++) x[i] = seed + i;
  for (int it = 0; it < reps; it++) {
#pragma unroll
    for (int u = 0; u < 4; u++) {
      if constexpr (KIND == 0) {
        if (u & 1) c1 = __builtin_amdgcn_mfma_i32_32x32x32_i8(a, b, c1, 0, 0, 0);
        else c0 = __builtin_amdgcn_mfma_i32_32x32x32_i8(a, b, c0, 0, 0, 0);
      } else if constexpr (KIND == 1) {
        if (u & 1) f1 = __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(a8, b8, f1, 0, 0, 0, 0, 0, 0);
        else f0 = __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(a8, b8, f0, 0, 0, 0, 0, 0, 0);
      } else {
        if (u & 1) f1 = __builtin_amdgcn_mfma_f32_32x32x16_f16(ah, bh, f1, 0, 0, 0);
        else f0 = __builtin_amdgcn_mfma_f32_32x32x16_f16(ah, bh, f0, 0, 0, 0);
      }
#pragma unroll
      for (int v = 0; v < NV; v++) asm volatile("v_add_f32 %0, %0, %1" : "+v"(x[v & 7]) : "v"(x[(v + 1) & 7]));
    }
  }
  float s = 0.f;
#pragma unroll
  for (int i = 0; i < 8; i++) s += x[i];
#pragma unroll
  for (int i = 0; i < 16; i++) s += (float)(c0[i] + c1[i]) + f0[i] + f1[i];
  out[blockIdx.x * 256 + threadIdx.x] = s;
}
template <int KIND>
static bool launch_issue_kind(float *out, int nv, int reps, int blocks, hipStream_t st) {
  switch (nv) {
    case 0: issue_probe_kernel<KIND, 0><<<blocks, 256, 0, st>>>(out, 0.5f, reps); return true;
    case 8: issue_probe_kernel<KIND, 8><<<blocks, 256, 0, st>>>(out, 0.5f, reps); return true;
    case 16: issue_probe_kernel<KIND, 16><<<blocks, 256, 0, st>>>(out, 0.5f, reps); return true;
    case 32: issue_probe_kernel<KIND, 32><<<blocks, 256, 0, st>>>(out, 0.5f, reps); return true;
    case 64: issue_probe_kernel<KIND, 64><<<blocks, 256, 0, st>>>(out, 0.5f, reps); return true;
    default: return false;
  }
}
// out: blocks * 256 floats.  blocks = CUs * wavefronts per SIMD gives every SIMD that many wavefronts.
bool launch_issue_probe(float *out, int kind, int nv, int reps, int blocks, hipStream_t st) {
  if (kind == 0) return launch_issue_kind<0>(out, nv, reps, blocks, st);
  if (kind == 1) return launch_issue_kind<1>(out, nv, reps, blocks, st);
  if (kind == 2) return launch_issue_kind<2>(out, nv, reps, blocks, st);
  return false;
}

}  // namespace spg
