// V path for gfx950: fp16 cast, per-(b,h,channel) absmax, FP8 e4m3 quantisation written straight into the
// [B][H][nk][D][64] tile layout the attention kernel's V^T operand reads.  Inside a 64-byte tile row (one channel,
// 64 keys) the four 16-key chunks are stored XOR-swizzled: key chunk kc sits at slot kc ^ ((d >> 2) & 3), which is
// the LDS bank-conflict swizzle of the attention kernel baked into the HBM layout (a tile is copied to LDS verbatim).
// Replaces TransposePadPermuteKernel + MeanScaleKernel (csrc/fused/fused.cu:26-77, 80-191) called with
// scale_max = 2.25 (spas_sage_attn/core.py:147-151).  HBM-bound: V is read twice (absmax, quantise), written once
// at 1 B/element.  Compile with -ffp-contract=off.
#include "common.h"
#include "launch.h"

namespace spg {

template <int DT>
__device__ __forceinline__ float elem_to_f16_f32(uint16_t b) {
  // value of the element after the cast to fp16 the reference applies to V (core.py:117)
  if constexpr (DT == 0) return elem_to_f32<0>(b);
  const _Float16 h = (_Float16)elem_to_f32<1>(b);
  return (float)h;
}

__global__ void fill_u32_kernel(uint32_t *p, uint32_t v, int n) {
  const int i = blockIdx.x * blockDim.x + threadIdx.x;
  if (i < n) p[i] = v;
}

template <int D, int DT>
__global__ __launch_bounds__(256) void v_absmax_kernel(const uint16_t *__restrict__ v, const Strides vs, int H,
                                                       uint32_t *__restrict__ amax_bits, int N, int rows_per_chunk) {
  constexpr int TPR = D / 8;
  constexpr int RPP = 256 / TPR;
  const int bh = blockIdx.y, chunk = blockIdx.x;
  const int c = threadIdx.x % TPR, r = threadIdx.x / TPR;
  const int row0 = chunk * rows_per_chunk;
  const int row1 = min(N, row0 + rows_per_chunk);
  const uint16_t *base = v + (size_t)(bh / H) * vs.sb + (size_t)(bh % H) * vs.sh + c * 8;
  // The cast to fp16 is monotonic in the magnitude, so the largest |fp16(v)| is the cast of the largest |v|: the maximum
  // is taken on the 16-bit magnitude patterns (which order like the magnitudes), two per instruction, and only the
  // result is converted.
  typedef unsigned short u16x2_t __attribute__((ext_vector_type(2)));
  constexpr uint32_t INF16 = DT == 1 ? 0x7f80u : 0x7c00u;
  uint32_t mp[4] = {0, 0, 0, 0};
#pragma unroll 4
  for (int row = row0 + r; row < row1; row += RPP) {
    const uint4 q = load_stream_u4(base + (size_t)row * vs.sn);
    const uint32_t w[4] = {q.x, q.y, q.z, q.w};
#pragma unroll
    for (int j = 0; j < 4; j++)
      mp[j] = __builtin_bit_cast(uint32_t, __builtin_elementwise_max(__builtin_bit_cast(u16x2_t, mp[j]),
                                                                      __builtin_bit_cast(u16x2_t, w[j] & 0x7fff7fffu)));
  }
  // A NaN pattern lies above the infinity pattern and would win the maximum, whereas the reference's fmaxf / fminf
  // (fused.cu:120-123) ignore NaN: only the NaN elements themselves are poisoned, not their channel's scale.  The
  // common case pays one test; a thread that met a NaN goes over its rows again with the NaN patterns taken as zero.
  if (max(max(mp[0] & 0xffffu, mp[0] >> 16), max(mp[1] & 0xffffu, mp[1] >> 16)) > INF16 ||
      max(max(mp[2] & 0xffffu, mp[2] >> 16), max(mp[3] & 0xffffu, mp[3] >> 16)) > INF16) {
    mp[0] = mp[1] = mp[2] = mp[3] = 0;
    for (int row = row0 + r; row < row1; row += RPP) {
      const uint4 q = *(const uint4 *)(base + (size_t)row * vs.sn);
      const uint32_t w[4] = {q.x, q.y, q.z, q.w};
#pragma unroll
      for (int j = 0; j < 4; j++) {
        uint32_t lo = w[j] & 0x7fffu, hi = (w[j] >> 16) & 0x7fffu;
        lo = lo > INF16 ? 0u : lo;
        hi = hi > INF16 ? 0u : hi;
        mp[j] = max(mp[j] & 0xffffu, lo) | (max(mp[j] >> 16, hi) << 16);
      }
    }
  }
  float m[8];
#pragma unroll
  for (int e = 0; e < 8; e++)
    m[e] = elem_to_f16_f32<DT>((uint16_t)((e & 1) ? (mp[e >> 1] >> 16) : (mp[e >> 1] & 0xffffu)));
  __shared__ float sm[RPP][D];
#pragma unroll
  for (int e = 0; e < 8; e++) sm[r][c * 8 + e] = m[e];
  __syncthreads();
  if (threadIdx.x < D) {
    float s = 0.f;
    for (int i = 0; i < RPP; i++) s = fmaxf(s, sm[i][threadIdx.x]);
    // non-negative floats order like their bit patterns; max is order independent
    atomicMax(amax_bits + (size_t)bh * D + threadIdx.x, __builtin_bit_cast(uint32_t, s));
  }
}

// One workgroup per 64-key tile.  LDS holds the transposed tile [D][64] bytes.
template <int D, int DT>
__global__ __launch_bounds__(256) void v_quant_kernel(const uint16_t *__restrict__ v, const Strides vs, int H,
                                                      const float *__restrict__ amax, uint8_t *__restrict__ v8, int N, int nk) {
  constexpr int TPR = D / 8;
  constexpr int RPP = 256 / TPR;
  constexpr int NP = 64 / RPP;
  constexpr int LDW = 64 + 4;  // padded row (bytes) of the transposed tile
  __shared__ __align__(16) uint8_t tile[D * LDW];
  const int blk = blockIdx.x, bh = blockIdx.y, tid = threadIdx.x;
  const int c = tid % TPR, r = tid / TPR;
  float recp[8];
#pragma unroll
  for (int e = 0; e < 8; e++) recp[e] = 2.25f / amax[(size_t)bh * D + c * 8 + e];
  const uint16_t *base = v + (size_t)(bh / H) * vs.sb + (size_t)(bh % H) * vs.sh + (size_t)blk * 64 * vs.sn + c * 8;
  const int last_row = min(63, N - 1 - blk * 64);
  uint4 raw[NP];                     // every load is issued before the first use; rows beyond N re-read the last row
#pragma unroll
  for (int p = 0; p < NP; p++) raw[p] = load_stream_u4(base + (size_t)min(r + p * RPP, last_row) * vs.sn);
#pragma unroll
  for (int p = 0; p < NP; p++) {
    const int row = r + p * RPP;
    const bool ok = row <= last_row;
    const uint4 q = raw[p];
    const uint32_t w[4] = {q.x, q.y, q.z, q.w};
#pragma unroll
    for (int e = 0; e < 8; e += 2) {
      const float a = elem_to_f16_f32<DT>((uint16_t)(w[e >> 1] & 0xffffu)) * recp[e];
      const float b = elem_to_f16_f32<DT>((uint16_t)(w[e >> 1] >> 16)) * recp[e + 1];
      const int pk = ok ? __builtin_amdgcn_cvt_pk_fp8_f32(a, b, 0, false) : 0;   // rows beyond N are zero
      tile[(c * 8 + e) * LDW + row] = (uint8_t)(pk & 0xff);
      tile[(c * 8 + e + 1) * LDW + row] = (uint8_t)((pk >> 8) & 0xff);
    }
  }
  __syncthreads();
  uint8_t *out = v8 + ((size_t)bh * nk + blk) * (size_t)(D * 64);
  for (int i = tid; i < D * 4; i += 256) {   // 16-byte pieces: D rows x 4 slots
    const int d = i >> 2, slot = i & 3;
    const int kc = slot ^ ((d >> 2) & 3);      // key chunk stored in this slot
    const uint32_t *src = (const uint32_t *)(tile + d * LDW + kc * 16);
    *(uint4 *)(out + d * 64 + slot * 16) = make_uint4(src[0], src[1], src[2], src[3]);
  }
}

// V -> fp16 -> V^T tiles [nk][D][64] fp16 for the fp16-PV attention variant.  Inside a 128-byte tile row (one channel,
// 64 keys) the eight 8-key chunks are stored at slot = chunk ^ ((d >> 1) & 7) (the LDS swizzle of the attention kernel).
// Keys at or beyond N are zero.  One workgroup per 64-key tile.
template <int D, int DT>
__global__ __launch_bounds__(256) void v_tiles_f16_kernel(const uint16_t *__restrict__ v, const Strides vs, int H,
                                                          uint16_t *__restrict__ vt, int N, int nk) {
  constexpr int TPR = D / 8;
  constexpr int RPP = 256 / TPR;
  constexpr int NP = 64 / RPP;
  constexpr int LDW = 64 + 2;  // padded row (halves) of the transposed tile
  __shared__ __align__(16) uint16_t tile[D * LDW];
  const int blk = blockIdx.x, bh = blockIdx.y, tid = threadIdx.x;
  const int c = tid % TPR, r = tid / TPR;
  const uint16_t *base = v + (size_t)(bh / H) * vs.sb + (size_t)(bh % H) * vs.sh + (size_t)blk * 64 * vs.sn + c * 8;
  const int last_row = min(63, N - 1 - blk * 64);
  uint4 raw[NP];
#pragma unroll
  for (int p = 0; p < NP; p++) raw[p] = load_stream_u4(base + (size_t)min(r + p * RPP, last_row) * vs.sn);
#pragma unroll
  for (int p = 0; p < NP; p++) {
    const int row = r + p * RPP;
    const uint4 q = row <= last_row ? raw[p] : make_uint4(0, 0, 0, 0);
    const uint32_t w[4] = {q.x, q.y, q.z, q.w};
#pragma unroll
    for (int e = 0; e < 8; e++) {
      const uint16_t b = (uint16_t)((e & 1) ? (w[e >> 1] >> 16) : (w[e >> 1] & 0xffffu));
      uint16_t h = b;
      if constexpr (DT == 1) h = f32_to_elem<0>(elem_to_f32<1>(b));     // bf16 -> fp16, one rounding
      tile[(c * 8 + e) * LDW + row] = h;
    }
  }
  __syncthreads();
  uint16_t *out = vt + ((size_t)bh * nk + blk) * (size_t)(D * 64);
  for (int i = tid; i < D * 8; i += 256) {   // 16-byte pieces: D rows x 8 slots
    const int d = i >> 3, slot = i & 7;
    const int kc = slot ^ ((d >> 1) & 7);      // key chunk stored in this slot
    const uint16_t *src = tile + d * LDW + kc * 8;
    uint32_t o[4];
#pragma unroll
    for (int e = 0; e < 4; e++) o[e] = (uint32_t)src[2 * e] | ((uint32_t)src[2 * e + 1] << 16);
    *(uint4 *)(out + d * 64 + slot * 8) = make_uint4(o[0], o[1], o[2], o[3]);
  }
}

__global__ void v_scale_final_kernel(float *v_scale, int n) {
  const int i = blockIdx.x * blockDim.x + threadIdx.x;
  if (i < n) v_scale[i] = v_scale[i] / 2.25f;
}

static int v_chunks(int B, int H, int N) {
  int want = (4096 + B * H - 1) / (B * H);
  int maxc = (N + 255) / 256;
  int c = want < maxc ? want : maxc;
  return c < 1 ? 1 : c;
}

template <int D, int DT>
static void launch_vq2(const void *v, Strides vs, uint8_t *v8, float *v_scale, int B, int H, int N, hipStream_t st) {
  const int n = B * H * D;
  const int nk = (N + 63) / 64;
  const int nchunk = v_chunks(B, H, N);
  const int rpc = (N + nchunk - 1) / nchunk;
  fill_u32_kernel<<<(n + 255) / 256, 256, 0, st>>>((uint32_t *)v_scale, 0u, n);
  v_absmax_kernel<D, DT><<<dim3(nchunk, B * H), 256, 0, st>>>((const uint16_t *)v, vs, H, (uint32_t *)v_scale, N, rpc);
  v_quant_kernel<D, DT><<<dim3(nk, B * H), 256, 0, st>>>((const uint16_t *)v, vs, H, v_scale, v8, N, nk);
  v_scale_final_kernel<<<(n + 255) / 256, 256, 0, st>>>(v_scale, n);
}

void launch_v_quant_fp8(const void *v, Strides vs, uint8_t *v8, float *v_scale, int B, int H, int N, int D, int dtype,
                        hipStream_t st) {
  if (D == 64) { if (dtype == 0) launch_vq2<64, 0>(v, vs, v8, v_scale, B, H, N, st); else launch_vq2<64, 1>(v, vs, v8, v_scale, B, H, N, st); }
  else         { if (dtype == 0) launch_vq2<128, 0>(v, vs, v8, v_scale, B, H, N, st); else launch_vq2<128, 1>(v, vs, v8, v_scale, B, H, N, st); }
}

void launch_v_tiles_f16(const void *v, Strides vs, void *vt, int B, int H, int N, int D, int dtype, hipStream_t st) {
  const int nk = (N + 63) / 64;
  const dim3 grid(nk, B * H);
  const uint16_t *vp = (const uint16_t *)v;
  uint16_t *op = (uint16_t *)vt;
  if (D == 64) { if (dtype == 0) v_tiles_f16_kernel<64, 0><<<grid, 256, 0, st>>>(vp, vs, H, op, N, nk); else v_tiles_f16_kernel<64, 1><<<grid, 256, 0, st>>>(vp, vs, H, op, N, nk); }
  else         { if (dtype == 0) v_tiles_f16_kernel<128, 0><<<grid, 256, 0, st>>>(vp, vs, H, op, N, nk); else v_tiles_f16_kernel<128, 1><<<grid, 256, 0, st>>>(vp, vs, H, op, N, nk); }
}

}  // namespace spg
