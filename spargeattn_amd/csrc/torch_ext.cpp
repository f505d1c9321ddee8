// PyTorch-ROCm extension over the C ABI of libspargeattn_amd.so: operators registered under torch.ops.spargeattn_amd.*
// with meta kernels, taking the place of the reference's pybind modules (csrc/qattn/pybind.cpp:20-36,
// csrc/fused/pybind.cpp:21-25).  The shim does what those entry points do around their kernels
// (csrc/qattn/qk_int_sv_f8_cuda_sm89.cu:213-254, 339-363): device / dtype / dimension / shape / contiguity checks
// (TORCH_CHECK), allocation of the outputs, the current HIP stream - and then hands raw pointers, sizes and strides to
// the extern "C" functions of include/spargeattn_amd.h.  No kernel lives here.
#include <ATen/ATen.h>
#include <ATen/hip/impl/HIPGuardImplMasqueradingAsCUDA.h>
#include <ATen/hip/impl/HIPStreamMasqueradingAsCUDA.h>
#include <torch/library.h>

#include <array>
#include <tuple>

#include "../../include/spargeattn_amd.h"

namespace {

using at::Tensor;

#define CHECK_GPU(x) TORCH_CHECK((x).is_cuda(), "Tensor " #x " must be on the GPU (there is no CPU path)")
#define CHECK_DTYPE(x, dt) TORCH_CHECK((x).scalar_type() == (dt), "Tensor " #x " must have dtype (" #dt ")")
#define CHECK_DIMS(x, n) TORCH_CHECK((x).dim() == (n), "Tensor " #x " must have dimension number (" #n ")")
#define CHECK_CONTIGUOUS(x) TORCH_CHECK((x).is_contiguous(), "Tensor " #x " must be contiguous")
#define CHECK_LASTDIM_CONTIGUOUS(x) TORCH_CHECK((x).stride(-1) == 1, "Tensor " #x " must be contiguous at the last dimension")
#define CHECK_SHAPE(x, ...) \
  TORCH_CHECK((x).sizes() == at::IntArrayRef({__VA_ARGS__}), "Tensor " #x " must have shape (" #__VA_ARGS__ "), got ", (x).sizes())

// A ROCm build of PyTorch presents its GPUs under the device type "cuda"; the guard and stream classes that accept that
// device type are the "masquerading" ones.  The stream is torch's current stream of the tensor's device.
using DeviceGuard = c10::hip::HIPGuardMasqueradingAsCUDA;
void *stream_of(const Tensor &t) {
  return (void *)c10::hip::getCurrentHIPStreamMasqueradingAsCUDA(t.device().index()).stream();
}

// status of the C ABI -> the exception classes of the ctypes binding (ValueError for argument errors, as the
// reference's std::invalid_argument; RuntimeError for HIP failures)
void check(int rc) {
  if (rc == SPG_OK) return;
  const std::string msg = spg_last_error();
  TORCH_CHECK_VALUE(rc != SPG_ERR_INVALID && rc != SPG_ERR_UNSUPPORTED, msg);
  TORCH_CHECK(false, msg);
}

int dtype_of(const Tensor &t) {
  TORCH_CHECK(t.scalar_type() == at::kHalf || t.scalar_type() == at::kBFloat16, "expected a float16 or bfloat16 tensor, got ",
              t.scalar_type());
  return t.scalar_type() == at::kHalf ? SPG_F16 : SPG_BF16;
}

// (B,H,N,D) tensor with a contiguous last dimension and 16-byte aligned rows: {batch, head, row} element strides, or
// NULL (via `use`) when the tensor is contiguous
struct StridesArg {
  std::array<int64_t, 3> s{};
  bool use = false;
  const int64_t *ptr() const { return use ? s.data() : nullptr; }
};
StridesArg strides_of(const Tensor &t, const char *name) {
  TORCH_CHECK(t.dim() == 4 && t.stride(3) == 1, "Tensor ", name, " must be 4-D with a contiguous last dimension");
  TORCH_CHECK(t.stride(0) % 8 == 0 && t.stride(1) % 8 == 0 && t.stride(2) % 8 == 0 && (uintptr_t)t.data_ptr() % 16 == 0,
              "Tensor ", name, ": rows must be 16-byte aligned (strides multiples of 8 elements)");
  StridesArg a;
  a.use = !t.is_contiguous();
  a.s = {t.stride(0), t.stride(1), t.stride(2)};
  return a;
}

const void *opt_ptr(const c10::optional<Tensor> &t) { return t.has_value() ? t->data_ptr() : nullptr; }

// ---- A2 ----------------------------------------------------------------------------------------------------------
Tensor km_mean(const Tensor &k) {
  CHECK_GPU(k);
  const DeviceGuard guard(k.device());
  const auto ks = strides_of(k, "k");
  const int B = k.size(0), H = k.size(1), N = k.size(2), D = k.size(3);
  Tensor km = at::empty({B, H, 1, D}, k.options());
  Tensor ws = at::empty({(int64_t)std::max<size_t>(1, spg_km_mean_workspace_bytes(B, H, N, D))}, k.options().dtype(at::kByte));
  check(spg_km_mean(k.data_ptr(), ks.ptr(), km.data_ptr(), ws.data_ptr(), B, H, N, D, dtype_of(k), stream_of(k)));
  return km;
}
Tensor km_mean_meta(const Tensor &k) { return at::empty({k.size(0), k.size(1), 1, k.size(3)}, k.options()); }

// ---- A3 / A4 / A13 -----------------------------------------------------------------------------------------------
std::tuple<Tensor, Tensor, Tensor, Tensor> psq_alloc(const Tensor &x, int64_t block, bool with_pool, int64_t quant_rows) {
  TORCH_CHECK_VALUE(block > 0 && quant_rows > 0 && block % quant_rows == 0, "quant_rows (", quant_rows,
                    ") must divide the block size (", block, ")");
  const int64_t B = x.size(0), H = x.size(1), N = x.size(2), D = x.size(3), nb = (N + block - 1) / block;
  Tensor xq = at::empty({B, H, N, D}, x.options().dtype(at::kChar));
  Tensor scale = at::empty({B, H, nb * (block / quant_rows)}, x.options().dtype(at::kFloat));
  Tensor pool = with_pool ? at::empty({B, H, nb, D}, x.options()) : at::empty({0}, x.options());
  Tensor sim = with_pool ? at::empty({B, H, nb}, x.options().dtype(at::kBool)) : at::empty({0}, x.options().dtype(at::kBool));
  return {pool, sim, xq, scale};
}
std::tuple<Tensor, Tensor, Tensor, Tensor> pool_sim_quant(const Tensor &x, const c10::optional<Tensor> &km, int64_t block,
                                                          const c10::optional<Tensor> &simthreshd1, bool with_pool,
                                                          int64_t quant_rows) {
  CHECK_GPU(x);
  const DeviceGuard guard(x.device());
  const auto xs = strides_of(x, "x");
  if (km.has_value()) { CHECK_GPU(*km); CHECK_CONTIGUOUS(*km); TORCH_CHECK(km->scalar_type() == x.scalar_type(), "km must have x's dtype"); }
  if (with_pool) {
    TORCH_CHECK(simthreshd1.has_value(), "simthreshd1 is needed for pooling");
    CHECK_GPU(*simthreshd1); CHECK_CONTIGUOUS(*simthreshd1); CHECK_DTYPE(*simthreshd1, at::kFloat);
    CHECK_SHAPE(*simthreshd1, x.size(1));
  }
  auto [pool, sim, xq, scale] = psq_alloc(x, block, with_pool, quant_rows);
  check(spg_pool_sim_quant(x.data_ptr(), xs.ptr(), opt_ptr(km), with_pool ? pool.data_ptr() : nullptr,
                           with_pool ? (uint8_t *)sim.data_ptr() : nullptr, (int8_t *)xq.data_ptr(), (float *)scale.data_ptr(),
                           with_pool ? (const float *)simthreshd1->data_ptr() : nullptr, x.size(0), x.size(1), x.size(2),
                           x.size(3), (int)block, (int)quant_rows, dtype_of(x), stream_of(x)));
  return {pool, sim, xq, scale};
}
std::tuple<Tensor, Tensor, Tensor, Tensor> pool_sim_quant_meta(const Tensor &x, const c10::optional<Tensor> &, int64_t block,
                                                               const c10::optional<Tensor> &, bool with_pool,
                                                               int64_t quant_rows) {
  return psq_alloc(x, block, with_pool, quant_rows);
}

// ---- A5-A8 ------------------------------------------------------------------------------------------------------
std::tuple<Tensor, Tensor, Tensor> bs_alloc(const Tensor &pool_q, const Tensor &pool_k, bool return_map) {
  const int64_t B = pool_q.size(0), H = pool_q.size(1), nq = pool_q.size(2), nk = pool_k.size(2);
  const auto io = pool_q.options().dtype(at::kInt);
  return {at::empty({B, H, nq, nk}, io), at::empty({B, H, nq}, io),
          return_map ? at::empty({B, H, nq, nk}, pool_q.options().dtype(at::kBool)) : at::empty({0}, pool_q.options().dtype(at::kBool))};
}
std::tuple<Tensor, Tensor, Tensor> block_select(const Tensor &pool_q, const Tensor &sim_q, const Tensor &pool_k,
                                                const Tensor &sim_k, const c10::optional<Tensor> &topk,
                                                const c10::optional<Tensor> &cdfthreshd, bool is_causal, bool attention_sink,
                                                bool return_map) {
  CHECK_GPU(pool_q); CHECK_GPU(sim_q); CHECK_GPU(pool_k); CHECK_GPU(sim_k);
  CHECK_CONTIGUOUS(pool_q); CHECK_CONTIGUOUS(sim_q); CHECK_CONTIGUOUS(pool_k); CHECK_CONTIGUOUS(sim_k);
  CHECK_DIMS(pool_q, 4); CHECK_DIMS(pool_k, 4);
  CHECK_DTYPE(sim_q, at::kBool); CHECK_DTYPE(sim_k, at::kBool);
  const DeviceGuard guard(pool_q.device());
  const int B = pool_q.size(0), H = pool_q.size(1), nq = pool_q.size(2), D = pool_q.size(3);
  const int Hkv = pool_k.size(1), nk = pool_k.size(2);
  TORCH_CHECK(pool_k.size(0) == B && pool_k.size(3) == D && pool_k.scalar_type() == pool_q.scalar_type(),
              "pooled tensors disagree: pool_q ", pool_q.sizes(), ", pool_k ", pool_k.sizes());
  CHECK_SHAPE(sim_q, B, H, nq);
  CHECK_SHAPE(sim_k, B, Hkv, nk);
  for (const auto *t : {&topk, &cdfthreshd})
    if (t->has_value()) {
      CHECK_GPU(**t); CHECK_CONTIGUOUS(**t); CHECK_DTYPE(**t, at::kFloat);
      TORCH_CHECK((*t)->numel() == H, "per-head hyper-parameter has ", (*t)->numel(), " entries, expected ", H);
    }
  auto [lut, valid, bmap] = bs_alloc(pool_q, pool_k, return_map);
  check(spg_block_select(pool_q.data_ptr(), (const uint8_t *)sim_q.data_ptr(), pool_k.data_ptr(), (const uint8_t *)sim_k.data_ptr(),
                         (const float *)opt_ptr(topk), (const float *)opt_ptr(cdfthreshd), is_causal, attention_sink,
                         (int32_t *)lut.data_ptr(), (int32_t *)valid.data_ptr(), return_map ? (uint8_t *)bmap.data_ptr() : nullptr, B,
                         H, Hkv, nq, nk, D, dtype_of(pool_q), stream_of(pool_q)));
  return {lut, valid, bmap};
}
std::tuple<Tensor, Tensor, Tensor> block_select_meta(const Tensor &pool_q, const Tensor &, const Tensor &pool_k, const Tensor &,
                                                     const c10::optional<Tensor> &, const c10::optional<Tensor> &, bool, bool,
                                                     bool return_map) {
  return bs_alloc(pool_q, pool_k, return_map);
}

int mask_kind_of(const Tensor &m) {
  switch (m.scalar_type()) {
    case at::kBool: case at::kByte: case at::kChar: return SPG_MASK_I8;
    case at::kShort: return SPG_MASK_I16;
    case at::kInt: return SPG_MASK_I32;
    case at::kLong: return SPG_MASK_I64;
    case at::kHalf: case at::kBFloat16: return SPG_MASK_F16;
    case at::kFloat: return SPG_MASK_F32;
    case at::kDouble: return SPG_MASK_F64;
    default: TORCH_CHECK(false, "unsupported mask dtype ", m.scalar_type());
  }
}
std::tuple<Tensor, Tensor> map_to_lut(const Tensor &block_map) {
  CHECK_GPU(block_map); CHECK_CONTIGUOUS(block_map); CHECK_DIMS(block_map, 4);
  const DeviceGuard guard(block_map.device());
  const int B = block_map.size(0), H = block_map.size(1), nq = block_map.size(2), nk = block_map.size(3);
  const auto io = block_map.options().dtype(at::kInt);
  Tensor lut = at::empty({B, H, nq, nk}, io), valid = at::empty({B, H, nq}, io);
  check(spg_map_to_lut(block_map.data_ptr(), mask_kind_of(block_map), (int32_t *)lut.data_ptr(), (int32_t *)valid.data_ptr(), B, H,
                       nq, nk, stream_of(block_map)));
  return {lut, valid};
}
std::tuple<Tensor, Tensor> map_to_lut_meta(const Tensor &m) {
  const auto io = m.options().dtype(at::kInt);
  return {at::empty(m.sizes(), io), at::empty({m.size(0), m.size(1), m.size(2)}, io)};
}

// ---- A9 / A10 ---------------------------------------------------------------------------------------------------
std::tuple<Tensor, Tensor> v_quant_fp8(const Tensor &v) {
  CHECK_GPU(v);
  const DeviceGuard guard(v.device());
  const auto vs = strides_of(v, "v");
  const int64_t B = v.size(0), H = v.size(1), N = v.size(2), D = v.size(3), nk = (N + 63) / 64;
  Tensor v8 = at::empty({B, H, nk, D, 64}, v.options().dtype(at::kByte));
  Tensor v_scale = at::empty({B, H, D}, v.options().dtype(at::kFloat));
  check(spg_v_quant_fp8(v.data_ptr(), vs.ptr(), (uint8_t *)v8.data_ptr(), (float *)v_scale.data_ptr(), B, H, N, D, dtype_of(v),
                        stream_of(v)));
  return {v8, v_scale};
}
std::tuple<Tensor, Tensor> v_quant_fp8_meta(const Tensor &v) {
  return {at::empty({v.size(0), v.size(1), (v.size(2) + 63) / 64, v.size(3), 64}, v.options().dtype(at::kByte)),
          at::empty({v.size(0), v.size(1), v.size(3)}, v.options().dtype(at::kFloat))};
}
Tensor v_tiles_f16(const Tensor &v) {
  CHECK_GPU(v);
  const DeviceGuard guard(v.device());
  const auto vs = strides_of(v, "v");
  const int64_t B = v.size(0), H = v.size(1), N = v.size(2), D = v.size(3), nk = (N + 63) / 64;
  Tensor vt = at::empty({B, H, nk, D, 64}, v.options().dtype(at::kHalf));
  check(spg_v_tiles_f16(v.data_ptr(), vs.ptr(), vt.data_ptr(), B, H, N, D, dtype_of(v), stream_of(v)));
  return vt;
}
Tensor v_tiles_f16_meta(const Tensor &v) {
  return at::empty({v.size(0), v.size(1), (v.size(2) + 63) / 64, v.size(3), 64}, v.options().dtype(at::kHalf));
}

// ---- A11 ---------------------------------------------------------------------------------------------------------
// the checks of the reference's entry point (sm89.cu:213-254, 339-363); V arrives in this library's tile layout
struct AttnDims { int B, H, Hkv, N, Nk, D; };
AttnDims check_attn(const Tensor &query, const Tensor &key, const Tensor &value, const Tensor &output, const Tensor &lut,
                    const Tensor &valid_block_num, const Tensor &pv_threshold, const Tensor &query_scale, const Tensor &key_scale,
                    const c10::optional<Tensor> &value_scale, int64_t qk_quant_gran, at::ScalarType v_dtype) {
  CHECK_GPU(query); CHECK_GPU(key); CHECK_GPU(value); CHECK_GPU(output); CHECK_GPU(lut); CHECK_GPU(valid_block_num);
  CHECK_GPU(pv_threshold); CHECK_GPU(query_scale); CHECK_GPU(key_scale);
  CHECK_CONTIGUOUS(query); CHECK_CONTIGUOUS(key); CHECK_CONTIGUOUS(value);
  CHECK_LASTDIM_CONTIGUOUS(output);
  CHECK_CONTIGUOUS(lut); CHECK_CONTIGUOUS(valid_block_num); CHECK_CONTIGUOUS(pv_threshold); CHECK_CONTIGUOUS(query_scale);
  CHECK_CONTIGUOUS(key_scale);
  CHECK_DTYPE(query, at::kChar); CHECK_DTYPE(key, at::kChar); CHECK_DTYPE(value, v_dtype); CHECK_DTYPE(lut, at::kInt);
  CHECK_DTYPE(valid_block_num, at::kInt); CHECK_DTYPE(pv_threshold, at::kFloat); CHECK_DTYPE(query_scale, at::kFloat);
  CHECK_DTYPE(key_scale, at::kFloat);
  CHECK_DIMS(query, 4); CHECK_DIMS(key, 4); CHECK_DIMS(value, 5); CHECK_DIMS(output, 4); CHECK_DIMS(lut, 4);
  CHECK_DIMS(valid_block_num, 3); CHECK_DIMS(pv_threshold, 1); CHECK_DIMS(query_scale, 3); CHECK_DIMS(key_scale, 3);
  const int64_t B = query.size(0), H = query.size(1), N = query.size(2), D = query.size(3);
  const int64_t Hkv = key.size(1), Nk = key.size(2), nq = (N + 127) / 128, nk = (Nk + 63) / 64;
  TORCH_CHECK(key.size(0) == B && key.size(3) == D, "k shape ", key.sizes(), " does not match q shape ", query.sizes());
  TORCH_CHECK(value.sizes() == at::IntArrayRef({B, Hkv, nk, D, 64}), "V tiles have shape ", value.sizes(), ", expected (",
              B, ", ", Hkv, ", ", nk, ", ", D, ", 64) for kv_len ", Nk);
  CHECK_SHAPE(output, B, H, N, D);
  TORCH_CHECK_VALUE(qk_quant_gran != 3, "qk_quant_gran 3 (per thread) is not supported on gfx950");
  TORCH_CHECK_VALUE(qk_quant_gran == SPG_QUANT_PER_BLOCK || qk_quant_gran == SPG_QUANT_PER_WARP,
                    "Unsupported qk_quant_gran: ", qk_quant_gran);
  const int64_t nqs = qk_quant_gran == SPG_QUANT_PER_WARP ? nq * 4 : nq;
  TORCH_CHECK(query_scale.sizes() == at::IntArrayRef({B, H, nqs}) && key_scale.sizes() == at::IntArrayRef({B, Hkv, nk}),
              "q_scale / k_scale have shapes ", query_scale.sizes(), " / ", key_scale.sizes(), ", expected (", B, ", ", H, ", ", nqs,
              ") / (", B, ", ", Hkv, ", ", nk, ") for qk_quant_gran = ", qk_quant_gran);
  if (value_scale.has_value()) {
    CHECK_GPU(*value_scale); CHECK_CONTIGUOUS(*value_scale); CHECK_DTYPE(*value_scale, at::kFloat);
    CHECK_SHAPE(*value_scale, B, Hkv, D);
  }
  TORCH_CHECK(lut.sizes() == at::IntArrayRef({B, H, nq, nk}) && valid_block_num.sizes() == at::IntArrayRef({B, H, nq}),
              "lut / valid_block_num have shapes ", lut.sizes(), " / ", valid_block_num.sizes(), ", expected (", B, ", ", H, ", ", nq,
              ", ", nk, ") / (", B, ", ", H, ", ", nq, ")");
  CHECK_SHAPE(pv_threshold, H);
  return {(int)B, (int)H, (int)Hkv, (int)N, (int)Nk, (int)D};
}
Tensor pv_count_alloc(const Tensor &q, bool return_pv_count) {
  return return_pv_count ? at::zeros({q.size(0), q.size(1), 4 * ((q.size(2) + 127) / 128)}, q.options().dtype(at::kInt))
                         : at::empty({0}, q.options().dtype(at::kInt));
}
Tensor block_sparse_attn(const Tensor &q8, const Tensor &k8, const Tensor &v8, Tensor out, const Tensor &lut, const Tensor &valid,
                         const Tensor &pvthreshd, const Tensor &q_scale, const Tensor &k_scale, const Tensor &v_scale,
                         double sm_scale, bool is_causal, int64_t qk_quant_gran, int64_t pv_mode, bool return_pv_count) {
  const AttnDims d = check_attn(q8, k8, v8, out, lut, valid, pvthreshd, q_scale, k_scale, v_scale, qk_quant_gran, at::kByte);
  const DeviceGuard guard(q8.device());
  const auto os = strides_of(out, "out");
  Tensor pvc = pv_count_alloc(q8, return_pv_count);
  check(spg_block_sparse_attn((const int8_t *)q8.data_ptr(), (const int8_t *)k8.data_ptr(), (const uint8_t *)v8.data_ptr(),
                              out.data_ptr(), os.ptr(), dtype_of(out), (const int32_t *)lut.data_ptr(),
                              (const int32_t *)valid.data_ptr(), (const float *)pvthreshd.data_ptr(), (const float *)q_scale.data_ptr(),
                              (const float *)k_scale.data_ptr(), (const float *)v_scale.data_ptr(), d.B, d.H, d.Hkv, d.N, d.Nk, d.D,
                              (float)sm_scale, is_causal, (int)qk_quant_gran, (int)pv_mode,
                              return_pv_count ? (int32_t *)pvc.data_ptr() : nullptr, stream_of(q8)));
  return pvc;
}
Tensor block_sparse_attn_meta(const Tensor &q8, const Tensor &, const Tensor &, Tensor, const Tensor &, const Tensor &, const Tensor &,
                              const Tensor &, const Tensor &, const Tensor &, double, bool, int64_t, int64_t, bool return_pv_count) {
  return pv_count_alloc(q8, return_pv_count);
}
Tensor block_sparse_attn_f16v(const Tensor &q8, const Tensor &k8, const Tensor &vt, Tensor out, const Tensor &lut,
                              const Tensor &valid, const Tensor &pvthreshd, const Tensor &q_scale, const Tensor &k_scale,
                              double sm_scale, bool is_causal, int64_t qk_quant_gran, int64_t pv_mode, bool return_pv_count) {
  const AttnDims d = check_attn(q8, k8, vt, out, lut, valid, pvthreshd, q_scale, k_scale, c10::nullopt, qk_quant_gran, at::kHalf);
  const DeviceGuard guard(q8.device());
  const auto os = strides_of(out, "out");
  Tensor pvc = pv_count_alloc(q8, return_pv_count);
  check(spg_block_sparse_attn_f16v((const int8_t *)q8.data_ptr(), (const int8_t *)k8.data_ptr(), vt.data_ptr(), out.data_ptr(),
                                   os.ptr(), dtype_of(out), (const int32_t *)lut.data_ptr(), (const int32_t *)valid.data_ptr(),
                                   (const float *)pvthreshd.data_ptr(), (const float *)q_scale.data_ptr(),
                                   (const float *)k_scale.data_ptr(), d.B, d.H, d.Hkv, d.N, d.Nk, d.D, (float)sm_scale, is_causal,
                                   (int)qk_quant_gran, (int)pv_mode, return_pv_count ? (int32_t *)pvc.data_ptr() : nullptr,
                                   stream_of(q8)));
  return pvc;
}
Tensor block_sparse_attn_f16v_meta(const Tensor &q8, const Tensor &, const Tensor &, Tensor, const Tensor &, const Tensor &,
                                   const Tensor &, const Tensor &, const Tensor &, double, bool, int64_t, int64_t,
                                   bool return_pv_count) {
  return pv_count_alloc(q8, return_pv_count);
}

// ---- measurement comparator and self tests ------------------------------------------------------------------------
Tensor dense_attn_f16(const Tensor &q, const Tensor &k, const Tensor &vt, Tensor out, double sm_scale, bool is_causal) {
  CHECK_GPU(q); CHECK_GPU(k); CHECK_GPU(vt); CHECK_GPU(out);
  CHECK_CONTIGUOUS(q); CHECK_CONTIGUOUS(k); CHECK_CONTIGUOUS(vt); CHECK_CONTIGUOUS(out);
  CHECK_DTYPE(q, at::kHalf); CHECK_DTYPE(k, at::kHalf); CHECK_DTYPE(vt, at::kHalf); CHECK_DTYPE(out, at::kHalf);
  CHECK_DIMS(q, 4);
  const int64_t B = q.size(0), H = q.size(1), N = q.size(2), D = q.size(3);
  CHECK_SHAPE(k, B, H, N, D); CHECK_SHAPE(out, B, H, N, D); CHECK_SHAPE(vt, B, H, (N + 63) / 64, D, 64);
  const DeviceGuard guard(q.device());
  check(spg_dense_attn_f16(q.data_ptr(), k.data_ptr(), vt.data_ptr(), out.data_ptr(), B, H, N, D, (float)sm_scale, is_causal,
                           stream_of(q)));
  return out;
}
Tensor dense_attn_f16_meta(const Tensor &, const Tensor &, const Tensor &, Tensor out, double, bool) { return out; }

Tensor selftest_fp8_pack(const Tensor &x, bool saturate) {
  CHECK_GPU(x); CHECK_CONTIGUOUS(x); CHECK_DTYPE(x, at::kFloat);
  const DeviceGuard guard(x.device());
  Tensor codes = at::empty(x.sizes(), x.options().dtype(at::kByte));
  check(spg_selftest_fp8_pack((const float *)x.data_ptr(), (uint8_t *)codes.data_ptr(), (int)x.numel(), saturate, stream_of(x)));
  return codes;
}
Tensor selftest_fp8_pack_meta(const Tensor &x, bool) { return at::empty(x.sizes(), x.options().dtype(at::kByte)); }

Tensor selftest_division(const Tensor &counts, int64_t n_divisors, int64_t seed) {
  CHECK_GPU(counts); CHECK_CONTIGUOUS(counts); CHECK_DTYPE(counts, at::kLong);
  TORCH_CHECK(counts.numel() >= 2, "counts needs two entries");
  const DeviceGuard guard(counts.device());
  check(spg_selftest_division((unsigned long long *)counts.data_ptr(), (int)n_divisors, (unsigned int)seed, stream_of(counts)));
  return counts;
}
Tensor selftest_division_meta(const Tensor &counts, int64_t, int64_t) { return counts; }

}  // namespace

TORCH_LIBRARY(spargeattn_amd, m) {
  m.def("km_mean(Tensor k) -> Tensor");
  m.def("pool_sim_quant(Tensor x, Tensor? km, int block, Tensor? simthreshd1, bool with_pool, int quant_rows) -> (Tensor, Tensor, Tensor, Tensor)");
  m.def("block_select(Tensor pool_q, Tensor sim_q, Tensor pool_k, Tensor sim_k, Tensor? topk, Tensor? cdfthreshd, bool is_causal, bool attention_sink, bool return_map) -> (Tensor, Tensor, Tensor)");
  m.def("map_to_lut(Tensor block_map) -> (Tensor, Tensor)");
  m.def("v_quant_fp8(Tensor v) -> (Tensor, Tensor)");
  m.def("v_tiles_f16(Tensor v) -> Tensor");
  m.def("block_sparse_attn(Tensor q8, Tensor k8, Tensor v8, Tensor(a!) out, Tensor lut, Tensor valid_block_num, Tensor pvthreshd, Tensor q_scale, Tensor k_scale, Tensor v_scale, float sm_scale, bool is_causal, int qk_quant_gran, int pv_threshold_mode, bool return_pv_count) -> Tensor");
  m.def("block_sparse_attn_f16v(Tensor q8, Tensor k8, Tensor vt, Tensor(a!) out, Tensor lut, Tensor valid_block_num, Tensor pvthreshd, Tensor q_scale, Tensor k_scale, float sm_scale, bool is_causal, int qk_quant_gran, int pv_threshold_mode, bool return_pv_count) -> Tensor");
  m.def("dense_attn_f16(Tensor q, Tensor k, Tensor vt, Tensor(a!) out, float sm_scale, bool is_causal) -> Tensor(a!)");
  m.def("selftest_fp8_pack(Tensor x, bool saturate) -> Tensor");
  m.def("selftest_division(Tensor(a!) counts, int n_divisors, int seed) -> Tensor(a!)");
}

// torch's "CUDA" dispatch key is the GPU key of a ROCm build as well
TORCH_LIBRARY_IMPL(spargeattn_amd, CUDA, m) {
  m.impl("km_mean", &km_mean);
  m.impl("pool_sim_quant", &pool_sim_quant);
  m.impl("block_select", &block_select);
  m.impl("map_to_lut", &map_to_lut);
  m.impl("v_quant_fp8", &v_quant_fp8);
  m.impl("v_tiles_f16", &v_tiles_f16);
  m.impl("block_sparse_attn", &block_sparse_attn);
  m.impl("block_sparse_attn_f16v", &block_sparse_attn_f16v);
  m.impl("dense_attn_f16", &dense_attn_f16);
  m.impl("selftest_fp8_pack", &selftest_fp8_pack);
  m.impl("selftest_division", &selftest_division);
}

TORCH_LIBRARY_IMPL(spargeattn_amd, Meta, m) {
  m.impl("km_mean", &km_mean_meta);
  m.impl("pool_sim_quant", &pool_sim_quant_meta);
  m.impl("block_select", &block_select_meta);
  m.impl("map_to_lut", &map_to_lut_meta);
  m.impl("v_quant_fp8", &v_quant_fp8_meta);
  m.impl("v_tiles_f16", &v_tiles_f16_meta);
  m.impl("block_sparse_attn", &block_sparse_attn_meta);
  m.impl("block_sparse_attn_f16v", &block_sparse_attn_f16v_meta);
  m.impl("dense_attn_f16", &dense_attn_f16_meta);
  m.impl("selftest_fp8_pack", &selftest_fp8_pack_meta);
  m.impl("selftest_division", &selftest_division_meta);
}
