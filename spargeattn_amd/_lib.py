"""Bindings of libspargeattn_amd.so (the C ABI in include/spargeattn_amd.h).

Two interchangeable bindings sit under the stage wrappers of this module:

* ``"ctypes"`` (default, nothing to compile beyond the library): PyTorch supplies device memory and the current
  stream, the wrappers hand raw ``data_ptr()`` addresses to the C functions;
* ``"torch"``: the PyTorch extension ``libspargeattn_amd_torch.so`` (csrc/torch_ext.cpp), whose operators are
  registered as ``torch.ops.spargeattn_amd.*`` with meta kernels and do their own TORCH_CHECKs, allocation and stream
  lookup in C++ - the form the reference's pybind modules have (csrc/qattn/pybind.cpp:20-36).

Select with ``set_binding("torch")`` or the environment variable ``SPARGEATTN_AMD_BINDING``.  There is no CPU or eager
fallback in either: if the library is missing, or no GPU tensor is given, the call raises.
"""
import contextlib
import ctypes
import os

import torch

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "libspargeattn_amd.so")
TORCH_EXT_PATH = os.path.join(_HERE, "libspargeattn_amd_torch.so")

SPG_OK, SPG_ERR_INVALID, SPG_ERR_UNSUPPORTED, SPG_ERR_HIP = 0, 1, 2, 3
SPG_F16, SPG_BF16 = 0, 1

_c = ctypes
_vp, _i, _f, _sz = _c.c_void_p, _c.c_int, _c.c_float, _c.c_size_t

# symbol -> (restype, argtypes); must list every function include/spargeattn_amd.h declares
SIGNATURES = {
    "spg_version": (_i, []),
    "spg_last_error": (_c.c_char_p, []),
    "spg_km_mean_workspace_bytes": (_sz, [_i, _i, _i, _i]),
    "spg_km_mean": (_i, [_vp, _vp, _vp, _vp, _i, _i, _i, _i, _i, _vp]),
    "spg_km_mean_static": (_i, [_vp, _vp, _vp, _i, _i, _i, _i, _i, _vp]),
    "spg_pool_sim_quant": (_i, [_vp, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _i, _i, _i, _i, _i, _i, _i, _vp]),
    "spg_block_select": (_i, [_vp, _vp, _vp, _vp, _vp, _vp, _i, _i, _vp, _vp, _vp, _i, _i, _i, _i, _i, _i, _i, _vp]),
    "spg_map_to_lut": (_i, [_vp, _i, _vp, _vp, _i, _i, _i, _i, _vp]),
    "spg_v_quant_fp8": (_i, [_vp, _vp, _vp, _vp, _i, _i, _i, _i, _i, _vp]),
    "spg_block_sparse_attn": (_i, [_vp, _vp, _vp, _vp, _vp, _i, _vp, _vp, _vp, _vp, _vp, _vp, _i, _i, _i, _i, _i, _i, _f, _i, _i, _i, _vp, _vp]),
    "spg_v_tiles_f16": (_i, [_vp, _vp, _vp, _i, _i, _i, _i, _i, _vp]),
    "spg_block_sparse_attn_f16v": (_i, [_vp] * 5 + [_i] + [_vp] * 5 + [_i] * 6 + [_f, _i, _i, _i, _vp, _vp]),
    "spg_dense_attn_f16": (_i, [_vp, _vp, _vp, _vp, _i, _i, _i, _i, _f, _i, _vp]),
    "spg_selftest_division": (_i, [_vp, _i, ctypes.c_uint, _vp]),
    "spg_selftest_fp8_pack": (_i, [_vp, _vp, _i, _i, _vp]),
}

_lib = None
_ops = None          # torch.ops.spargeattn_amd once the extension is loaded
_binding = None      # "ctypes" or "torch"; resolved on first use from SPARGEATTN_AMD_BINDING


class SpargeError(RuntimeError):
    pass


def set_binding(name):
    """Route the stage wrappers through the ctypes binding ("ctypes") or the PyTorch extension ("torch")."""
    global _binding
    if name not in ("ctypes", "torch"):
        raise ValueError(f"unknown binding {name!r}: expected 'ctypes' or 'torch'")
    if name == "torch":
        load_torch_ext()
    _binding = name


def get_binding():
    global _binding
    if _binding is None:
        set_binding(os.environ.get("SPARGEATTN_AMD_BINDING", "ctypes"))
    return _binding


def _torch():
    """torch.ops.spargeattn_amd when the torch binding is selected, else None."""
    return _ops if get_binding() == "torch" else None


def load_torch_ext():
    """Load the PyTorch extension (once) and return torch.ops.spargeattn_amd.  Raises if it has not been built."""
    global _ops
    if _ops is None:
        load()                                   # the extension links against the C-ABI library beside it
        if not os.path.exists(TORCH_EXT_PATH):
            raise SpargeError(f"{TORCH_EXT_PATH} not found: build it with `python -m spargeattn_amd.build`.")
        torch.ops.load_library(TORCH_EXT_PATH)
        _ops = torch.ops.spargeattn_amd
    return _ops


def load():
    """Load the shared library (once).  Raises if it has not been built."""
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            raise SpargeError(
                f"{LIB_PATH} not found: build it with `python -m spargeattn_amd.build` (hipcc, gfx950). "
                "There is no fallback path.")
        lib = ctypes.CDLL(LIB_PATH)
        for name, (res, args) in SIGNATURES.items():
            fn = getattr(lib, name)
            fn.restype, fn.argtypes = res, args
        _lib = lib
    return _lib


def _check(rc):
    if rc == SPG_OK:
        return
    msg = load().spg_last_error().decode()
    if rc in (SPG_ERR_INVALID, SPG_ERR_UNSUPPORTED):
        raise ValueError(msg)
    raise SpargeError(msg)


def _dt(t):
    if t.dtype == torch.float16:
        return SPG_F16
    if t.dtype == torch.bfloat16:
        return SPG_BF16
    raise RuntimeError(f"expected a float16 or bfloat16 tensor, got {t.dtype}")


def _dev(*ts):
    for t in ts:
        if t is None:
            continue
        if not t.is_cuda:
            raise RuntimeError("spargeattn_amd kernels need GPU tensors (there is no CPU path)")
        if not t.is_contiguous():
            raise RuntimeError("tensor must be contiguous")


def _p(t):
    return None if t is None else t.data_ptr()


def _dev_strided(*ts):
    """GPU tensors (B,H,N,D) whose last dimension is contiguous; the other strides are free (HND, NHD views, slices)."""
    for t in ts:
        if not t.is_cuda:
            raise RuntimeError("spargeattn_amd kernels need GPU tensors (there is no CPU path)")
        if t.dim() != 4 or t.stride(3) != 1:
            raise RuntimeError("expected a 4-D tensor whose last dimension is contiguous")
        if any(st % 8 for st in t.stride()[:3]) or t.data_ptr() % 16:
            raise RuntimeError("rows must be 16-byte aligned (strides multiples of 8 elements)")


def _st(t):
    """{batch, head, row} element strides as the host array the C ABI takes (NULL when contiguous)."""
    if t.is_contiguous():
        return None
    return (ctypes.c_int64 * 3)(t.stride(0), t.stride(1), t.stride(2))


def _stream(stream=None):
    """Raw HIP stream handle: torch's current stream, or the given torch stream.  Wrappers that take ``stream=``
    allocate their outputs in the caller's (current) stream context and only LAUNCH on the given one, so the caching
    allocator keeps treating the outputs as the caller's; the caller orders the two streams with events."""
    return (torch.cuda.current_stream() if stream is None else stream).cuda_stream


_MASK_KIND = {
    torch.bool: 0, torch.uint8: 0, torch.int8: 0, torch.int16: 1, torch.int32: 2, torch.int64: 3,
    torch.float16: 4, torch.bfloat16: 4, torch.float32: 5, torch.float64: 6,
}


# ----------------------------------------------------------------------------------------------
# stage wrappers (allocate outputs with torch, call the C ABI)
# ----------------------------------------------------------------------------------------------

def km_mean(k):
    """k (B,H,N,D) -> km (B,H,1,D), same dtype."""
    _dev_strided(k)
    if _torch() is not None:
        return _ops.km_mean(k)
    B, H, N, D = k.shape
    lib = load()
    km = torch.empty((B, H, 1, D), dtype=k.dtype, device=k.device)
    ws = torch.empty(max(1, lib.spg_km_mean_workspace_bytes(B, H, N, D)), dtype=torch.uint8, device=k.device)
    _check(lib.spg_km_mean(_p(k), _st(k), _p(km), _p(ws), B, H, N, D, _dt(k), _stream()))
    return km


def pool_sim_quant(x, km, block, simthreshd1=None, with_pool=True, stream=None, quant_rows=None):
    """Returns (pool, sim, x_int8, scale) - pool and sim are None when with_pool is False.
    quant_rows: rows that share one INT8 scale (default: the block; 32 for the per-warp granularity of Q), scale is
    (B, H, nb * block / quant_rows)."""
    _dev_strided(x)
    _dev(km, simthreshd1)
    B, H, N, D = x.shape
    nb = (N + block - 1) // block
    quant_rows = block if quant_rows is None else int(quant_rows)
    if quant_rows <= 0 or block % quant_rows:
        raise ValueError(f"quant_rows ({quant_rows}) must divide the block size ({block})")
    if _torch() is not None:
        with torch.cuda.stream(stream) if stream is not None else contextlib.nullcontext():
            pool, sim, xq, scale = _ops.pool_sim_quant(x, km, block, simthreshd1 if with_pool else None, with_pool, quant_rows)
        return (pool, sim, xq, scale) if with_pool else (None, None, xq, scale)
    xq = torch.empty((B, H, N, D), dtype=torch.int8, device=x.device)
    scale = torch.empty((B, H, nb * (block // quant_rows)), dtype=torch.float32, device=x.device)
    pool = sim = None
    if with_pool:
        pool = torch.empty((B, H, nb, D), dtype=x.dtype, device=x.device)
        sim = torch.empty((B, H, nb), dtype=torch.bool, device=x.device)
    _check(load().spg_pool_sim_quant(_p(x), _st(x), _p(km), _p(pool), _p(sim), _p(xq), _p(scale), _p(simthreshd1),
                                     B, H, N, D, block, quant_rows, _dt(x), _stream(stream)))
    return pool, sim, xq, scale


def block_select(pool_q, sim_q, pool_k, sim_k, topk=None, cdfthreshd=None, is_causal=False,
                 attention_sink=False, return_map=False):
    _dev(pool_q, sim_q, pool_k, sim_k, topk, cdfthreshd)
    B, H, nq, D = pool_q.shape
    Hkv, nk = pool_k.shape[1], pool_k.shape[2]
    if (pool_k.shape[0], pool_k.shape[3]) != (B, D) or tuple(sim_q.shape) != (B, H, nq) or tuple(sim_k.shape) != (B, Hkv, nk):
        raise RuntimeError(f"pooled tensors disagree: pool_q {tuple(pool_q.shape)}, sim_q {tuple(sim_q.shape)}, "
                           f"pool_k {tuple(pool_k.shape)}, sim_k {tuple(sim_k.shape)}")
    for t in (topk, cdfthreshd):
        if t is not None and t.numel() != H:
            raise RuntimeError(f"per-head hyper-parameter has {t.numel()} entries, expected {H}")
    if _torch() is not None:
        lut, valid, bmap = _ops.block_select(pool_q, sim_q, pool_k, sim_k, topk, cdfthreshd, bool(is_causal),
                                             bool(attention_sink), bool(return_map))
        return lut, valid, (bmap if return_map else None)
    lut = torch.empty((B, H, nq, nk), dtype=torch.int32, device=pool_q.device)
    valid = torch.empty((B, H, nq), dtype=torch.int32, device=pool_q.device)
    bmap = torch.empty((B, H, nq, nk), dtype=torch.bool, device=pool_q.device) if return_map else None
    _check(load().spg_block_select(_p(pool_q), _p(sim_q), _p(pool_k), _p(sim_k), _p(topk), _p(cdfthreshd),
                                   int(bool(is_causal)), int(bool(attention_sink)), _p(lut), _p(valid), _p(bmap),
                                   B, H, Hkv, nq, nk, D, _dt(pool_q), _stream()))
    return lut, valid, bmap


def map_to_lut(block_map):
    _dev(block_map)
    if block_map.dtype not in _MASK_KIND:
        raise RuntimeError(f"unsupported mask dtype {block_map.dtype}")
    if _torch() is not None:
        return tuple(_ops.map_to_lut(block_map))
    B, H, nq, nk = block_map.shape
    lut = torch.empty((B, H, nq, nk), dtype=torch.int32, device=block_map.device)
    valid = torch.empty((B, H, nq), dtype=torch.int32, device=block_map.device)
    _check(load().spg_map_to_lut(_p(block_map), _MASK_KIND[block_map.dtype], _p(lut), _p(valid), B, H, nq, nk, _stream()))
    return lut, valid


def v_quant_fp8(v, stream=None):
    """v (B,H,N,D) fp16/bf16 -> (v8 uint8 codes in tile layout (B,H,nk,D,64), v_scale (B,H,D) float32)."""
    _dev_strided(v)
    if _torch() is not None:
        with torch.cuda.stream(stream) if stream is not None else contextlib.nullcontext():
            return tuple(_ops.v_quant_fp8(v))
    B, H, N, D = v.shape
    nk = (N + 63) // 64
    v8 = torch.empty((B, H, nk, D, 64), dtype=torch.uint8, device=v.device)
    v_scale = torch.empty((B, H, D), dtype=torch.float32, device=v.device)
    _check(load().spg_v_quant_fp8(_p(v), _st(v), _p(v8), _p(v_scale), B, H, N, D, _dt(v), _stream(stream)))
    return v8, v_scale


def _v_swizzle_index(D, device):
    """slot index (D,4) such that tile[d, slot] holds key chunk slot ^ ((d >> 2) & 3)."""
    d = torch.arange(D, device=device)
    return torch.arange(4, device=device)[None, :] ^ ((d >> 2) & 3)[:, None]


def v8_tiles_to_natural(v8):
    """(B,H,nk,D,64) swizzled tile layout -> (B,H,nk*64,D) codes in natural key order."""
    B, H, nk, D, _ = v8.shape
    idx = _v_swizzle_index(D, v8.device)                       # natural chunk kc sits at slot kc ^ swz = idx[d, kc]
    t = v8.view(B, H, nk, D, 4, 16)
    nat = torch.gather(t, 4, idx.view(1, 1, 1, D, 4, 1).expand(B, H, nk, D, 4, 16))
    return nat.reshape(B, H, nk, D, 64).permute(0, 1, 2, 4, 3).reshape(B, H, nk * 64, D)


def v8_natural_to_tiles(v8_nat):
    """(B,H,nk*64,D) codes in natural key order -> the (B,H,nk,D,64) swizzled tile layout the attention kernel reads."""
    B, H, n64, D = v8_nat.shape
    nk = n64 // 64
    t = v8_nat.view(B, H, nk, 64, D).permute(0, 1, 2, 4, 3).contiguous().view(B, H, nk, D, 4, 16)
    idx = _v_swizzle_index(D, v8_nat.device)                   # slot s holds chunk s ^ swz = idx[d, s]
    sw = torch.gather(t, 4, idx.view(1, 1, 1, D, 4, 1).expand(B, H, nk, D, 4, 16))
    return sw.reshape(B, H, nk, D, 64).contiguous()


PV_NONE, PV_PER_BLOCK, PV_PER_WARP = 0, 1, 2
QUANT_PER_BLOCK, QUANT_PER_WARP = 1, 2


def quant_gran(value):
    """qk_quant_gran as the reference's kernel entry takes it (1 per block, 2 per warp, 3 per thread,
    csrc/pytorch_extensions_utils.cuh:71-85) or by name -> 1 or 2; anything else raises ValueError."""
    names = {"per_block": 1, "per_warp": 2, "per_thread": 3}
    g = names.get(value, value) if isinstance(value, str) else value
    if g in (QUANT_PER_BLOCK, QUANT_PER_WARP) and not isinstance(g, bool):
        return int(g)
    if g == 3:
        raise ValueError("qk_quant_gran 3 (per thread) is not supported on gfx950")
    raise ValueError(f"Unsupported qk_quant_gran: {value}")


def _check_attn_shapes(q8, k8, vt, lut, valid, q_scale, k_scale, v_scale=None, qk_quant_gran=QUANT_PER_BLOCK):
    """Shapes the attention kernels index with: raises before a launch could read past a buffer.
    The query length N and the key/value length N_kv are independent (qo_len / kv_len of
    csrc/qattn/qk_int_sv_f8_cuda_sm89.cu:256-300)."""
    B, H, N, D = q8.shape
    Hkv, Nk = k8.shape[1], k8.shape[2]
    nq, nk = (N + 127) // 128, (Nk + 63) // 64
    if k8.shape[0] != B or k8.shape[3] != D:
        raise RuntimeError(f"k shape {tuple(k8.shape)} does not match q shape {tuple(q8.shape)}")
    if tuple(vt.shape) != (B, Hkv, nk, D, 64):
        raise RuntimeError(f"V tiles have shape {tuple(vt.shape)}, expected {(B, Hkv, nk, D, 64)} for kv_len {Nk}")
    if tuple(lut.shape) != (B, H, nq, nk) or tuple(valid.shape) != (B, H, nq):
        raise RuntimeError(f"lut / valid_block_num have shapes {tuple(lut.shape)} / {tuple(valid.shape)}, "
                           f"expected {(B, H, nq, nk)} / {(B, H, nq)}")
    nqs = nq * 4 if qk_quant_gran == QUANT_PER_WARP else nq
    if tuple(q_scale.shape) != (B, H, nqs) or tuple(k_scale.shape) != (B, Hkv, nk):
        raise RuntimeError(f"q_scale / k_scale have shapes {tuple(q_scale.shape)} / {tuple(k_scale.shape)}, "
                           f"expected {(B, H, nqs)} / {(B, Hkv, nk)} for qk_quant_gran = {qk_quant_gran}")
    if v_scale is not None and tuple(v_scale.shape) != (B, Hkv, D):
        raise RuntimeError(f"v_scale has shape {tuple(v_scale.shape)}, expected {(B, Hkv, D)}")
    return B, H, Hkv, N, Nk, D


def block_sparse_attn(q8, k8, v8, out, lut, valid, pvthreshd, q_scale, k_scale, v_scale, sm_scale,
                      is_causal=False, return_pv_count=False, pv_mode=PV_PER_BLOCK, qk_quant_gran=QUANT_PER_BLOCK):
    _dev(q8, k8, v8, lut, valid, pvthreshd, q_scale, k_scale, v_scale)
    _dev_strided(out)
    qk_quant_gran = quant_gran(qk_quant_gran)
    B, H, Hkv, N, Nk, D = _check_attn_shapes(q8, k8, v8, lut, valid, q_scale, k_scale, v_scale, qk_quant_gran)
    if tuple(out.shape) != (B, H, N, D) or pvthreshd.numel() != H:
        raise RuntimeError("out must have q's shape and pvthreshd one entry per query head")
    if _torch() is not None:
        pvc = _ops.block_sparse_attn(q8, k8, v8, out, lut, valid, pvthreshd, q_scale, k_scale, v_scale, float(sm_scale),
                                     bool(is_causal), qk_quant_gran, int(pv_mode), bool(return_pv_count))
        return pvc if return_pv_count else None
    pvc = torch.zeros((B, H, 4 * ((N + 127) // 128)), dtype=torch.int32, device=q8.device) if return_pv_count else None
    _check(load().spg_block_sparse_attn(_p(q8), _p(k8), _p(v8), _p(out), _st(out), _dt(out), _p(lut), _p(valid), _p(pvthreshd),
                                        _p(q_scale), _p(k_scale), _p(v_scale), B, H, Hkv, N, Nk, D, float(sm_scale),
                                        int(bool(is_causal)), qk_quant_gran, int(pv_mode), _p(pvc), _stream()))
    return pvc


def v_tiles_f16_swizzled(v, stream=None):
    """v (B,H,N,D) fp16/bf16 -> (B,H,nk,D,64) fp16 V^T tiles, chunk-swizzled, the operand of block_sparse_attn_f16v."""
    _dev_strided(v)
    if _torch() is not None:
        with torch.cuda.stream(stream) if stream is not None else contextlib.nullcontext():
            return _ops.v_tiles_f16(v)
    B, H, N, D = v.shape
    nk = (N + 63) // 64
    vt = torch.empty((B, H, nk, D, 64), dtype=torch.float16, device=v.device)
    _check(load().spg_v_tiles_f16(_p(v), _st(v), _p(vt), B, H, N, D, _dt(v), _stream(stream)))
    return vt


def v_tiles_f16_to_natural(vt):
    """(B,H,nk,D,64) swizzled fp16 tiles -> (B,H,nk*64,D) in natural key order."""
    B, H, nk, D, _ = vt.shape
    d = torch.arange(D, device=vt.device)
    idx = torch.arange(8, device=vt.device)[None, :] ^ ((d >> 1) & 7)[:, None]      # chunk kc sits at slot kc ^ ((d >> 1) & 7)
    t = vt.view(B, H, nk, D, 8, 8)
    nat = torch.gather(t, 4, idx.view(1, 1, 1, D, 8, 1).expand(B, H, nk, D, 8, 8))
    return nat.reshape(B, H, nk, D, 64).permute(0, 1, 2, 4, 3).reshape(B, H, nk * 64, D)


def block_sparse_attn_f16v(q8, k8, vt, out, lut, valid, pvthreshd, q_scale, k_scale, sm_scale, is_causal=False,
                           return_pv_count=False, pv_mode=PV_PER_BLOCK, qk_quant_gran=QUANT_PER_BLOCK):
    _dev(q8, k8, vt, lut, valid, pvthreshd, q_scale, k_scale)
    _dev_strided(out)
    qk_quant_gran = quant_gran(qk_quant_gran)
    B, H, Hkv, N, Nk, D = _check_attn_shapes(q8, k8, vt, lut, valid, q_scale, k_scale, None, qk_quant_gran)
    if tuple(out.shape) != (B, H, N, D) or pvthreshd.numel() != H:
        raise RuntimeError("out must have q's shape and pvthreshd one entry per query head")
    if _torch() is not None:
        pvc = _ops.block_sparse_attn_f16v(q8, k8, vt, out, lut, valid, pvthreshd, q_scale, k_scale, float(sm_scale),
                                          bool(is_causal), qk_quant_gran, int(pv_mode), bool(return_pv_count))
        return pvc if return_pv_count else None
    pvc = torch.zeros((B, H, 4 * ((N + 127) // 128)), dtype=torch.int32, device=q8.device) if return_pv_count else None
    _check(load().spg_block_sparse_attn_f16v(_p(q8), _p(k8), _p(vt), _p(out), _st(out), _dt(out), _p(lut), _p(valid),
                                             _p(pvthreshd), _p(q_scale), _p(k_scale), B, H, Hkv, N, Nk, D, float(sm_scale),
                                             int(bool(is_causal)), qk_quant_gran, int(pv_mode), _p(pvc), _stream()))
    return pvc


def dense_attn_f16(q, k, vt, sm_scale, is_causal=False, out=None):
    """Dense fp16 flash attention (measurement comparator).  vt = v_tiles_f16_swizzled(v)."""
    _dev(q, k, vt)
    assert q.dtype == k.dtype == vt.dtype == torch.float16
    B, H, N, D = q.shape
    if out is None:
        out = torch.empty_like(q)
    if _torch() is not None:
        return _ops.dense_attn_f16(q, k, vt, out, float(sm_scale), bool(is_causal))
    _check(load().spg_dense_attn_f16(_p(q), _p(k), _p(vt), _p(out), B, H, N, D, float(sm_scale),
                                     int(bool(is_causal)), _stream()))
    return out


def selftest_fp8_pack(x, saturate=True):
    """float32 GPU tensor (size a multiple of 4) -> uint8 e4m3 codes from the attention kernel's pack."""
    _dev(x)
    assert x.dtype == torch.float32 and x.numel() % 4 == 0
    if _torch() is not None:
        return _ops.selftest_fp8_pack(x, bool(saturate))
    codes = torch.empty(x.numel(), dtype=torch.uint8, device=x.device)
    _check(load().spg_selftest_fp8_pack(_p(x), _p(codes), x.numel(), int(bool(saturate)), _stream()))
    return codes.view(x.shape)


def selftest_division(n_divisors, seed=1):
    """Returns (comparisons, mismatches) of the shared-reciprocal division against the hardware's IEEE division."""
    counts = torch.zeros(2, dtype=torch.int64, device="cuda")
    if _torch() is not None:
        return tuple(int(c) for c in _ops.selftest_division(counts, int(n_divisors), int(seed)).cpu())
    _check(load().spg_selftest_division(_p(counts), int(n_divisors), int(seed), _stream()))
    return tuple(int(c) for c in counts.cpu())
