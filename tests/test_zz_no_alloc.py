"""spg_km_mean_static - the entry point that allocates nothing - against spg_km_mean, through the C ABI.

Collected last on purpose (the file name sorts after every other test file): it must pass both alone in a fresh
process and after the rest of the suite has used the library.
"""
import ctypes

import pytest
import torch

from spargeattn_amd import _lib
from gpu_common import rand_T

pytestmark = pytest.mark.gpu


def _static_mean(k):
    """Calls the C ABI directly: only the OUTPUT is allocated here (by the caller, as for every entry point)."""
    B, H, N, D = k.shape
    km = torch.empty((B, H, 1, D), dtype=k.dtype, device=k.device)
    lib = _lib.load()
    rc = lib.spg_km_mean_static(k.data_ptr(), _lib._st(k), km.data_ptr(), B, H, N, D, _lib._dt(k),
                                torch.cuda.current_stream().cuda_stream)
    assert rc == _lib.SPG_OK, lib.spg_last_error().decode()
    return km


def test_static_scratch_mean_matches_the_workspace_variant_on_two_calls_in_a_row():
    big = rand_T((2, 8, 5000, 128), torch.bfloat16, 301, shift=0.7)
    small = rand_T((1, 3, 333, 64), torch.float16, 302, shift=-0.2)      # second call: smaller input, other dtype / head_dim
    want_big, want_small = _lib.km_mean(big), _lib.km_mean(small)
    got_big = _static_mean(big)
    got_small = _static_mean(small)
    torch.cuda.synchronize()
    assert torch.equal(got_big.view(torch.int16), want_big.view(torch.int16))
    assert torch.equal(got_small.view(torch.int16), want_small.view(torch.int16))
    # and once more in the other order, on a strided (NHD) view
    nhd = rand_T((1, 700, 4, 64), torch.bfloat16, 303).transpose(1, 2)
    assert torch.equal(_static_mean(nhd), _lib.km_mean(nhd))
    assert torch.equal(_static_mean(big), want_big)


def test_static_scratch_mean_allocates_nothing_and_runs_under_graph_capture():
    """The property the entry point exists for: no device memory is taken by a call, and the call can be recorded into
    a HIP graph (plain kernel launches only) and replayed, each replay giving the bits of spg_km_mean."""
    k = rand_T((1, 4, 2048, 128), torch.bfloat16, 311, shift=0.3)
    km = torch.empty((1, 4, 1, 128), dtype=k.dtype, device=k.device)
    lib = _lib.load()

    def call(stream):
        rc = lib.spg_km_mean_static(k.data_ptr(), None, km.data_ptr(), 1, 4, 2048, 128, _lib._dt(k), stream)
        assert rc == _lib.SPG_OK, lib.spg_last_error().decode()

    call(torch.cuda.current_stream().cuda_stream)          # warm-up: the array's address is looked up here
    torch.cuda.synchronize()
    want = _lib.km_mean(k)
    torch.cuda.synchronize()
    free_before, _ = torch.cuda.mem_get_info()
    call(torch.cuda.current_stream().cuda_stream)
    torch.cuda.synchronize()
    free_after, _ = torch.cuda.mem_get_info()
    assert free_after == free_before                       # neither the driver's nor torch's pool grew
    assert torch.equal(km.view(torch.int16), want.view(torch.int16))

    g = torch.cuda.CUDAGraph()
    km.zero_()
    torch.cuda.synchronize()
    with torch.cuda.graph(g):
        call(torch.cuda.current_stream().cuda_stream)
    for shift in (0.3, -1.5, 4.0):                         # replays with other contents, eager work in between
        k.copy_(rand_T((1, 4, 2048, 128), torch.bfloat16, 312, shift=shift))
        want = _lib.km_mean(k)
        km.zero_()
        g.replay()
        torch.cuda.synchronize()
        assert torch.equal(km.view(torch.int16), want.view(torch.int16)), shift


def test_static_scratch_mean_refuses_shapes_beyond_its_array():
    lib = _lib.load()
    rc = lib.spg_km_mean_static(1, None, 1, 1, 8193, 128, 128, 0, None)       # 8193 heads x 128 x 8 B > 8 MiB
    assert rc == _lib.SPG_ERR_UNSUPPORTED and b"scratch" in lib.spg_last_error()
