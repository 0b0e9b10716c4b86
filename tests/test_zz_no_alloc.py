"""The entry point that allocates nothing (kx_gemv_awq_bf16_static): same bits as kx_gemv_awq_bf16 with a
caller-provided workspace, on consecutive calls that share the library's static scratch array."""
import numpy as np
import pytest

from mykuiperllama_amd import synth
from tests import helpers as H

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def torch():
    import torch as _t
    assert _t.cuda.is_available()
    return _t


@pytest.fixture(scope="module")
def capi():
    from mykuiperllama_amd import capi as _c
    _c.load()
    return _c


def _both(capi, torch, name, M, K, N):
    p = synth.make_awq_problem(name, M, K, N)
    x = H.to_dev_bf16(p["x"], torch)
    qw = H.to_dev_i32(p["qweight"], torch)
    sc = H.to_dev_f16(p["scales"], torch)
    qz = H.to_dev_i32(p["qzeros"], torch)
    want = torch.full((M, N), float("nan"), dtype=torch.bfloat16, device="cuda")
    got = torch.full((M, N), float("nan"), dtype=torch.bfloat16, device="cuda")
    ws = capi.make_workspace(M, K, N)
    capi.gemv_awq_bf16(x, qw, sc, qz, want, p["group"], ws)
    capi.gemv_awq_bf16_static(x, qw, sc, qz, got, p["group"])
    torch.cuda.synchronize()
    return p, H.bf16_bits(want, torch), H.bf16_bits(got, torch)


def test_static_scratch_entry_point_matches_the_workspace_entry_point(capi, torch, oracle):
    print("no-alloc entry point: 12288x4096 M=1, then 1024x512 M=2, then 4096x12288 M=3", flush=True)
    assert capi.load().kx_gemv_awq_static_scratch_bytes() == 524288 + (8 << 20)
    # two calls in a row on the shared array, the second one smaller, a third one on the MFMA kernel
    for name, M, K, N in (("static_a", 1, 12288, 4096), ("static_b", 2, 1024, 512), ("static_c", 3, 4096, 12288)):
        p, want, got = _both(capi, torch, name, M, K, N)
        assert np.array_equal(want, got), f"{name}: the static-scratch call differs from the workspace call"
        ref64 = oracle.gemv_awq_f64(p["x"], p["qweight"], p["scales"], p["qzeros"], p["group"])
        ref = H.bf16_to_f64(oracle.f32_to_bf16(ref64.astype(np.float32)))
        assert H.rel_l2(H.bf16_to_f64(got), ref) <= 1e-3  # the path's tolerance against the oracle
    # and the same first shape again: nothing of the calls in between is left in the array
    p, want, got = _both(capi, torch, "static_a", 1, 12288, 4096)
    assert np.array_equal(want, got)


def test_static_scratch_entry_point_rejects_what_does_not_fit(capi, torch):
    L = capi.load()
    s = torch.cuda.current_stream().cuda_stream
    M, K, N = 16, 25600, 5120  # partial sums of this call would need far more than 8 MiB
    assert capi.workspace_bytes(M, K, N) > L.kx_gemv_awq_static_scratch_bytes()
    x = torch.zeros((M, K), dtype=torch.bfloat16, device="cuda")
    qw = torch.zeros((K, N // 8), dtype=torch.int32, device="cuda")
    sc = torch.ones((K // 128, N), dtype=torch.float16, device="cuda")
    qz = torch.zeros((K // 128, N // 8), dtype=torch.int32, device="cuda")
    y = torch.full((M, N), 7.0, dtype=torch.bfloat16, device="cuda")
    args = (x.data_ptr(), qw.data_ptr(), sc.data_ptr(), qz.data_ptr(), y.data_ptr())
    assert L.kx_gemv_awq_bf16_static(*args, M, K, N, 128, s) == -3
    assert L.kx_gemv_awq_bf16_static(None, *args[1:], 1, K, N, 128, s) == -1
    assert L.kx_gemv_awq_bf16_static(*args, 1, K, N, 100, s) == -2
    assert L.kx_gemv_awq_bf16_static(args[0] + 2, *args[1:], 1, K, N, 128, s) == -4  # x not 16-byte aligned
    # the fused 8B shapes at several rows are past the array as well: gate|up 4096 -> 24576 at four rows
    assert capi.workspace_bytes(4, 4096, 24576) > L.kx_gemv_awq_static_scratch_bytes()
    torch.cuda.synchronize()
    assert bool((y == 7.0).all())  # nothing was launched
