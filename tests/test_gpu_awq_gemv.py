"""GPU parity of the fused INT4 AWQ dequantise+GEMV against the CPU oracle, through the C ABI.

Tolerances (from the path's specification): unpacked codes and dequantised bf16 weights
bit-exact; GEMV outputs within relative L2 <= 1e-3 and max-abs <= 2 bf16 ulp of the output scale
against the oracle's evaluation of w = (q - z) * s rounded to the output type.  Against the
unrounded fp64 value the bf16 store alone contributes ~1.6e-3 relative L2, so that comparison
uses 3e-3 and is there to catch systematic error, not rounding.
"""
import numpy as np
import pytest

from mykuiperllama_amd import synth
from tests import helpers as H

pytestmark = pytest.mark.gpu

REL_L2_ROUNDED = 1e-3
REL_L2_UNROUNDED = 3e-3


@pytest.fixture(scope="module")
def torch():
    import torch as _t
    assert _t.cuda.is_available(), "GPU tests need a visible MI355X"
    return _t


@pytest.fixture(scope="module")
def capi():
    from mykuiperllama_amd import capi as _c
    _c.load()
    return _c


def run_awq(capi, torch, p):
    x = H.to_dev_bf16(p["x"], torch)
    qw = H.to_dev_i32(p["qweight"], torch)
    sc = H.to_dev_f16(p["scales"], torch)
    qz = H.to_dev_i32(p["qzeros"], torch)
    y = torch.full((p["M"], p["N"]), float("nan"), dtype=torch.bfloat16, device="cuda")
    ws = capi.make_workspace(p["M"], p["K"], p["N"])
    capi.gemv_awq_bf16(x, qw, sc, qz, y, p["group"], ws)
    torch.cuda.synchronize()
    return H.bf16_bits(y, torch), (x, qw, sc, qz, ws)


def check_against_oracle(oracle, p, y_bits):
    ref64 = oracle.gemv_awq_f64(p["x"], p["qweight"], p["scales"], p["qzeros"], p["group"])
    ref_rounded = H.bf16_to_f64(oracle.f32_to_bf16(ref64.astype(np.float32)))
    got = H.bf16_to_f64(y_bits)
    assert np.isfinite(got).all()
    scale = np.abs(ref64).max()
    ulp = H.bf16_ulp_of(scale)
    assert H.rel_l2(got, ref_rounded) <= REL_L2_ROUNDED
    assert np.abs(got - ref_rounded).max() <= 2 * ulp
    assert H.rel_l2(got, ref64) <= REL_L2_UNROUNDED


SHAPES_8B = sorted(set(synth.QWEN3_8B.values()))


@pytest.fixture(params=["by_shape", "vector", "mfma"], autouse=True)
def kernel_policy(request, capi):
    """Every test in this file runs under each kernel policy: the product's choice and either product kernel
    forced through the internal entry point."""
    capi.set_awq_kernel_policy({"by_shape": 0, "vector": 1, "mfma": 2}[request.param])
    yield request.param
    capi.set_awq_kernel_policy(0)


SHAPES_32B = sorted(set(synth.QWEN3_32B.values()))
# the launches a decode step fuses along N; 4096 -> 24576 takes the 32-rows-per-lane plan
SHAPES_FUSED = [(4096, 6144), (4096, 24576), (5120, 10240)]


@pytest.mark.parametrize("K,N", [(1024, 2048)] + SHAPES_8B + SHAPES_32B + SHAPES_FUSED)
def test_gemv_m1_matches_oracle(capi, torch, oracle, K, N):
    p = synth.make_awq_problem(f"gemv_m1_{K}x{N}", 1, K, N)
    y, _ = run_awq(capi, torch, p)
    check_against_oracle(oracle, p, y)


@pytest.mark.parametrize("M,K,N", [(M, K, N) for M in (2, 3, 4, 5, 8, 16)
                                   for K, N in [(4096, 4096), (4096, 1024), (12288, 4096), (4096, 12288), (4096, 24576)]] +
                         # the 32B-shaped MLP: K = 25 600 takes the four-step MFMA plan from five rows on
                         [(M, K, N) for M in (2, 8, 16) for K, N in [(5120, 51200), (25600, 5120)]])
def test_gemv_small_batch_matches_oracle(capi, torch, oracle, M, K, N):
    p = synth.make_awq_problem(f"gemv_m{M}_{K}x{N}", M, K, N)
    y, _ = run_awq(capi, torch, p)
    check_against_oracle(oracle, p, y)


def test_one_hot_rows_reproduce_dequantised_weights_bit_exactly(capi, torch, oracle):
    """x = e_k  =>  y == w[k, :] bit for bit (ties the GEMV to the dequant formula)."""
    K, N = 512, 1024
    p = synth.make_awq_problem("one_hot", 1, K, N)
    w_ref = oracle.awq_dequant_bf16(p["qweight"], p["scales"], p["qzeros"], p["group"])
    for k in (0, 1, 7, 8, 127, 128, 255, 300, 511):
        x = np.zeros((1, K), np.uint16)
        x[0, k] = 0x3F80  # 1.0
        q = dict(p, x=x)
        y, _ = run_awq(capi, torch, q)
        assert np.array_equal(y[0], w_ref[k]), f"row {k}"


def test_exact_special_cases(capi, torch, oracle):
    K, N = 1024, 512
    p = synth.make_awq_problem("special", 1, K, N)
    # x == 0  =>  y == +0
    y, _ = run_awq(capi, torch, dict(p, x=np.zeros((1, K), np.uint16)))
    assert not y.any()
    # q == z everywhere  =>  y == 0 up to fp32 rounding of the two partial sums it is the
    # difference of (typical |y| for these inputs is ~1)
    qz_rows = np.repeat(p["qzeros"], p["group"], axis=0)
    y, _ = run_awq(capi, torch, dict(p, qweight=qz_rows))
    assert np.abs(H.bf16_to_f64(y)).max() <= 1e-4
    # s == 1, z == 0, q == 1, x == 1  =>  y == K (exact in bf16 for K = 1024)
    ones = dict(p,
                x=np.full((1, K), 0x3F80, np.uint16),
                qweight=np.full((K, N // 8), 0x11111111, np.int32),
                qzeros=np.zeros((K // p["group"], N // 8), np.int32),
                scales=np.full((K // p["group"], N), 0x3C00, np.uint16))
    y, _ = run_awq(capi, torch, ones)
    assert (H.bf16_to_f64(y) == float(K)).all()


def test_repeated_launches_are_bitwise_identical_and_workspace_reusable(capi, torch):
    p = synth.make_awq_problem("determinism", 1, 12288, 4096)
    y0, (x, qw, sc, qz, ws) = run_awq(capi, torch, p)
    for _ in range(5):
        y = torch.empty((1, p["N"]), dtype=torch.bfloat16, device="cuda")
        capi.gemv_awq_bf16(x, qw, sc, qz, y, p["group"], ws)  # same workspace, no re-init
        torch.cuda.synchronize()
        assert np.array_equal(H.bf16_bits(y, torch), y0)


@pytest.mark.parametrize("K,N,G", [(128, 8, 128), (256, 24, 128), (384, 264, 128), (64, 2056, 32),
                                   (2048, 40, 64), (1024, 512, 256), (1024, 1000, 512), (192, 64, 96)])
def test_ragged_and_small_shapes(capi, torch, oracle, K, N, G):
    p = synth.make_awq_problem(f"ragged_{K}x{N}", 3, K, N, group=G)
    y, _ = run_awq(capi, torch, p)
    check_against_oracle(oracle, p, y)


@pytest.mark.parametrize("M", [6, 9, 16])
@pytest.mark.parametrize("K,N,G", [(1024, 1008, 128), (512, 272, 128), (2048, 48, 64), (256, 16, 128),
                                   (1536, 784, 256), (384, 264, 128), (8192, 512, 128)])
def test_ragged_shapes_with_many_rows(capi, torch, oracle, M, K, N, G):
    """Five to sixteen activation rows on column counts that end inside a tile (and, for the MFMA kernel's
    two-column read-back, inside a pair of threads), on K that one workgroup covers, and on N that only
    the vector kernel takes (not a multiple of sixteen)."""
    p = synth.make_awq_problem(f"ragged_rows_{M}_{K}x{N}", M, K, N, group=G)
    y, _ = run_awq(capi, torch, p)
    check_against_oracle(oracle, p, y)


def test_linearity_in_x_at_full_size(capi, torch):
    """y(a) + y(b) ~= y(a + b) at a full-size shape, a property that needs no oracle."""
    K, N = 4096, 12288
    pa = synth.make_awq_problem("lin_a", 1, K, N)
    xb = synth.make_awq_problem("lin_b", 1, K, N)["x"]
    fa, fb = synth.bf16_bits_to_f32(pa["x"]), synth.bf16_bits_to_f32(xb)
    # keep a + b exactly representable: use power-of-two multiples of one vector
    xb = synth.f32_to_bf16_bits(fa * 0.5)
    xc = synth.f32_to_bf16_bits(fa * 1.5)
    ya, _ = run_awq(capi, torch, pa)
    yb, _ = run_awq(capi, torch, dict(pa, x=xb))
    yc, _ = run_awq(capi, torch, dict(pa, x=xc))
    lhs = H.bf16_to_f64(ya) + H.bf16_to_f64(yb)
    assert H.rel_l2(H.bf16_to_f64(yc), lhs) <= 4e-3  # three bf16 roundings
    del fb


def test_bad_arguments_are_rejected_before_launch(capi, torch):
    p = synth.make_awq_problem("bad", 1, 1024, 64)
    x = H.to_dev_bf16(p["x"], torch)
    qw = H.to_dev_i32(p["qweight"], torch)
    sc = H.to_dev_f16(p["scales"], torch)
    qz = H.to_dev_i32(p["qzeros"], torch)
    y = torch.empty((1, 64), dtype=torch.bfloat16, device="cuda")
    L = capi.load()
    s = torch.cuda.current_stream().cuda_stream
    args = (x.data_ptr(), qw.data_ptr(), sc.data_ptr(), qz.data_ptr(), y.data_ptr())
    small = torch.empty(262144 + 64, dtype=torch.uint8, device="cuda")
    assert L.kx_gemv_awq_bf16(*args, 1, 1024, 64, 128, None, 0, s) == -3     # K is split: needs a workspace
    assert L.kx_gemv_awq_bf16(*args, 1, 1024, 64, 128, small.data_ptr(), small.numel(), s) == -3  # too small
    assert L.kx_gemv_awq_bf16(*args, 0, 1024, 64, 128, None, 0, s) == -2     # M = 0
    assert L.kx_gemv_awq_bf16(*args, 17, 1024, 64, 128, None, 0, s) == -2    # M too large
    assert L.kx_gemv_awq_bf16(*args, 1, 1000, 64, 128, None, 0, s) == -2     # K not a group multiple
    assert L.kx_gemv_awq_bf16(*args, 1, 1024, 60, 128, None, 0, s) == -2     # N not a multiple of 8
    assert L.kx_gemv_awq_bf16(*args, 1, 1024, 64, 48, None, 0, s) == -2      # group not a multiple of 32
    assert L.kx_gemv_awq_bf16(None, *args[1:], 1, 1024, 64, 128, None, 0, s) == -1
    assert L.kx_gemv_awq_bf16(args[0] + 2, *args[1:], 1, 1024, 64, 128, None, 0, s) == -4  # x misaligned
    assert capi.workspace_bytes(1, 1024, 64) > 262144
    assert capi.workspace_bytes(0, 1024, 64) == 0
    torch.cuda.synchronize()


def test_unsplit_k_needs_no_workspace(capi, torch, oracle):
    """K that fits one workgroup is reduced without the exchange: a null workspace is accepted."""
    p = synth.make_awq_problem("unsplit", 2, 256, 512)
    x = H.to_dev_bf16(p["x"], torch)
    qw = H.to_dev_i32(p["qweight"], torch)
    sc = H.to_dev_f16(p["scales"], torch)
    qz = H.to_dev_i32(p["qzeros"], torch)
    y = torch.full((2, 512), float("nan"), dtype=torch.bfloat16, device="cuda")
    capi.gemv_awq_bf16(x, qw, sc, qz, y, p["group"], None)
    torch.cuda.synchronize()
    check_against_oracle(oracle, p, H.bf16_bits(y, torch))
