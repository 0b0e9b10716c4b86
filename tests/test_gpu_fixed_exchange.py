"""The one-row plain launch adds the K tiles of a column in 64-bit fixed point (one returning atomic per
workgroup and column).  Its unit comes from a sample of the activation row and the column's scale in group 0,
so it is a guess, and a partial sum the guess has no room for goes a slow way round (parked as fp32, marked,
added by the finishing thread).  These tests drive both ways through the C ABI and check them against the
CPU oracle: ragged shapes at one row, activations the sample does not see, scales far from group 0's,
non-finite inputs, and that either way leaves the workspace as it found it.
"""
import numpy as np
import pytest

from mykuiperllama_amd import synth
from tests import helpers as H
from tests.test_gpu_awq_gemv import check_against_oracle, run_awq

pytestmark = pytest.mark.gpu


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


@pytest.fixture(scope="module")
def oracle():
    from oracle import oracle as _o
    return _o


def bf16(v):
    return synth.f32_to_bf16_bits(np.asarray(v, np.float32))


def sampled_positions(K):
    """Elements of the activation row that the kernel's sample reads: eight runs of eight 16-byte pieces."""
    pieces = K // 8
    pos = set()
    for run in range(8):
        for j in range(8):
            pc = min((run * pieces) // 8 + j, pieces - 1)
            pos.update(range(8 * pc, 8 * pc + 8))
    return pos


@pytest.mark.parametrize("K,N,G", [(384, 264, 128), (512, 8, 128), (1056, 1000, 32), (2048, 40, 64), (4096, 2056, 128),
                                   (1536, 784, 256), (8064, 520, 64), (12288, 4104, 128), (640, 256, 128)])
def test_one_row_ragged_shapes_match_the_oracle(capi, torch, oracle, K, N, G):
    """One activation row on column counts that end inside a tile and K that ends inside a workgroup."""
    p = synth.make_awq_problem(f"fixed_ragged_{K}x{N}", 1, K, N, group=G)
    y, _ = run_awq(capi, torch, p)
    check_against_oracle(oracle, p, y)


@pytest.mark.parametrize("K,N", [(512, 32768), (512, 32776), (8064, 264), (8192, 264)])
def test_shapes_at_the_limits_of_the_slot_area_match_the_oracle(capi, torch, oracle, K, N):
    """32768 columns fill the zeroed area with slots and masks, eight more take the ordered exchange; 8064 rows are
    63 K tiles of 128 rows, the most a slot can count, 8192 rows take workgroups of 256 rows."""
    p = synth.make_awq_problem(f"fixed_limit_{K}x{N}", 1, K, N)
    y, (x, qw, sc, qz, ws) = run_awq(capi, torch, p)
    check_against_oracle(oracle, p, y)
    y2 = torch.empty((1, N), dtype=torch.bfloat16, device="cuda")
    capi.gemv_awq_bf16(x, qw, sc, qz, y2, p["group"], ws)
    torch.cuda.synchronize()
    assert np.array_equal(H.bf16_bits(y2, torch), y)


@pytest.mark.parametrize("K,N", [(4096, 1024), (4096, 4096), (12288, 4096), (5120, 10240)])
def test_one_hot_rows_the_sample_does_not_see_are_exact(capi, torch, oracle, K, N):
    """x = e_k with k outside the sample: the unit is the smallest one, the one non-zero partial sum of every
    column takes the slow path, and y is still the dequantised row k bit for bit."""
    p = synth.make_awq_problem(f"fixed_one_hot_{K}x{N}", 1, K, N)
    w_ref = oracle.awq_dequant_bf16(p["qweight"], p["scales"], p["qzeros"], p["group"])
    seen = sampled_positions(K)
    unseen = [k for k in (100, 257, K // 2 + 300, K - 1) if k not in seen]
    assert len(unseen) >= 3
    for k in unseen + [0, K // 8 + 5]:  # the last two are sampled: the fast path, exact as well
        x = np.zeros((1, K), np.uint16)
        x[0, k] = 0x3F80
        y, _ = run_awq(capi, torch, dict(p, x=x))
        assert np.array_equal(y[0], w_ref[k]), f"row {k}"


def test_large_activations_outside_the_sample_take_the_slow_path_and_agree(capi, torch, oracle):
    """Small activations where the sample looks, a few of 10^5 times their size elsewhere: the K tiles that hold
    the large ones overflow the unit and are added from their parked fp32 values, the others in fixed point."""
    K, N = 4096, 2048
    p = synth.make_awq_problem("fixed_outliers", 1, K, N)
    x = synth.bf16_bits_to_f32(p["x"]).copy() * 1e-3
    seen = sampled_positions(K)
    big = [k for k in (70, 700, 1500, 2300, 3900) if k not in seen]
    assert len(big) >= 4
    for i, k in enumerate(big):
        x[0, k] = (-1) ** i * 100.0 * (i + 1)
    q = dict(p, x=bf16(x))
    y, (xd, qw, sc, qz, ws) = run_awq(capi, torch, q)
    check_against_oracle(oracle, q, y)
    # the same launch again on the same workspace, then an ordinary one: nothing was left behind
    y2 = torch.empty((1, N), dtype=torch.bfloat16, device="cuda")
    capi.gemv_awq_bf16(xd, qw, sc, qz, y2, p["group"], ws)
    torch.cuda.synchronize()
    assert np.array_equal(H.bf16_bits(y2, torch), y)
    y3 = torch.empty((1, N), dtype=torch.bfloat16, device="cuda")
    capi.gemv_awq_bf16(H.to_dev_bf16(p["x"], torch), qw, sc, qz, y3, p["group"], ws)
    torch.cuda.synchronize()
    check_against_oracle(oracle, p, H.bf16_bits(y3, torch))


def test_scales_far_above_group_zero_take_the_slow_path_and_agree(capi, torch, oracle):
    """Group 0 of every other column carries the smallest normal fp16 scale, the other groups scales 30 000 times
    larger, and the activations of group 0 are tiny: the unit of those columns is far too small for the partial
    sums of the other groups."""
    K, N = 2048, 1024
    p = synth.make_awq_problem("fixed_scales", 1, K, N)
    scales = p["scales"].copy()
    scales[0, ::2] = 0x0400        # 2^-14
    scales[1:, ::2] = 0x3C00       # 1.0
    x = synth.bf16_bits_to_f32(p["x"]).copy()
    q = dict(p, scales=scales, x=bf16(x * 50.0))
    y, (xd, qw, sc, qz, ws) = run_awq(capi, torch, q)
    check_against_oracle(oracle, q, y)
    y2 = torch.empty((1, N), dtype=torch.bfloat16, device="cuda")
    capi.gemv_awq_bf16(H.to_dev_bf16(p["x"], torch), H.to_dev_i32(p["qweight"], torch), H.to_dev_f16(p["scales"], torch),
                       H.to_dev_i32(p["qzeros"], torch), y2, p["group"], ws)
    torch.cuda.synchronize()
    check_against_oracle(oracle, p, H.bf16_bits(y2, torch))


def test_zero_scales_in_group_zero_and_zero_activations(capi, torch, oracle):
    K, N = 1024, 512
    p = synth.make_awq_problem("fixed_zero", 1, K, N)
    scales = p["scales"].copy()
    scales[0, :] = 0  # the reference magnitude is zero: every non-zero partial sum takes the slow path
    q = dict(p, scales=scales)
    y, _ = run_awq(capi, torch, q)
    check_against_oracle(oracle, q, y)
    y, _ = run_awq(capi, torch, dict(p, x=np.zeros((1, K), np.uint16)))
    assert not y.any()


@pytest.mark.parametrize("bad", ["nan", "inf"])
@pytest.mark.parametrize("where", ["sampled", "unsampled"])
def test_non_finite_activations_reach_every_output_and_leave_the_workspace_clean(capi, torch, oracle, bad, where):
    """A NaN or an infinity in x makes every partial sum of its K tile non-finite (the zero point is taken out as
    (16 + z) * sum x), so every output must be non-finite; the launch after it on the same workspace is exact."""
    K, N = 4096, 1024
    p = synth.make_awq_problem("fixed_nonfinite", 1, K, N)
    seen = sampled_positions(K)
    k = 3 if where == "sampled" else next(k for k in range(200, K) if k not in seen)
    x = p["x"].copy()
    x[0, k] = 0x7FC0 if bad == "nan" else 0x7F80
    y, (xd, qw, sc, qz, ws) = run_awq(capi, torch, dict(p, x=x))
    assert not np.isfinite(H.bf16_to_f64(y)).any()
    y2 = torch.empty((1, N), dtype=torch.bfloat16, device="cuda")
    capi.gemv_awq_bf16(H.to_dev_bf16(p["x"], torch), qw, sc, qz, y2, p["group"], ws)
    torch.cuda.synchronize()
    check_against_oracle(oracle, p, H.bf16_bits(y2, torch))


@pytest.mark.parametrize("K,N", sorted(set(synth.QWEN3_8B.values())) + [(4096, 6144), (8192, 5120)])
def test_fixed_point_and_ordered_exchange_agree_and_share_a_workspace(capi, torch, K, N):
    """The product's launch (fixed point) and the vector kernel with the ordered fp32 exchange (policy 1), turn
    about on one workspace: each repeats its own bits, and the two differ by rounding only."""
    p = synth.make_awq_problem(f"fixed_vs_ordered_{K}x{N}", 1, K, N)
    y_fixed, (x, qw, sc, qz, ws) = run_awq(capi, torch, p)
    outs = {}
    for rep in range(3):
        for policy in (1, 0):
            capi.set_awq_kernel_policy(policy)
            try:
                y = torch.empty((1, N), dtype=torch.bfloat16, device="cuda")
                capi.gemv_awq_bf16(x, qw, sc, qz, y, p["group"], ws)
                torch.cuda.synchronize()
            finally:
                capi.set_awq_kernel_policy(0)
            bits = H.bf16_bits(y, torch)
            assert np.array_equal(outs.setdefault(policy, bits), bits), f"policy {policy}, repetition {rep}"
    assert np.array_equal(outs[0], y_fixed)
    a, b = H.bf16_to_f64(outs[0]), H.bf16_to_f64(outs[1])
    assert H.rel_l2(a, b) <= 1e-3
    assert (outs[0] != outs[1]).mean() <= 0.02  # a bf16 unit here and there, where the two sums straddle a tie


def test_graph_replay_of_the_fixed_point_launch(capi, torch, oracle):
    p = synth.make_awq_problem("fixed_graph", 1, 4096, 4096)
    y_ref, (x, qw, sc, qz, ws) = run_awq(capi, torch, p)
    y = torch.empty((1, p["N"]), dtype=torch.bfloat16, device="cuda")
    side = torch.cuda.Stream()
    with torch.cuda.stream(side):
        capi.gemv_awq_bf16(x, qw, sc, qz, y, p["group"], ws)
        side.synchronize()
        g = torch.cuda.CUDAGraph()
        with torch.cuda.graph(g):
            for _ in range(4):
                capi.gemv_awq_bf16(x, qw, sc, qz, y, p["group"], ws)
        for _ in range(3):
            y.zero_()
            torch.cuda.synchronize()
            g.replay()
            side.synchronize()
            assert np.array_equal(H.bf16_bits(y, torch), y_ref)
    torch.cuda.synchronize()
