"""GPU parity of the export kernels (bit-exact) and of the BF16 GEMV fallback."""
import numpy as np
import pytest

from mykuiperllama_amd import synth
from tests import helpers as H

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


@pytest.mark.parametrize("K,N", [(1024, 2048), (4096, 1024), (256, 8), (128, 24)])
def test_unpack_is_bit_exact(capi, torch, oracle, K, N):
    p = synth.make_awq_problem(f"unpack_{K}x{N}", 1, K, N)
    words = H.to_dev_i32(p["qweight"], torch)
    codes = torch.full((K, N), 255, dtype=torch.uint8, device="cuda")
    capi.awq_unpack_u8(words, codes)
    torch.cuda.synchronize()
    assert np.array_equal(codes.cpu().numpy(), oracle.awq_unpack(p["qweight"]))


def test_unpack_known_answer_word(capi, torch):
    words = torch.tensor([[0x76543210]], dtype=torch.int32, device="cuda")
    codes = torch.zeros((1, 8), dtype=torch.uint8, device="cuda")
    capi.awq_unpack_u8(words, codes)
    torch.cuda.synchronize()
    # nibble i holds column ORDER[i] = (0,2,4,6,1,3,5,7): column c reads nibble INV[c]
    assert codes.cpu().tolist() == [[0, 4, 1, 5, 2, 6, 3, 7]]


@pytest.mark.parametrize("K,N,G", [(1024, 2048, 128), (4096, 4096, 128), (256, 24, 64)])
def test_dequant_is_bit_exact(capi, torch, oracle, K, N, G):
    p = synth.make_awq_problem(f"dequant_{K}x{N}", 1, K, N, group=G)
    w = torch.zeros((K, N), dtype=torch.bfloat16, device="cuda")
    capi.awq_dequant_bf16(H.to_dev_i32(p["qweight"], torch), H.to_dev_f16(p["scales"], torch),
                          H.to_dev_i32(p["qzeros"], torch), w, G)
    torch.cuda.synchronize()
    ref = oracle.awq_dequant_bf16(p["qweight"], p["scales"], p["qzeros"], G)
    assert np.array_equal(H.bf16_bits(w, torch), ref)


def test_dequant_exhaustive_over_q_z_and_every_fp16_scale(capi, torch, oracle):
    """16 x 16 (q, z) pairs times all 65536 fp16 bit patterns, NaN compared as NaN."""
    # one group of 128 rows is enough: rows carry q, the group carries one z per column
    N = 65536
    scales = np.arange(N, dtype=np.uint32).astype(np.uint16).reshape(1, N)
    sc = H.to_dev_f16(scales, torch)
    for z in range(16):
        zw = np.full((1, N // 8), z * 0x11111111, np.uint32).view(np.int32)
        qrows = np.zeros((128, N // 8), np.uint32)
        for q in range(16):
            qrows[q, :] = q * 0x11111111
        w = torch.zeros((128, N), dtype=torch.bfloat16, device="cuda")
        capi.awq_dequant_bf16(H.to_dev_i32(qrows.view(np.int32), torch), sc, H.to_dev_i32(zw, torch), w, 128)
        torch.cuda.synchronize()
        got = H.bf16_bits(w, torch)[:16]
        ref = oracle.awq_dequant_bf16(qrows.view(np.int32), scales, zw, 128)[:16]
        nan_ref = (ref & 0x7FFF) > 0x7F80
        nan_got = (got & 0x7FFF) > 0x7F80
        assert np.array_equal(nan_ref, nan_got)
        assert np.array_equal(got[~nan_ref], ref[~nan_ref]), f"z={z}"


@pytest.mark.parametrize("M", [1, 2, 3, 4, 7, 8, 9, 12, 16])  # 8 | 9: one block of sixteen columns | four blocks per workgroup
@pytest.mark.parametrize("K,N", [(4096, 4096), (1024, 3000), (5120, 1001)])
def test_bf16_gemv_matches_oracle(capi, torch, oracle, M, K, N):
    p = synth.make_bf16_problem(f"bf16_{M}_{K}x{N}", M, K, N)
    x = H.to_dev_bf16(p["x"], torch)
    w = H.to_dev_bf16(p["w"], torch)
    y = torch.full((M, N), float("nan"), dtype=torch.bfloat16, device="cuda")
    capi.gemv_bf16(x, w, y)
    torch.cuda.synchronize()
    ref64 = oracle.gemv_bf16_f64(p["x"], p["w"])
    ref_rounded = H.bf16_to_f64(oracle.f32_to_bf16(ref64.astype(np.float32)))
    got = H.bf16_to_f64(H.bf16_bits(y, torch))
    assert H.rel_l2(got, ref_rounded) <= 1e-3
    assert np.abs(got - ref_rounded).max() <= 2 * H.bf16_ulp_of(np.abs(ref64).max())


@pytest.mark.parametrize("M", [1, 2, 3, 5, 8, 9, 12, 16])
@pytest.mark.parametrize("K,N", [(8, 1), (40, 15), (1000, 17), (4104, 1001), (72, 64)])
def test_bf16_gemv_ragged_shapes(capi, torch, oracle, M, K, N):
    """K that is a multiple of eight but not of a sweep or of a 32-element MFMA step, N below and just past a
    tile of sixteen rows, for the one-row, two-row and matrix-core kernels."""
    p = synth.make_bf16_problem(f"bf16_ragged_{M}_{K}x{N}", M, K, N)
    y = torch.full((M, N), float("nan"), dtype=torch.bfloat16, device="cuda")
    capi.gemv_bf16(H.to_dev_bf16(p["x"], torch), H.to_dev_bf16(p["w"], torch), y)
    torch.cuda.synchronize()
    ref64 = oracle.gemv_bf16_f64(p["x"], p["w"])
    ref_rounded = H.bf16_to_f64(oracle.f32_to_bf16(ref64.astype(np.float32)))
    got = H.bf16_to_f64(H.bf16_bits(y, torch))
    assert np.isfinite(got).all()
    assert H.rel_l2(got, ref_rounded) <= 1e-3
    assert np.abs(got - ref_rounded).max() <= 2 * H.bf16_ulp_of(np.abs(ref64).max())


@pytest.mark.parametrize("M", [1, 16])
def test_bf16_gemv_at_the_size_of_the_qwen3_lm_head(capi, torch, oracle, M):
    """K = 4096, N = 151 936 (37 984 workgroups at one row): a strided subset of 4 748 output rows plus the rows
    of the first and the last workgroups against the oracle, everything else checked to be finite."""
    K, N = 4096, 151936
    gen = torch.Generator(device="cuda")
    gen.manual_seed(424242 + M)
    w = (torch.randn((N, K), device="cuda", generator=gen) * 0.02).bfloat16()
    x = torch.randn((M, K), device="cuda", generator=gen).bfloat16()
    y = torch.full((M, N), float("nan"), dtype=torch.bfloat16, device="cuda")
    capi.gemv_bf16(x, w, y)
    torch.cuda.synchronize()
    assert torch.isfinite(y.float()).all()
    rows = np.unique(np.concatenate([np.arange(0, N, 32), np.arange(0, 64), np.arange(N - 64, N)]))
    assert len(rows) >= 4096
    idx = torch.from_numpy(rows).cuda()
    w_sub = H.bf16_bits(w.index_select(0, idx), torch)
    ref64 = oracle.gemv_bf16_f64(H.bf16_bits(x, torch), w_sub)
    ref_rounded = H.bf16_to_f64(oracle.f32_to_bf16(ref64.astype(np.float32)))
    got = H.bf16_to_f64(H.bf16_bits(y.index_select(1, idx), torch))
    assert H.rel_l2(got, ref_rounded) <= 1e-3
    assert np.abs(got - ref_rounded).max() <= 2 * H.bf16_ulp_of(np.abs(ref64).max())


def test_bf16_gemv_one_hot_returns_the_weight_column_exactly(capi, torch):
    K, N = 1024, 512
    p = synth.make_bf16_problem("bf16_onehot", 1, K, N)
    w = H.to_dev_bf16(p["w"], torch)
    for k in (0, 5, 511, 1023):
        xb = np.zeros((1, K), np.uint16)
        xb[0, k] = 0x3F80
        y = torch.empty((1, N), dtype=torch.bfloat16, device="cuda")
        capi.gemv_bf16(H.to_dev_bf16(xb, torch), w, y)
        torch.cuda.synchronize()
        assert np.array_equal(H.bf16_bits(y, torch)[0], p["w"][:, k])


def test_gpu_reproduces_golden_fixture(capi, torch):
    """The committed fixture (numpy restatement of the layout + torch's bf16 cast) end to end."""
    import os
    g = np.load(os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "awq_small.npz"))
    group = int(g["group"])
    K, N = g["codes"].shape
    qw, qz = H.to_dev_i32(g["qweight"], torch), H.to_dev_i32(g["qzeros"], torch)
    sc = H.to_dev_f16(g["scales"], torch)
    codes = torch.zeros((K, N), dtype=torch.uint8, device="cuda")
    capi.awq_unpack_u8(qw, codes)
    zc = torch.zeros(tuple(g["zero_codes"].shape), dtype=torch.uint8, device="cuda")
    capi.awq_unpack_u8(qz, zc)
    w = torch.zeros((K, N), dtype=torch.bfloat16, device="cuda")
    capi.awq_dequant_bf16(qw, sc, qz, w, group)
    x = H.to_dev_bf16(g["x"], torch)
    y = torch.zeros((x.shape[0], N), dtype=torch.bfloat16, device="cuda")
    capi.gemv_awq_bf16(x, qw, sc, qz, y, group, capi.make_workspace(x.shape[0], K, N))
    torch.cuda.synchronize()
    assert np.array_equal(codes.cpu().numpy(), g["codes"])
    assert np.array_equal(zc.cpu().numpy(), g["zero_codes"])
    assert np.array_equal(H.bf16_bits(w, torch), g["w_bf16"])
    got = H.bf16_to_f64(H.bf16_bits(y, torch))
    ref = H.bf16_to_f64(synth.f32_to_bf16_bits(g["y_f64"].astype(np.float32)))
    assert H.rel_l2(got, ref) <= 1e-3
    assert np.abs(got - ref).max() <= 2 * H.bf16_ulp_of(np.abs(g["y_f64"]).max())
