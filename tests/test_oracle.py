"""Pins the CPU oracle (oracle/kx_oracle.c) without a GPU.

The reference tree holds no implementation, vector or test of this arithmetic, so the pins are:
library casts for the 16-bit float conversions (exhaustive), an independent numpy restatement of
the layout (tests/spec_numpy.py), the committed fixture tests/golden/awq_small.npz, and what the
closed form w = (q - z) * s fixes on its own (invariants, exact special cases).
"""
import os

import numpy as np
import pytest
import torch
from hypothesis import given, settings, strategies as st

from mykuiperllama_amd import synth
from tests import helpers as H
from tests import spec_numpy as spec

GOLDEN = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "awq_small.npz")


def is_nan_bf16(b):
    return (b & 0x7FFF) > 0x7F80


def is_nan_f16(b):
    return (b & 0x7FFF) > 0x7C00


# ------------------------------------------------------------------ conversions
def test_bf16_to_f32_all_patterns_match_torch(oracle):
    bits = np.arange(65536, dtype=np.uint32).astype(np.uint16)
    got = oracle.bf16_to_f32(bits)
    ref = torch.from_numpy(bits.view(np.int16)).view(torch.bfloat16).float().numpy()
    assert np.array_equal(got.view(np.uint32), ref.view(np.uint32))


def test_f16_to_f32_all_patterns_match_numpy(oracle):
    bits = np.arange(65536, dtype=np.uint32).astype(np.uint16)
    got = oracle.f16_to_f32(bits)
    ref = bits.view(np.float16).astype(np.float32)
    nan = np.isnan(ref)
    assert np.array_equal(np.isnan(got), nan)
    assert np.array_equal(got.view(np.uint32)[~nan], ref.view(np.uint32)[~nan])


def _float_test_set():
    rng = np.random.default_rng(7)
    parts = [rng.integers(0, 2**32, 2_000_000, dtype=np.uint64).astype(np.uint32)]
    # every bf16 / fp16 value, and every midpoint between neighbours (ties)
    b = np.arange(65536, dtype=np.uint32) << 16
    parts += [b, b | 0x8000, b | 0x7FFF, b | 0x8001]
    h = np.arange(65536, dtype=np.uint32).astype(np.uint16).view(np.float16).astype(np.float32).view(np.uint32)
    parts += [h, h + 0x1000, h + 0x0FFF, h + 0x1001]
    # around the fp16 subnormal / overflow boundaries
    edges = np.array([2.0**-24, 2.0**-25, 2.0**-25 * 1.0000001, 2.0**-26, 65504.0, 65519.9, 65520.0,
                      65536.0, 1e-8, 6.1e-5, 6.0e-5, 0.0], np.float32)
    parts += [edges.view(np.uint32), (-edges).view(np.uint32)]
    return np.concatenate(parts).view(np.float32)


def test_f32_to_bf16_matches_torch(oracle):
    f = _float_test_set()
    got = oracle.f32_to_bf16(f)
    ref = torch.from_numpy(f).to(torch.bfloat16).view(torch.int16).numpy().view(np.uint16)
    nan = np.isnan(f)
    assert is_nan_bf16(got[nan]).all()
    assert np.array_equal(got[~nan], ref[~nan])
    # the numpy rounding used by the input generator agrees as well (finite inputs)
    fin = np.isfinite(f)
    assert np.array_equal(synth.f32_to_bf16_bits(f[fin]), ref[fin])


def test_f32_to_f16_matches_numpy(oracle):
    f = _float_test_set()
    got = oracle.f32_to_f16(f)
    with np.errstate(over="ignore"):
        ref = f.astype(np.float16).view(np.uint16)
    nan = np.isnan(f)
    assert is_nan_f16(got[nan]).all()
    assert np.array_equal(got[~nan], ref[~nan])


# ------------------------------------------------------------------ nibble stream
def test_unpack_known_answer_word(oracle):
    codes = oracle.awq_unpack(np.array([[0x76543210]], np.int32))
    # nibble i = i sits in column ORDER[i]
    assert codes.tolist() == [[0, 4, 1, 5, 2, 6, 3, 7]]
    for i, col in enumerate(spec.ORDER):
        assert codes[0, col] == i


def test_unpack_treats_the_sign_bit_as_payload(oracle):
    # 0xFFFFFFFF is the int32 -1: eight codes of 15, the top nibble included.
    assert oracle.awq_unpack(np.array([[-1]], np.int32)).tolist() == [[15] * 8]
    assert oracle.awq_pack(np.full((1, 8), 15, np.uint8)).view(np.uint32).tolist() == [[0xFFFFFFFF]]
    # 0x80000000: only nibble 7 (column ORDER[7] = 7) is set, to 8.
    assert oracle.awq_unpack(np.array([[-2**31]], np.int32)).tolist() == [[0, 0, 0, 0, 0, 0, 0, 8]]


def test_pack_every_position_and_code(oracle):
    for col in range(8):
        for code in range(16):
            c = np.zeros((1, 8), np.uint8)
            c[0, col] = code
            w = int(oracle.awq_pack(c).view(np.uint32)[0, 0])
            nib = spec.ORDER.index(col)
            assert w == code << (4 * nib)
            assert np.array_equal(oracle.awq_unpack(np.array([[w]], np.uint32).view(np.int32)), c)


def test_pack_unpack_match_numpy_restatement(oracle):
    words = synth.random_words(123, 64 * 40).reshape(64, 40)
    assert np.array_equal(oracle.awq_unpack(words), spec.unpack(words))
    codes = spec.unpack(words)
    assert np.array_equal(oracle.awq_pack(codes), spec.pack(codes))
    assert np.array_equal(oracle.awq_pack(codes), words)


@settings(max_examples=60, deadline=None)
@given(st.integers(1, 6), st.integers(1, 6), st.integers(0, 2**32 - 1))
def test_unpack_inverts_pack(oracle, rows, wcols, seed):
    codes = np.random.default_rng(seed).integers(0, 16, (rows, wcols * 8), dtype=np.uint8)
    assert np.array_equal(oracle.awq_unpack(oracle.awq_pack(codes)), codes)


def test_pack_rejects_bad_input(oracle):
    with pytest.raises(ValueError):
        oracle.awq_pack(np.full((1, 8), 16, np.uint8))
    with pytest.raises(ValueError):
        oracle.awq_pack(np.zeros((1, 12), np.uint8))
    assert oracle.awq_pack(np.zeros((0, 8), np.uint8)).shape == (0, 1)


# ------------------------------------------------------------------ dequant
def test_dequant_exhaustive_q_z_scale(oracle):
    """16 x 16 x 65536 cases against torch's bf16 cast of the exact product."""
    N = 65536
    scales = np.arange(N, dtype=np.uint32).astype(np.uint16).reshape(1, N)
    s32 = scales.view(np.float16).astype(np.float32)
    qrows = np.zeros((128, N // 8), np.uint32)
    for q in range(16):
        qrows[q, :] = q * 0x11111111
    for z in range(16):
        zw = np.full((1, N // 8), z * 0x11111111, np.uint32).view(np.int32)
        got = oracle.awq_dequant_bf16(qrows.view(np.int32), scales, zw, 128)[:16]
        d = (np.arange(16, dtype=np.float32) - np.float32(z)).reshape(16, 1)
        with np.errstate(invalid="ignore"):
            prod = d * s32  # exact in fp32: |d| <= 15, 11-bit significand
        ref = torch.from_numpy(prod).to(torch.bfloat16).view(torch.int16).numpy().view(np.uint16)
        nan = np.isnan(prod)
        assert is_nan_bf16(got[nan]).all()
        assert np.array_equal(got[~nan], ref[~nan]), f"z={z}"


def test_dequant_invariants(oracle):
    rng = np.random.default_rng(3)
    for sbits in [0x3C00, 0x0001, 0x03FF, 0x7BFF, 0x1234, 0xB456] + list(rng.integers(0, 0x7C00, 50)):
        sbits = int(sbits)
        for q in range(16):
            for z in range(16):
                w = oracle.awq_dequant_one(q, z, sbits)
                if q == z:
                    assert (w & 0x7FFF) == 0
                else:
                    assert w == (oracle.awq_dequant_one(z, q, sbits) ^ 0x8000)  # antisymmetry
                if sbits == 0x3C00:  # s = 1: w = q - z exactly
                    assert H.bf16_to_f64(np.array([w], np.uint16))[0] == q - z


# ------------------------------------------------------------------ golden fixture
def test_oracle_reproduces_golden_fixture(oracle):
    g = np.load(GOLDEN)
    group = int(g["group"])
    assert np.array_equal(oracle.awq_unpack(g["qweight"]), g["codes"])
    assert np.array_equal(oracle.awq_unpack(g["qzeros"]), g["zero_codes"])
    assert np.array_equal(oracle.awq_dequant_bf16(g["qweight"], g["scales"], g["qzeros"], group), g["w_bf16"])
    y = oracle.gemv_awq_f64(g["x"], g["qweight"], g["scales"], g["qzeros"], group)
    assert np.allclose(y, g["y_f64"], rtol=1e-12, atol=1e-12)


def test_fixture_generator_is_reproducible():
    """The seeded generator still produces the tensors the fixture was built from."""
    g = np.load(GOLDEN)
    p = synth.make_awq_problem("golden_small", 2, 256, 64, group=128)
    for k in ("x", "qweight", "scales", "qzeros"):
        assert np.array_equal(p[k], g[k]), k


# ------------------------------------------------------------------ AWQ GEMV
@pytest.mark.parametrize("M,K,N,G", [(1, 128, 8, 128), (3, 256, 16, 128), (2, 128, 24, 32), (1, 512, 40, 64)])
def test_gemv_f64_matches_numpy_brute_force(oracle, M, K, N, G):
    p = synth.make_awq_problem(f"brute_{M}_{K}_{N}", M, K, N, group=G)
    got = oracle.gemv_awq_f64(p["x"], p["qweight"], p["scales"], p["qzeros"], G)
    ref = spec.gemv_awq_f64(p["x"], p["qweight"], p["scales"], p["qzeros"], G)
    assert np.allclose(got, ref, rtol=1e-12, atol=1e-13)


def test_gemv_tiny_pure_python_loops(oracle):
    """K = 128, N = 8 by explicit Python loops over the definition."""
    p = synth.make_awq_problem("py_loops", 1, 128, 8)
    qw = p["qweight"].view(np.uint32)
    zw = int(p["qzeros"].view(np.uint32)[0, 0])
    ref = [0.0] * 8
    for k in range(128):
        xv = float(spec.bf16_bits_to_f64(p["x"][0, k:k + 1])[0])
        for i in range(8):
            n = spec.ORDER[i]
            q = (int(qw[k, 0]) >> (4 * i)) & 15
            z = (zw >> (4 * i)) & 15
            s = float(spec.f16_bits_to_f64(p["scales"][0, n:n + 1])[0])
            ref[n] += xv * (q - z) * s
    got = oracle.gemv_awq_f64(p["x"], p["qweight"], p["scales"], p["qzeros"], 128)[0]
    assert np.allclose(got, ref, rtol=1e-12, atol=1e-14)


def test_gemv_exact_special_cases(oracle):
    K, N = 1024, 64
    p = synth.make_awq_problem("special_cpu", 1, K, N)
    w = oracle.awq_dequant_bf16(p["qweight"], p["scales"], p["qzeros"], 128)
    for k in (0, 127, 128, 1023):  # one-hot x picks row k of the dequantised weights, bit for bit
        x = np.zeros((1, K), np.uint16)
        x[0, k] = 0x3F80
        assert np.array_equal(oracle.gemv_awq_f32(x, p["qweight"], p["scales"], p["qzeros"], 128)[0], w[k])
    zero = oracle.gemv_awq_f32(np.zeros((1, K), np.uint16), p["qweight"], p["scales"], p["qzeros"], 128)
    assert not zero.any()
    same = oracle.gemv_awq_f64(p["x"], np.repeat(p["qzeros"], 128, axis=0), p["scales"], p["qzeros"], 128)
    assert not same.any()
    ones = oracle.gemv_awq_f32(np.full((1, K), 0x3F80, np.uint16), np.full((K, N // 8), 0x11111111, np.int32),
                               np.full((K // 128, N), 0x3C00, np.uint16), np.zeros((K // 128, N // 8), np.int32), 128)
    assert (H.bf16_to_f64(ones) == K).all()


def test_gemv_linearity_and_f32_vs_f64(oracle):
    K, N = 4096, 256
    p = synth.make_awq_problem("lin_cpu", 2, K, N)
    y = oracle.gemv_awq_f64(p["x"], p["qweight"], p["scales"], p["qzeros"], 128)
    xa = synth.bf16_bits_to_f32(p["x"][0:1])
    x2 = synth.f32_to_bf16_bits(xa * 2.0)  # exact
    y2 = oracle.gemv_awq_f64(x2, p["qweight"], p["scales"], p["qzeros"], 128)
    assert np.allclose(y2[0], 2.0 * y[0], rtol=1e-13)
    y32 = H.bf16_to_f64(oracle.gemv_awq_f32(p["x"], p["qweight"], p["scales"], p["qzeros"], 128))
    rounded = H.bf16_to_f64(oracle.f32_to_bf16(y.astype(np.float32)))
    assert H.rel_l2(y32, rounded) < 1e-3
    assert H.rel_l2(y32, y) < 3e-3  # bf16 store alone is ~1.6e-3


def test_gemv_rejects_inconsistent_shapes(oracle):
    p = synth.make_awq_problem("reject", 1, 256, 16)
    with pytest.raises(ValueError):
        oracle.gemv_awq_f64(p["x"], p["qweight"], p["scales"][:1], p["qzeros"], 128)
    with pytest.raises(ValueError):
        oracle.gemv_awq_f64(p["x"], p["qweight"], p["scales"], p["qzeros"], 100)


# ------------------------------------------------------------------ BF16 GEMV
@pytest.mark.parametrize("M,K,N", [(1, 256, 33), (4, 1024, 17)])
def test_bf16_gemv_matches_torch(oracle, M, K, N):
    p = synth.make_bf16_problem(f"bf16_cpu_{M}", M, K, N)
    xt = torch.from_numpy(p["x"].view(np.int16)).view(torch.bfloat16).double()
    wt = torch.from_numpy(p["w"].view(np.int16)).view(torch.bfloat16).double()
    ref = (xt @ wt.T).numpy()
    assert np.allclose(oracle.gemv_bf16_f64(p["x"], p["w"]), ref, rtol=1e-12, atol=1e-14)
    got = H.bf16_to_f64(oracle.gemv_bf16_f32(p["x"], p["w"]))
    assert H.rel_l2(got, ref) < 3e-3
    x1 = np.zeros((1, K), np.uint16)
    x1[0, 5] = 0x3F80
    assert np.array_equal(oracle.gemv_bf16_f32(x1, p["w"])[0], p["w"][:, 5])


def test_threaded_fp32_gemv_returns_the_single_thread_bits(oracle):
    """The column-range entry point is the body of the full-range one: any split gives the same bits."""
    from mykuiperllama_amd import synth
    p = synth.make_awq_problem("threads", 2, 512, 1064, 128)
    one = oracle.gemv_awq_f32(p["x"], p["qweight"], p["scales"], p["qzeros"], p["group"])
    for threads in (1, 2, 3, 7, 133, 1000):
        many = oracle.gemv_awq_f32_threads(p["x"], p["qweight"], p["scales"], p["qzeros"], p["group"], threads)
        assert np.array_equal(one, many), threads
