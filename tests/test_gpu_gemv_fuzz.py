"""Seeded random shapes for the AWQ GEMV entry point against the oracle: every M from 1 to 16, group
sizes 32..256, K any multiple of the group (including K that no workgroup shape divides), N any
multiple of eight (ragged column tiles, N that only the vector kernel takes).  The draw is fixed, so
a failure names its case."""
import random

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


def draw_cases(count, seed):
    rng = random.Random(seed)
    cases = []
    for i in range(count):
        group = rng.choice([32, 64, 128, 128, 128, 256])
        K = group * rng.randint(1, max(1, 4096 // group))
        if i % 5 == 0:  # K that the 384-row workgroup shape divides
            K = max(group, (K // 384) * 384 or 384)
            K -= K % group
            K = max(K, group)
        N = 8 * rng.randint(1, 256)
        if i % 3 == 0:
            N = 16 * rng.randint(1, 128)  # the matrix-core kernel's N
        M = 1 if i % 4 == 1 else rng.randint(1, 16)  # the decode case often
        cases.append((M, K, N, group))
    return cases


CASES = draw_cases(48, 20251125)


@pytest.mark.parametrize("policy", [0, 2])
@pytest.mark.parametrize("M,K,N,group", CASES)
def test_random_shapes_match_the_oracle(capi, torch, oracle, policy, M, K, N, group):
    p = synth.make_awq_problem(f"fuzz_{M}_{K}_{N}_{group}", M, K, N, group=group)
    capi.set_awq_kernel_policy(policy)
    try:
        x = H.to_dev_bf16(p["x"], torch)
        qw = H.to_dev_i32(p["qweight"], torch)
        sc = H.to_dev_f16(p["scales"], torch)
        qz = H.to_dev_i32(p["qzeros"], torch)
        y = torch.full((M, N), float("nan"), dtype=torch.bfloat16, device="cuda")
        ws = capi.make_workspace(M, K, N)
        capi.gemv_awq_bf16(x, qw, sc, qz, y, group, ws)
        capi.gemv_awq_bf16(x, qw, sc, qz, y, group, ws)  # the workspace is left ready for the next launch
        torch.cuda.synchronize()
    finally:
        capi.set_awq_kernel_policy(0)
    got = H.bf16_to_f64(H.bf16_bits(y, torch))
    ref64 = oracle.gemv_awq_f64(p["x"], p["qweight"], p["scales"], p["qzeros"], group)
    ref_rounded = H.bf16_to_f64(oracle.f32_to_bf16(ref64.astype(np.float32)))
    assert np.isfinite(got).all()
    # tolerance of the path: relative L2 1e-3 and two bf16 ulps of the output scale against the rounded reference
    assert H.rel_l2(got, ref_rounded) <= 1e-3
    assert np.abs(got - ref_rounded).max() <= 2 * H.bf16_ulp_of(np.abs(ref64).max())
