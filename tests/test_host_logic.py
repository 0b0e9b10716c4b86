"""CPU-side checks: seeded generators, byte accounting, and the C ABI's symbols and argument
checks (no kernel is launched: every call below returns before it reaches HIP)."""
import ctypes
import os
import re

import numpy as np
import pytest

from mykuiperllama_amd import build, synth

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def test_splitmix64_known_answers():
    out = synth.splitmix64(0, 3)
    assert [hex(int(v)) for v in out] == ["0xe220a8397b1dcdaf", "0x6e789e6aa1b965f4", "0x6c45d188009454f"]


def test_generators_are_deterministic_and_in_range():
    a = synth.make_awq_problem("det", 2, 256, 64)
    b = synth.make_awq_problem("det", 2, 256, 64)
    for k in ("x", "qweight", "scales", "qzeros"):
        assert np.array_equal(a[k], b[k])
    c = synth.make_awq_problem("det2", 2, 256, 64)
    assert not np.array_equal(a["qweight"], c["qweight"])
    s = synth.f16_bits_to_f32(a["scales"])
    assert s.min() >= 0.001 - 1e-6 and s.max() <= 0.02 + 1e-5
    x = synth.bf16_bits_to_f32(synth.make_awq_problem("stat", 1, 65536, 8)["x"])
    assert abs(x.mean()) < 0.02 and abs(x.std() - 1.0) < 0.02
    codes = (synth.random_words(5, 100000).view(np.uint32)[:, None] >> (4 * np.arange(8, dtype=np.uint32))) & 15
    assert np.abs(np.bincount(codes.ravel(), minlength=16) / codes.size - 1 / 16).max() < 0.003


def test_algorithmic_bytes_match_the_published_table():
    assert synth.awq_gemv_bytes(1, 1024, 2048) == 1_095_680
    assert synth.awq_gemv_bytes(1, 4096, 1024) == 2_189_312
    assert synth.awq_gemv_bytes(1, 4096, 4096) == 8_732_672
    assert synth.awq_gemv_bytes(1, 4096, 12288) == 26_181_632
    assert synth.awq_gemv_bytes(1, 12288, 4096) == 26_181_632
    assert sum(synth.awq_gemv_bytes(1, *s) for s in synth.QWEN3_8B.values()) == 100_388_864
    assert synth.bf16_gemv_bytes(1, 4096, 151936) == 2 * 4096 * 151936 + 2 * (4096 + 151936)


def declared_functions():
    text = open(os.path.join(ROOT, "include", "kx_hip.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(kx_[a-z0-9_]+)\s*\(", text)))


@pytest.fixture(scope="module")
def lib():
    if not os.path.exists(build.KX_LIB):
        pytest.fail(f"{build.KX_LIB} has not been built (python -m mykuiperllama_amd.build)")
    from mykuiperllama_amd import capi
    return capi.load()


def test_library_exports_every_declared_symbol(lib):
    from mykuiperllama_amd import capi
    names = declared_functions()
    assert len(names) >= 8
    raw = ctypes.CDLL(build.KX_LIB)
    for n in names:
        assert hasattr(raw, n), f"{n} declared in include/kx_hip.h but not exported"
    assert sorted(capi.SIGNATURES) == names  # the Python binding covers the whole header


def test_abi_version_and_error_strings(lib):
    assert lib.kx_abi_version() == 3  # KX_ABI_VERSION of include/kx_hip.h
    assert lib.kx_error_string(0) == b"ok"
    for code in (-1, -2, -3, -4):
        assert len(lib.kx_error_string(code)) > 5
    assert b"unknown" in lib.kx_error_string(-99)


def test_workspace_size_query(lib):
    assert lib.kx_gemv_workspace_bytes(1, 4096, 4096) >= 262144 + (4096 // 256) * 4096 * 4
    assert lib.kx_gemv_workspace_bytes(16, 12288, 4096) >= 262144 + 16 * (12288 // 256) * 4096 * 4
    assert lib.kx_gemv_workspace_bytes(0, 4096, 4096) == 0
    assert lib.kx_gemv_workspace_bytes(17, 4096, 4096) == 0


def test_argument_checks_return_before_any_launch(lib):
    p = 0x1000  # never dereferenced: every call below is rejected on the host
    assert lib.kx_gemv_awq_bf16(None, p, p, p, p, 1, 256, 64, 128, None, 0, None) == -1
    assert lib.kx_gemv_awq_bf16(p, p, p, p, p, 0, 256, 64, 128, None, 0, None) == -2
    assert lib.kx_gemv_awq_bf16(p, p, p, p, p, 1, 256, 60, 128, None, 0, None) == -2
    assert lib.kx_gemv_awq_bf16(p, p, p, p, p, 1, 200, 64, 128, None, 0, None) == -2
    assert lib.kx_gemv_awq_bf16(p, p, p, p, p, 1, 4096, 64, 128, None, 0, None) == -3
    assert lib.kx_gemv_awq_bf16(p + 2, p, p, p, p, 1, 4096, 64, 128, None, 0, None) == -4
    assert lib.kx_gemv_bf16(None, p, p, 1, 256, 64, None, 0, None) == -1
    assert lib.kx_gemv_bf16(p, p, p, 1, 250, 64, None, 0, None) == -2
    assert lib.kx_gemv_bf16(p, p, p, 17, 256, 64, None, 0, None) == -2
    assert lib.kx_awq_unpack_u8(p, p, 4, 12, None) == -2
    assert lib.kx_awq_unpack_u8(None, None, 0, 8, None) == 0   # empty input: nothing to do
    assert lib.kx_awq_dequant_bf16(p, p, p, None, 256, 64, 128, None) == -1
    assert lib.kx_awq_dequant_bf16(p, p, p, p, 250, 64, 128, None) == -2
    assert lib.kx_workspace_init(None, 1 << 20, None) == -1
    assert lib.kx_workspace_init(p, 16, None) == -3


def test_bench_refuses_more_than_one_gpu():
    import subprocess
    import sys
    r = subprocess.run([sys.executable, os.path.join(ROOT, "bench.py"), "--gpus", "2"],
                       capture_output=True, text=True)
    assert r.returncode != 0 and "one GPU" in r.stderr
