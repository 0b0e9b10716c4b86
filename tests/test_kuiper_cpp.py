"""Runs the C++ tests of the kuiper host API (tests/cpp, built into mykuiperllama_amd/lib/test_kuiper).

The C++ runner restates the reference's own gtest cases for Buffer, Tensor and the add operator
(test/test_tensor/test_buffer.cpp, test_tensor.cpp, test/test_op/test_op_add.cpp) and adds the
MatmulLayer cases, which it checks against the CPU oracle linked into the runner.  One process per
group (host-only cases here, GPU cases on the GPU box); each C++ case shows up as its own pytest
case.
"""
import os
import subprocess

import pytest

from mykuiperllama_amd import build

_cache = {}


def _binary():
    if not os.path.exists(build.KUIPER_TEST):
        pytest.fail(f"{build.KUIPER_TEST} has not been built (python -m mykuiperllama_amd.build)")
    return build.KUIPER_TEST


def _list(flag):
    if not os.path.exists(build.KUIPER_TEST):
        return ["<not built>"]
    out = subprocess.run([build.KUIPER_TEST, flag, "--list"], capture_output=True, text=True, timeout=60)
    return [l.strip() for l in out.stdout.splitlines() if l.strip()]


def _run_group(flag):
    if flag not in _cache:
        proc = subprocess.run([_binary(), flag], capture_output=True, text=True, timeout=600)
        results = {}
        for line in proc.stdout.splitlines():
            if line.startswith("[ OK ] "):
                results[line[7:].strip()] = (True, "")
            elif line.startswith("[FAIL] "):
                name, _, why = line[7:].partition(": ")
                results[name.strip()] = (False, why)
        _cache[flag] = (proc.returncode, results, proc.stdout[-4000:], proc.stderr[-2000:])
    return _cache[flag]


@pytest.mark.parametrize("case", _list("--cpu"))
def test_host_cases(case):
    rc, results, out, err = _run_group("--cpu")
    assert case in results, f"{case} did not report (runner exit {rc})\n{out}\n{err}"
    ok, why = results[case]
    assert ok, why


@pytest.mark.gpu
@pytest.mark.parametrize("case", _list("--gpu"))
def test_gpu_cases(case):
    rc, results, out, err = _run_group("--gpu")
    assert case in results, f"{case} did not report (runner exit {rc})\n{out}\n{err}"
    ok, why = results[case]
    assert ok, why


def test_reference_cases_are_all_present():
    """Every gtest case of the reference has a counterpart in the C++ runner."""
    names = set(_list("--cpu")) | set(_list("--gpu"))
    expected = {
        # test/test_tensor/test_buffer.cpp
        "test_buffer.allocate_cpu", "test_buffer.allocate_cuda", "test_buffer.use_external",
        "test_buffer.cuda_memory1", "test_buffer.cuda_memory2", "test_buffer.cuda_memory3",
        # test/test_tensor/test_tensor.cpp (init1..init5 share one body, per device)
        "test_tensor.tensor_base", "test_tensor.clone_cuda", "test_tensor.clone_cpu", "test_tensor.to_cuda",
        "test_tensor.init1_to_init5_cuda", "test_tensor.init6_external_pointer", "test_tensor.dims_stride",
        "test_tensor.assign",
        # test/test_op/test_op_add.cpp
        "test_op_add.add_cuda_no_stream", "test_op_add.add_cuda_stream", "test_op_add.add_cpu",
        "test_op_add.add_cuda_align",
    }
    assert expected <= names, expected - names
