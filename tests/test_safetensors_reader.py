"""The C++ checkpoint reader against an independent writer: files written by the `safetensors`
package (torch tensors, including bf16) are listed by kx_safetensors_dump, which prints what
model::SafetensorsFile sees; names, dtypes, shapes, byte counts and an FNV-1a checksum of every
tensor's bytes must agree with the tensors that went in."""
import os
import subprocess

import numpy as np
import pytest

from mykuiperllama_amd import build, synth


def fnv1a64(data: bytes) -> int:
    h = 1469598103934665603
    # vectorised in chunks would change nothing about the definition; files here are small
    for b in data:
        h = ((h ^ b) * 1099511628211) & 0xFFFFFFFFFFFFFFFF
    return h


def dump(path):
    if not os.path.exists(build.SAFETENSORS_DUMP):
        pytest.fail(f"{build.SAFETENSORS_DUMP} has not been built (python -m mykuiperllama_amd.build)")
    return subprocess.run([build.SAFETENSORS_DUMP, str(path)], capture_output=True, text=True, timeout=60)


def test_reader_agrees_with_the_safetensors_package(tmp_path):
    import torch
    from safetensors.torch import save_file
    p = synth.make_awq_problem("st_reader", 1, 256, 64, 128)
    tensors = {
        "model.layers.0.mlp.down_proj.qweight": torch.from_numpy(p["qweight"].astype(np.int32)),
        "model.layers.0.mlp.down_proj.qzeros": torch.from_numpy(p["qzeros"].astype(np.int32)),
        "model.layers.0.mlp.down_proj.scales": torch.from_numpy(p["scales"].view(np.float16).copy()),
        "lm_head.weight": torch.randn(16, 32).bfloat16(),
        "norm.weight": torch.randn(7),
        "flags": torch.tensor([True, False, True]),
        "ids": torch.arange(5, dtype=torch.int64),
    }
    path = tmp_path / "model.safetensors"
    save_file(tensors, str(path), metadata={"format": "pt", "quant": "awq gemm, group 128"})
    out = dump(path)
    assert out.returncode == 0, out.stderr
    lines = [l for l in out.stdout.splitlines() if l and not l.startswith("#")]
    meta = {l[2:].split(" = ")[0]: l[2:].split(" = ", 1)[1] for l in out.stdout.splitlines() if l.startswith("# ")}
    assert meta == {"format": "pt", "quant": "awq gemm, group 128"}
    seen = {}
    for l in lines:
        name, dtype, shape, nbytes, digest = l.split(" ")
        seen[name] = (dtype, shape, int(nbytes), int(digest, 16))
    assert set(seen) == set(tensors)
    names = {torch.int32: "I32", torch.float16: "F16", torch.bfloat16: "BF16", torch.float32: "F32",
             torch.bool: "BOOL", torch.int64: "I64"}
    for name, t in tensors.items():
        raw = t.contiguous().view(torch.uint8).numpy().tobytes() if t.dtype != torch.bool \
            else t.numpy().astype(np.uint8).tobytes()
        dtype, shape, nbytes, digest = seen[name]
        assert dtype == names[t.dtype]
        assert shape == "x".join(str(d) for d in t.shape)
        assert nbytes == len(raw)
        assert digest == fnv1a64(raw), name


def test_dump_tool_reports_a_broken_file(tmp_path):
    path = tmp_path / "broken.safetensors"
    path.write_bytes((1 << 40).to_bytes(8, "little") + b"{}")
    out = dump(path)
    assert out.returncode == 1
    assert "header length" in out.stderr
