"""The C++ runner (kuiper `model::Qwen3Decoder`, driven through the kx_qwen3_decode tool) against
`decode.DecodeModel`, whose step is itself checked against an fp32 reference and against the
transformers Qwen3 model elsewhere in this suite.

A small checkpoint with Hugging Face's Qwen3 tensor names and separate q/k/v and gate/up
projections is written with the `safetensors` package; the tool reads the sizes off the tensors,
lays the projections side by side, and decodes a token sequence from an empty cache, launch by
launch and again from a captured HIP graph.  Both enqueue the launches that DecodeModel enqueues,
in the same order on the same kernels, so the next token and every bit of the logits must agree
at every position.
"""
import os
import subprocess

import numpy as np
import pytest

from mykuiperllama_amd import build
from tests.test_gpu_decode_step import CFG, make_weights, to_model_weights

TOKENS = [17, 3, 900, 41, 41, 512, 7, 1023, 0, 77]

PROJECTIONS = {"q": "self_attn.q_proj", "k": "self_attn.k_proj", "v": "self_attn.v_proj", "o": "self_attn.o_proj",
               "gate": "mlp.gate_proj", "up": "mlp.up_proj", "down": "mlp.down_proj"}
NORMS = {"in_norm": "input_layernorm.weight", "post_norm": "post_attention_layernorm.weight",
         "q_norm": "self_attn.q_norm.weight", "k_norm": "self_attn.k_norm.weight"}


def fnv1a64(data: bytes) -> int:
    h = 1469598103934665603
    for b in data:
        h = ((h ^ b) * 1099511628211) & 0xFFFFFFFFFFFFFFFF
    return h


def write_checkpoint(path, torch, layers_np, embed, lm_head, final_norm):
    from safetensors.torch import save_file
    tensors = {"model.embed_tokens.weight": embed.contiguous(), "model.norm.weight": final_norm.contiguous()}
    if lm_head is not None:
        tensors["lm_head.weight"] = lm_head.contiguous()
    for li, (packed, norms) in enumerate(layers_np):
        prefix = f"model.layers.{li}."
        for short, name in PROJECTIONS.items():
            p = packed[short]
            tensors[prefix + name + ".qweight"] = torch.from_numpy(np.ascontiguousarray(p["qweight"], np.int32))
            tensors[prefix + name + ".qzeros"] = torch.from_numpy(np.ascontiguousarray(p["qzeros"], np.int32))
            tensors[prefix + name + ".scales"] = torch.from_numpy(p["scales"].view(np.float16).copy())
        for short, name in NORMS.items():
            tensors[prefix + name] = norms[short].contiguous()
    save_file(tensors, str(path), metadata={"rope_theta": "1000000.0", "rms_norm_eps": "1e-06", "group_size": "128"})


def run_tool(args):
    if not os.path.exists(build.QWEN3_DECODE):
        pytest.fail(f"{build.QWEN3_DECODE} has not been built (python -m mykuiperllama_amd.build)")
    return subprocess.run([build.QWEN3_DECODE] + [str(a) for a in args], capture_output=True, text=True, timeout=110)


def parse(stdout):
    rows = []
    for line in stdout.strip().splitlines():
        pos, token, nxt, digest = line.split()
        rows.append((int(pos), int(token), int(nxt), int(digest, 16)))
    return rows


@pytest.mark.gpu
@pytest.mark.parametrize("max_positions", [48, 6000])
def test_cpp_decoder_built_from_layers_matches_the_unfused_python_step(tmp_path, oracle, max_positions):
    """--operators: one kuiper layer forward() per operator; DecodeModel.step(fused=False) enqueues the same
    ten launches per decoder layer through the C ABI."""
    import torch
    from mykuiperllama_amd import decode
    cfg = decode.ModelConfig(**CFG)
    layers_np, _, embed, lm_head, final_norm = make_weights(torch, oracle, cfg)
    path = tmp_path / "model.safetensors"
    write_checkpoint(path, torch, layers_np, embed, lm_head, final_norm)
    model = decode.DecodeModel(cfg, max_positions, weights=to_model_weights(torch, layers_np, embed, lm_head, final_norm))
    expected = []
    for pos, token in enumerate(TOKENS):
        model.set_input(token, pos)
        model.step(fused=False)
        torch.cuda.synchronize()
        logits = model.logits.view(torch.int16).cpu().numpy().tobytes()
        expected.append((pos, token, int(model.next_token.item()), fnv1a64(logits)))
    for mode in (["--operators"], ["--operators", "--graph"]):
        done = run_tool(mode + ["--max-positions", max_positions, path] + TOKENS)
        assert done.returncode == 0, done.stderr
        launches = model.launches_per_step(with_lm_head=True, fused=False)
        assert f"{launches} launches per step" in done.stderr
        assert parse(done.stdout) == expected, (mode, done.stderr)


@pytest.mark.gpu
@pytest.mark.parametrize("max_positions,tied", [(48, False), (6000, False), (10368, False), (48, True)])
def test_cpp_decoder_matches_the_python_driver_bit_for_bit(tmp_path, oracle, max_positions, tied):
    import torch
    from mykuiperllama_amd import decode
    cfg = decode.ModelConfig(**CFG)
    layers_np, _, embed, lm_head, final_norm = make_weights(torch, oracle, cfg)
    if tied:
        lm_head = embed
    path = tmp_path / "model.safetensors"
    write_checkpoint(path, torch, layers_np, embed, None if tied else lm_head, final_norm)

    model = decode.DecodeModel(cfg, max_positions, weights=to_model_weights(torch, layers_np, embed, lm_head, final_norm))
    expected = []
    for pos, token in enumerate(TOKENS):
        model.set_input(token, pos)
        model.step(fused=True)
        torch.cuda.synchronize()
        logits = model.logits.view(torch.int16).cpu().numpy().tobytes()
        expected.append((pos, token, int(model.next_token.item()), fnv1a64(logits)))

    for mode in ([], ["--graph"]):
        done = run_tool(mode + ["--max-positions", max_positions, path] + TOKENS)
        assert done.returncode == 0, done.stderr
        assert f"layers {cfg.layers} hidden {cfg.hidden} intermediate {cfg.intermediate} q heads {cfg.n_q} " \
               f"kv heads {cfg.n_kv} vocab {cfg.vocab} group 128" in done.stderr
        launches = model.launches_per_step(with_lm_head=True, fused=True)
        assert f"{launches} launches per step" in done.stderr
        assert parse(done.stdout) == expected, (mode, done.stderr)
    # --layers: the same launches, each the forward() of a kuiper layer (the projections in their fused form); the
    # first layer's row is normed by a launch of its own, which changes no bit
    for mode in (["--layers"], ["--layers", "--graph"]):
        done = run_tool(mode + ["--max-positions", max_positions, path] + TOKENS)
        assert done.returncode == 0, done.stderr
        assert f"{launches + 1} launches per step" in done.stderr
        assert parse(done.stdout) == expected, (mode, done.stderr)


def test_tool_reports_a_missing_file_and_a_file_without_a_model(tmp_path):
    import torch
    from safetensors.torch import save_file
    done = run_tool([tmp_path / "absent.safetensors", 1])
    assert done.returncode == 1 and done.stderr.strip()
    path = tmp_path / "other.safetensors"
    save_file({"weight": torch.zeros(4, 4)}, str(path))
    done = run_tool([path, 1])
    assert done.returncode == 1
    assert "model.embed_tokens.weight" in done.stderr
    done = run_tool([])
    assert done.returncode == 2 and "usage" in done.stderr


@pytest.mark.gpu
@pytest.mark.parametrize("mode", [[], ["--graph"]])
def test_tool_times_a_random_init_model(mode):
    import json
    done = run_tool(mode + ["--random", "tiny", "--context", 300, "--steps", 20, "--warmup", 5])
    assert done.returncode == 0, done.stderr
    line = json.loads(done.stdout)
    assert line["model"] == "tiny" and line["context"] == 300 and line["steps"] == 20
    assert line["graph"] is bool(mode)
    assert line["launches_per_step"] == 1 + 2 * 5 + 3
    assert 0.0 < line["ms_per_step"] < 50.0
    assert abs(line["tokens_per_s"] * line["ms_per_step"] - 1000.0) < 1.0


def test_tool_rejects_an_unknown_architecture_and_a_missing_context():
    done = run_tool(["--random", "qwen9-1t", "--context", 10])
    assert done.returncode == 2 and "unknown architecture" in done.stderr
    done = run_tool(["--random", "tiny"])
    assert done.returncode == 2 and "--context" in done.stderr


@pytest.mark.gpu
def test_greedy_continuation_follows_the_python_driver(tmp_path, oracle):
    import torch
    from mykuiperllama_amd import decode
    cfg = decode.ModelConfig(**CFG)
    layers_np, _, embed, lm_head, final_norm = make_weights(torch, oracle, cfg)
    path = tmp_path / "model.safetensors"
    write_checkpoint(path, torch, layers_np, embed, lm_head, final_norm)
    prompt, more = [17, 3, 900], 9
    model = decode.DecodeModel(cfg, len(prompt) + more, weights=to_model_weights(torch, layers_np, embed, lm_head, final_norm))
    fed, expected = list(prompt), []
    for pos in range(len(prompt) + more):
        model.set_input(fed[pos], pos)
        model.step(fused=True)
        torch.cuda.synchronize()
        nxt = int(model.next_token.item())
        expected.append((pos, fed[pos], nxt, fnv1a64(model.logits.view(torch.int16).cpu().numpy().tobytes())))
        if pos + 1 == len(fed):
            fed.append(nxt)
    done = run_tool(["--graph", "--generate", more, path] + prompt)
    assert done.returncode == 0, done.stderr
    assert parse(done.stdout) == expected
    done = run_tool(["--max-positions", 5, "--generate", more, path] + prompt)
    assert done.returncode == 2 and "--max-positions" in done.stderr
