"""Many split-K launches back to back on ONE workspace, cycling the seven Qwen3-8B projection shapes: every
output must equal, bit for bit, what the same shape returned the first time.

The split-K exchange orders its partial sums before the arrival counter by waiting for the stores'
acknowledgement, not by a release/acquire pair (an acquire-release counter update costs 3 to 27 us per launch
on this machine: it writes back and invalidates whole caches).  That is a contract with the hardware rather
than with the language's memory model, so it is watched: a stale partial sum or a counter left non-zero by
one launch shows up here as a changed bit in a later one.  The run stops at the first mismatch.
"""
import pytest

from mykuiperllama_amd import synth

pytestmark = pytest.mark.gpu

LAUNCHES = 2000
CHUNK = 100  # launches between comparisons


@pytest.mark.parametrize("policy", [0, 2], ids=["by_shape", "mfma"])
def test_two_thousand_launches_on_one_workspace_repeat_their_first_results(policy):
    import torch
    from mykuiperllama_amd import capi
    capi.load()
    assert torch.cuda.is_available()
    names = ["q_proj", "k_proj", "v_proj", "o_proj", "gate_proj", "up_proj", "down_proj"]
    shapes = [synth.QWEN3_8B[n] for n in names]
    gen = torch.Generator(device="cuda")
    gen.manual_seed(synth.BASE_SEED + 5)
    probs = []
    for K, N in shapes:
        qw = torch.randint(-2**31, 2**31 - 1, (K, N // 8), dtype=torch.int32, device="cuda", generator=gen)
        qz = torch.randint(-2**31, 2**31 - 1, (K // 128, N // 8), dtype=torch.int32, device="cuda", generator=gen)
        sc = (torch.rand((K // 128, N), device="cuda", generator=gen) * 0.019 + 0.001).half()
        x = torch.randn((1, K), device="cuda", generator=gen).bfloat16()
        probs.append((x, qw, sc, qz, N))
    ws = capi.make_workspace(1, max(k for k, _ in shapes), max(n for _, n in shapes))  # one workspace for all
    capi.set_awq_kernel_policy(policy)
    try:
        first = []
        for x, qw, sc, qz, N in probs:
            y = torch.empty((1, N), dtype=torch.bfloat16, device="cuda")
            capi.gemv_awq_bf16(x, qw, sc, qz, y, 128, ws)
            first.append(y)
        torch.cuda.synchronize()
        outs = [[torch.empty((1, N), dtype=torch.bfloat16, device="cuda") for _ in range(CHUNK // len(probs) + 1)]
                for (_, _, _, _, N) in probs]
        done = 0
        while done < LAUNCHES:
            used = [0] * len(probs)
            batch = []
            for i in range(done, min(done + CHUNK, LAUNCHES)):
                s = i % len(probs)
                x, qw, sc, qz, _ = probs[s]
                y = outs[s][used[s]]
                used[s] += 1
                capi.gemv_awq_bf16(x, qw, sc, qz, y, 128, ws)  # no synchronisation in between
                batch.append((i, s, y))
            torch.cuda.synchronize()
            for i, s, y in batch:
                assert torch.equal(y.view(torch.int16), first[s].view(torch.int16)), \
                    f"launch {i} ({names[s]}) differs from the first {names[s]} launch"
            done += len(batch)
    finally:
        capi.set_awq_kernel_policy(0)
