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


@pytest.mark.parametrize("policy", [0, 1, 2], ids=["by_shape", "vector_ordered", "mfma"])
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


def test_chained_launches_on_one_workspace_repeat_their_first_results():
    """The same watch over the exchanges of the fused epilogues: the o and down projections with the residual
    output (every wave of 64 columns finishes for itself) and the q|k|v projection with the rotary output (the two
    waves of a head share a counter), 1 400 launches cycling over the three on one workspace together with plain
    launches of the same shapes, which index the counter area differently."""
    import torch
    from mykuiperllama_amd import capi
    capi.load()
    gen = torch.Generator(device="cuda")
    gen.manual_seed(synth.BASE_SEED + 6)
    H, I, n_q, n_kv, max_pos, pos_value = 4096, 12288, 32, 8, 64, 17

    def weights(K, N):
        qw = torch.randint(-2**31, 2**31 - 1, (K, N // 8), dtype=torch.int32, device="cuda", generator=gen)
        qz = torch.randint(-2**31, 2**31 - 1, (K // 128, N // 8), dtype=torch.int32, device="cuda", generator=gen)
        sc = (torch.rand((K // 128, N), device="cuda", generator=gen) * 0.019 + 0.001).half()
        return qw, sc, qz

    def bf16(shape, scale=1.0):
        return (torch.randn(shape, device="cuda", generator=gen) * scale).bfloat16()

    w_o, w_down, w_qkv = weights(H, H), weights(I, H), weights(H, (n_q + 2 * n_kv) * 128)
    x_o, gate, up, x_qkv, resid = bf16((1, H)), bf16((1, I)), bf16((1, I)), bf16((1, H)), bf16((1, H), 2.0)
    q_gain, k_gain = 1 + bf16((128,), 0.1), 1 + bf16((128,), 0.1)
    pos = torch.tensor([pos_value], dtype=torch.int32, device="cuda")
    ws = capi.make_workspace(1, I, (n_q + 2 * n_kv) * 128)

    def run_residual(kind, out, sumsq):
        if kind == "o":
            capi.gemv_awq_chain_bf16({"in_kind": capi.IN_ROW, "x": x_o, "out_kind": capi.OUT_RESIDUAL,
                                      "residual_in": resid, "residual_out": out, "sumsq_out": sumsq},
                                     *w_o, H, H, 128, ws)
        else:
            capi.gemv_awq_chain_bf16({"in_kind": capi.IN_SWIGLU, "gate": gate, "up": up,
                                      "out_kind": capi.OUT_RESIDUAL, "residual_in": resid, "residual_out": out,
                                      "sumsq_out": sumsq}, *w_down, I, H, 128, ws)

    def run_rope(q_out, kc, vc):
        capi.gemv_awq_chain_bf16({"in_kind": capi.IN_ROW, "x": x_qkv, "out_kind": capi.OUT_QKV_ROPE,
                                  "q_gain": q_gain, "k_gain": k_gain, "q_out": q_out, "k_cache": kc, "v_cache": vc,
                                  "pos": pos, "rope_n_q_heads": n_q, "rope_n_kv_heads": n_kv, "rope_theta": 1e6,
                                  "qk_eps": 1e-6}, *w_qkv, H, (n_q + 2 * n_kv) * 128, 128, ws)

    def fresh():
        return {"o": (torch.empty((1, H), dtype=torch.bfloat16, device="cuda"),
                      torch.empty((H // 256, 4), dtype=torch.float32, device="cuda")),
                "down": (torch.empty((1, H), dtype=torch.bfloat16, device="cuda"),
                         torch.empty((H // 256, 4), dtype=torch.float32, device="cuda")),
                "rope": (torch.empty((1, n_q * 128), dtype=torch.bfloat16, device="cuda"),
                         torch.zeros((max_pos, n_kv, 128), dtype=torch.bfloat16, device="cuda"),
                         torch.zeros((max_pos, n_kv, 128), dtype=torch.bfloat16, device="cuda")),
                "plain": (torch.empty((1, H), dtype=torch.bfloat16, device="cuda"),)}

    def launch(kind, bufs):
        if kind in ("o", "down"):
            run_residual(kind, *bufs[kind])
        elif kind == "rope":
            run_rope(*bufs["rope"])
        else:
            capi.gemv_awq_bf16(x_o, *w_o, bufs["plain"][0], 128, ws)

    order = ["o", "rope", "plain", "down"]
    first = fresh()
    for kind in order:
        launch(kind, first)
    torch.cuda.synchronize()
    rounds, per_round = 14, 25   # 14 x 25 x 4 = 1 400 launches
    for r in range(rounds):
        sets = [fresh() for _ in range(per_round)]
        for bufs in sets:
            for kind in order:
                launch(kind, bufs)       # no synchronisation in between
        torch.cuda.synchronize()
        for i, bufs in enumerate(sets):
            for kind in order:
                for got, ref in zip(bufs[kind], first[kind]):
                    same = torch.equal(got.view(torch.int32) if got.dtype == torch.float32 else got.view(torch.int16),
                                       ref.view(torch.int32) if ref.dtype == torch.float32 else ref.view(torch.int16))
                    assert same, f"round {r}, set {i}: a {kind} launch differs from the first one"
