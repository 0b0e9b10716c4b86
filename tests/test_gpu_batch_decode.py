"""Several sequences decoded together (2 <= B <= 16): the batched rotation, attention, embedding and argmax
entry points against the one-sequence calls, bit for bit (the attention from four sequences on, where it
chunks a short cache differently, to rounding), and the batched decode step against B one-sequence
models stepped on their own (the GEMVs of a batch run on the matrix-core kernel, those of one sequence on the
vector kernel: equal to the rounding of fp32 sums in a different order, relative L2 <= 1e-2 on the logits of a
two-layer model)."""
import math

import pytest

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


def bf16_rand(torch, shape, seed, scale=1.0):
    g = torch.Generator(device="cuda")
    g.manual_seed(seed)
    return (torch.randn(shape, device="cuda", generator=g) * scale).bfloat16()


def bits(t, torch):
    return t.contiguous().view(torch.int16)


@pytest.mark.parametrize("B,n_q,n_kv,max_pos", [(2, 4, 2, 192), (5, 32, 8, 4224), (16, 64, 8, 8320)])
def test_batched_rotation_and_attention_equal_the_one_sequence_calls(capi, torch, B, n_q, n_kv, max_pos):
    heads = n_q + 2 * n_kv
    qkv = bf16_rand(torch, (B, heads * 128), 1)
    q_gain = bf16_rand(torch, (128,), 2, 0.1) + 1.0
    k_gain = bf16_rand(torch, (128,), 3, 0.1) + 1.0
    # every sequence at its own position; the first and last rows of a cache are among them
    positions = [(37 * b * b + 11 * b) % max_pos for b in range(B)]
    positions[0] = 0
    positions[-1] = max_pos - 1
    pos = torch.tensor(positions, dtype=torch.int32, device="cuda")
    kc = bf16_rand(torch, (B, max_pos, n_kv, 128), 4)
    vc = bf16_rand(torch, (B, max_pos, n_kv, 128), 5)
    kc1, vc1 = kc.clone(), vc.clone()

    q = torch.full((B, n_q * 128), float("nan"), dtype=torch.bfloat16, device="cuda")
    capi.qk_norm_rope_batch_bf16(qkv, q_gain, k_gain, q, kc, vc, n_q, n_kv, pos, 1e6, 1e-6)
    out = torch.full((B, n_q * 128), float("nan"), dtype=torch.bfloat16, device="cuda")
    ws = capi.attn_decode_batch_workspace(B, n_q, max_pos)
    capi.attn_decode_batch_bf16(q, kc, vc, out, n_q, n_kv, pos, max_pos, ws)
    torch.cuda.synchronize()

    ws1 = capi.attn_decode_workspace(n_q, max_pos)
    for b in range(B):
        qb = torch.empty((1, n_q * 128), dtype=torch.bfloat16, device="cuda")
        capi.qk_norm_rope_bf16(qkv[b:b + 1], q_gain, k_gain, qb, kc1[b], vc1[b], n_q, n_kv, pos[b:b + 1], 1e6, 1e-6)
        ob = torch.empty((1, n_q * 128), dtype=torch.bfloat16, device="cuda")
        capi.attn_decode_bf16(qb, kc1[b], vc1[b], ob, n_q, n_kv, pos[b:b + 1], max_pos, ws1)
        torch.cuda.synchronize()
        assert torch.equal(bits(q[b], torch), bits(qb[0], torch)), f"q of sequence {b}"
        if B < 4 or max_pos > 5120:
            assert torch.equal(bits(out[b], torch), bits(ob[0], torch)), f"attention of sequence {b}"
        else:
            # from four sequences on the batched call splits a short cache into chunks of 128 positions, the
            # one-sequence call into chunks of 64: the same sums in another order
            got, ref = out[b].float(), ob[0].float()
            assert ((got - ref).norm() / ref.norm()).item() <= 3e-3, f"attention of sequence {b}"
            assert (got - ref).abs().max().item() <= 2 * 2.0 ** (math.floor(math.log2(ref.abs().max().item())) - 7)
    assert torch.equal(bits(kc, torch), bits(kc1, torch))
    assert torch.equal(bits(vc, torch), bits(vc1, torch))


def test_batched_embedding_and_argmax(capi, torch):
    vocab, dim, B = 1000, 512, 7
    table = bf16_rand(torch, (vocab, dim), 6)
    tokens = torch.tensor([0, 999, 5, 5, -3, 4000, 17], dtype=torch.int32, device="cuda")  # two of them clamped
    out = torch.empty((B, dim), dtype=torch.bfloat16, device="cuda")
    capi.embedding_rows_bf16(table, tokens, out)
    expect = table[tokens.clamp(0, vocab - 1).long()]
    assert torch.equal(bits(out, torch), bits(expect, torch))

    for n in (151936, 1000, 13):
        x = bf16_rand(torch, (B, n + 24), 7 + n)[:, :n]   # rows further apart than they are long
        x[2, n // 2] = 100.0
        x[3, :] = 1.0                                      # ties: the first index
        x[4, 0] = float("nan")
        idx = torch.full((B,), -1, dtype=torch.int32, device="cuda")
        capi.argmax_rows_bf16(x, idx)
        torch.cuda.synchronize()
        for b in range(B):
            one = torch.full((1,), -1, dtype=torch.int32, device="cuda")
            capi.argmax_bf16(x[b].contiguous(), one)
            assert int(idx[b]) == int(one[0]), f"row {b} of {n}"
        assert int(idx[2]) == n // 2 and int(idx[3]) == 0


def test_batch_entry_points_reject_bad_arguments(capi, torch):
    B, n_q, n_kv, max_pos = 3, 4, 2, 128
    qkv = bf16_rand(torch, (B, 8 * 128), 1)
    gain = bf16_rand(torch, (128,), 2)
    q = torch.empty((B, n_q * 128), dtype=torch.bfloat16, device="cuda")
    cache = bf16_rand(torch, (B, max_pos, n_kv, 128), 3)
    pos = torch.zeros(B, dtype=torch.int32, device="cuda")
    lib = capi.load()
    p = lambda t: t.data_ptr()
    stride = cache.stride(0)
    rope = lambda batch, cs: lib.kx_qk_norm_rope_batch_bf16(p(qkv), p(gain), p(gain), p(q), p(cache), p(cache), cs, n_q,
                                                            n_kv, 128, p(pos), max_pos, 1e6, 1e-6, batch, None)
    assert rope(0, stride) == -2 and rope(17, stride) == -2
    assert rope(B, stride - 128) == -2          # caches that would overlap
    ws = capi.attn_decode_batch_workspace(B, n_q, max_pos)
    attn = lambda batch, cs, nbytes: lib.kx_attn_decode_batch_bf16(p(q), p(cache), p(cache), cs, p(q), n_q, n_kv, 128,
                                                                    p(pos), max_pos, p(ws), nbytes, batch, None)
    assert attn(B, stride, ws.numel() // B) == -3   # a workspace for one sequence
    assert attn(B, stride + 4, ws.numel()) == -2    # a cache that would not be 16-byte aligned
    assert attn(17, stride, ws.numel()) == -2
    assert lib.kx_argmax_rows_bf16(p(q), 100, 50, p(pos), 2, None) == -2   # rows that overlap


@pytest.mark.parametrize("B", [2, 5, 16])
def test_batched_step_matches_one_sequence_models(capi, torch, B):
    from mykuiperllama_amd import decode
    cfg = decode.ModelConfig(layers=2, hidden=1024, intermediate=3072, n_q=8, n_kv=2, vocab=2048)
    max_pos = 320
    single = decode.DecodeModel(cfg, max_pos)
    batch = decode.BatchDecodeModel(single, B, rope_in_qkv=(B != 16))  # both forms of the q|k|v launch
    lengths = [17 + 13 * b for b in range(B)]
    batch.prefill_cache_random(lengths)
    tokens = [(101 * b + 7) % cfg.vocab for b in range(B)]

    # two steps for all sequences, fused and unfused, from the same caches
    saved = [(k.clone(), v.clone()) for k, v in zip(batch.k_cache, batch.v_cache)]
    results = {}
    for mode in (True, False):
        for (k, v), (k0, v0) in zip(zip(batch.k_cache, batch.v_cache), saved):
            k.copy_(k0)
            v.copy_(v0)
        toks, outs = list(tokens), []
        for stepno in range(2):
            batch.set_input(toks, [n + stepno for n in lengths])
            batch.step(fused=mode)
            torch.cuda.synchronize()
            outs.append(batch.logits.clone())
            toks = [int(t) for t in batch.next_token.tolist()]
        results[mode] = outs
    for a, b_ in zip(results[True], results[False]):
        assert torch.isfinite(a.float()).all()
        err = ((a.float() - b_.float()).norm() / b_.float().norm()).item()
        assert err <= 5e-3, f"fused against unfused: {err}"

    # each sequence alone on the one-sequence model (vector kernels), first step
    for b in range(B):
        for li in range(cfg.layers):
            single.k_cache[li].copy_(saved[li][0][b])
            single.v_cache[li].copy_(saved[li][1][b])
        single.set_input(tokens[b], lengths[b])
        single.step(fused=False)
        torch.cuda.synchronize()
        ref = single.logits[0].float()
        got = results[False][0][b].float()
        err = ((got - ref).norm() / ref.norm()).item()
        assert err <= 1e-2, f"sequence {b}: {err}"

    # a captured step replays to the same bits
    batch.set_input(tokens, lengths)
    batch.step()
    torch.cuda.synchronize()
    eager = batch.logits.clone()
    side = torch.cuda.Stream()
    with torch.cuda.stream(side):
        g = torch.cuda.CUDAGraph()
        with torch.cuda.graph(g):
            batch.step()
        for _ in range(2):
            batch.logits.zero_()
            torch.cuda.synchronize()
            g.replay()
            side.synchronize()
            assert torch.equal(bits(batch.logits, torch), bits(eager, torch))
    torch.cuda.synchronize()
