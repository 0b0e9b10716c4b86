"""GPU parity of the GEMV with an activation prologue and / or the residual epilogue at several activation
rows (2 <= M <= 16), the matrix-core kernel's versions of what the decode step uses at M = 1.

Bitwise wherever the arithmetic is that of stand-alone kernels run back to back on the same kernel family
(SwiGLU in, residual add out); the RMSNorm input works from per-tile sums of squares, an order of its own,
and is compared with the fp32 restatement (relative L2 <= 2e-3) and with the one-row launch on the vector
kernel, row by row.
"""
import pytest

from mykuiperllama_amd import synth
from tests import helpers as H

pytestmark = pytest.mark.gpu

EPS = 1e-6


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


def weights(torch, name, K, N, group):
    p = synth.make_awq_problem(name, 1, K, N, group)
    return H.to_dev_i32(p["qweight"], torch), H.to_dev_f16(p["scales"], torch), H.to_dev_i32(p["qzeros"], torch)


def bf16_rand(torch, shape, seed, scale=1.0):
    g = torch.Generator(device="cuda")
    g.manual_seed(seed)
    return (torch.randn(shape, device="cuda", generator=g) * scale).bfloat16()


def bits(t, torch):
    return t.contiguous().view(torch.int16)


def rel_l2(a, b):
    a, b = a.double(), b.double()
    return float((a - b).norm() / b.norm())


def tile_sums(torch, rows):
    """fp64 sums of squares of every row of a bf16 [M, N] tensor per quarter (64 columns) of every tile of 256
    columns -> [M, ceil(N / 256), 4]."""
    v = rows.double()
    pad = (-v.shape[1]) % 256
    v = torch.cat([v, torch.zeros((v.shape[0], pad), dtype=torch.float64, device=v.device)], dim=1)
    return (v * v).view(v.shape[0], -1, 4, 64).sum(dim=3)


# K, N, group: the Qwen3-8B down projection, a 32B-shaped one, a narrow one with a ragged last tile, groups of
# 32 and 64 (one and two steps per wave)
SHAPES = [(12288, 4096, 128), (4096, 4096, 128), (25600, 5120, 128), (512, 272, 32), (1024, 512, 64)]
ROWS = [2, 3, 4, 8, 13, 16]


@pytest.mark.parametrize("K,N,group", SHAPES)
@pytest.mark.parametrize("M", ROWS)
def test_swiglu_input_equals_swiglu_then_gemv(capi, torch, K, N, group, M):
    qw, sc, qz = weights(torch, f"sb_swiglu_{K}_{N}", K, N, group)
    ws = capi.make_workspace(M, K, N)
    # gate and up as the two halves of one [M, 2K] tensor (the layout a fused gate|up projection leaves)
    gu = bf16_rand(torch, (M, 2 * K), 11 * M + K, 1.5)
    gate, up = gu[:, :K], gu[:, K:]
    act = torch.empty((M, K), dtype=torch.bfloat16, device="cuda")
    capi.swiglu_bf16(gate.contiguous(), up.contiguous(), act)
    expected = torch.empty((M, N), dtype=torch.bfloat16, device="cuda")
    capi.gemv_awq_bf16(act, qw, sc, qz, expected, group, ws)
    y = torch.full((M, N), float("nan"), dtype=torch.bfloat16, device="cuda")
    capi.gemv_awq_swiglu_bf16(gate, up, qw, sc, qz, y, group, ws)
    torch.cuda.synchronize()
    assert torch.equal(bits(y, torch), bits(expected, torch))


@pytest.mark.parametrize("K,N,group", SHAPES)
@pytest.mark.parametrize("M", ROWS)
@pytest.mark.parametrize("in_kind", ["row", "swiglu"])
def test_residual_output_equals_gemv_then_add(capi, torch, K, N, group, M, in_kind):
    qw, sc, qz = weights(torch, f"sb_res_{K}_{N}", K, N, group)
    ws = capi.make_workspace(M, K, N)
    resid = bf16_rand(torch, (M, N), N + M, 2.0)
    y = torch.empty((M, N), dtype=torch.bfloat16, device="cuda")
    desc = {"out_kind": capi.OUT_RESIDUAL, "rows": M}
    if in_kind == "row":
        x = bf16_rand(torch, (M, K), K + N + M)
        capi.gemv_awq_bf16(x, qw, sc, qz, y, group, ws)
        desc.update({"in_kind": capi.IN_ROW, "x": x})
    else:
        gu = bf16_rand(torch, (M, 2 * K), 5 * M + N, 1.5)
        capi.gemv_awq_swiglu_bf16(gu[:, :K], gu[:, K:], qw, sc, qz, y, group, ws)
        desc.update({"in_kind": capi.IN_SWIGLU, "gate": gu[:, :K], "up": gu[:, K:], "act_ld": 2 * K})
    expected = torch.empty_like(resid)
    capi.add_bf16(resid, y, expected)

    parts = (N + 255) // 256
    sumsq = torch.full((M, parts, 4), float("nan"), dtype=torch.float32, device="cuda")
    for in_place in (False, True):
        out = resid.clone() if in_place else torch.full((M, N), float("nan"), dtype=torch.bfloat16, device="cuda")
        desc.update({"residual_in": out if in_place else resid, "residual_out": out, "sumsq_out": sumsq})
        capi.gemv_awq_chain_bf16(desc, qw, sc, qz, K, N, group, ws)
        torch.cuda.synchronize()
        assert torch.equal(bits(out, torch), bits(expected, torch)), f"in_place={in_place}"
        ref = tile_sums(torch, expected)
        live = torch.arange(parts * 4, device="cuda").view(1, parts, 4).expand_as(ref) * 64 < N  # quarters with columns
        assert torch.allclose(sumsq.double()[live], ref[live], rtol=1e-5, atol=0)


@pytest.mark.parametrize("K,N,group", [(4096, 24576, 128), (5120, 10240, 128), (512, 272, 32), (1024, 512, 64)])
@pytest.mark.parametrize("M", ROWS)
def test_norm_input_matches_the_fp32_restatement_and_the_one_row_launch(capi, torch, oracle, K, N, group, M):
    p = synth.make_awq_problem(f"sb_norm_{K}_{N}", 1, K, N, group)
    qw, sc, qz = H.to_dev_i32(p["qweight"], torch), H.to_dev_f16(p["scales"], torch), H.to_dev_i32(p["qzeros"], torch)
    ws = capi.make_workspace(M, K, N)
    ws1 = capi.make_workspace(1, K, N)
    row = bf16_rand(torch, (M, K), 3 * K + M, 1.7)
    gain = bf16_rand(torch, (K,), K + 1, 0.5) + 1.0
    parts = (K + 255) // 256
    sumsq = tile_sums(torch, row).float().contiguous()
    assert sumsq.shape == (M, parts, 4)

    y = torch.full((M, N), float("nan"), dtype=torch.bfloat16, device="cuda")
    desc = {"in_kind": capi.IN_NORM, "norm_row": row, "norm_sumsq": sumsq, "norm_parts": parts, "norm_gain": gain,
            "norm_eps": EPS, "out_kind": capi.OUT_ROW, "y": y, "rows": M}
    capi.gemv_awq_chain_bf16(desc, qw, sc, qz, K, N, group, ws)
    torch.cuda.synchronize()
    again = torch.empty_like(y)
    capi.gemv_awq_chain_bf16(dict(desc, y=again), qw, sc, qz, K, N, group, ws)
    torch.cuda.synchronize()
    assert torch.equal(bits(y, torch), bits(again, torch))

    # the restatement: normalised row (bf16 rounding points as in the kernels), then the CPU oracle's GEMV
    inv = torch.rsqrt(sumsq.double().sum(dim=(1, 2)).view(-1, 1) / K + EPS).float()
    h = (gain.float() * (row.float() * inv).bfloat16().float()).bfloat16()
    ref = oracle.gemv_awq_f64(H.bf16_bits(h, torch), p["qweight"], p["scales"], p["qzeros"], group)
    assert rel_l2(y.float().cpu(), torch.from_numpy(ref)) <= 2e-3

    # row by row, the one-row launch on the vector kernel
    for m in range(M):
        y1 = torch.empty((1, N), dtype=torch.bfloat16, device="cuda")
        capi.gemv_awq_chain_bf16({"in_kind": capi.IN_NORM, "norm_row": row[m:m + 1], "norm_sumsq": sumsq[m],
                                  "norm_parts": parts, "norm_gain": gain, "norm_eps": EPS,
                                  "out_kind": capi.OUT_ROW, "y": y1}, qw, sc, qz, K, N, group, ws1)
        torch.cuda.synchronize()
        assert rel_l2(y[m].float(), y1[0].float()) <= 2e-3, f"row {m}"


@pytest.mark.parametrize("M", [2, 8, 16])
def test_mlp_block_in_two_launches_matches_five(capi, torch, M):
    """RMSNorm -> gate|up -> SwiGLU -> down -> residual add of a Qwen3-8B layer at M rows: two chained launches
    against the five stand-alone ones (equal up to the rounding of the norm's sum of squares)."""
    hidden, inter, group = 4096, 12288, 128
    gu_w = weights(torch, "sb_mlp_gateup", hidden, 2 * inter, group)
    dn_w = weights(torch, "sb_mlp_down", inter, hidden, group)
    ws = capi.make_workspace(M, hidden, 2 * inter)
    ws2 = capi.make_workspace(M, inter, hidden)
    resid = bf16_rand(torch, (M, hidden), 77 + M, 1.3)
    gain = bf16_rand(torch, (hidden,), 5, 0.5) + 1.0

    # five launches
    h = torch.empty_like(resid)
    capi.rmsnorm_bf16(resid, gain, h, EPS)
    gu = torch.empty((M, 2 * inter), dtype=torch.bfloat16, device="cuda")
    capi.gemv_awq_bf16(h, *gu_w, gu, group, ws)
    act = torch.empty((M, inter), dtype=torch.bfloat16, device="cuda")
    capi.swiglu_bf16(gu[:, :inter].contiguous(), gu[:, inter:].contiguous(), act)
    dn = torch.empty((M, hidden), dtype=torch.bfloat16, device="cuda")
    capi.gemv_awq_bf16(act, *dn_w, dn, group, ws2)
    expected = torch.empty_like(resid)
    capi.add_bf16(resid, dn, expected)

    # two launches
    parts = hidden // 256
    sumsq = tile_sums(torch, resid).float().contiguous()
    gu2 = torch.empty_like(gu)
    capi.gemv_awq_chain_bf16({"in_kind": capi.IN_NORM, "norm_row": resid, "norm_sumsq": sumsq, "norm_parts": parts,
                              "norm_gain": gain, "norm_eps": EPS, "out_kind": capi.OUT_ROW, "y": gu2, "rows": M},
                             *gu_w, hidden, 2 * inter, group, ws)
    out = torch.empty_like(resid)
    sumsq_out = torch.empty((M, parts, 4), dtype=torch.float32, device="cuda")
    capi.gemv_awq_chain_bf16({"in_kind": capi.IN_SWIGLU, "gate": gu2[:, :inter], "up": gu2[:, inter:],
                              "act_ld": 2 * inter, "out_kind": capi.OUT_RESIDUAL, "residual_in": resid,
                              "residual_out": out, "sumsq_out": sumsq_out, "rows": M},
                             *dn_w, inter, hidden, group, ws2)
    torch.cuda.synchronize()
    assert torch.isfinite(out.float()).all()
    assert rel_l2(gu2.float(), gu.float()) <= 2e-3
    assert rel_l2(out.float(), expected.float()) <= 2e-3
    assert torch.allclose(sumsq_out.double(), tile_sums(torch, out), rtol=1e-5, atol=0)


@pytest.mark.parametrize("K,n_q,n_kv,group", [(4096, 32, 8, 128), (5120, 64, 8, 128), (512, 4, 2, 32)])
@pytest.mark.parametrize("M", ROWS)
def test_rotary_output_equals_gemv_then_batched_rotation(capi, torch, K, n_q, n_kv, group, M):
    """q|k|v projection of M sequences with per-head norm, rotation and cache append on the way out: bit for
    bit the plain GEMV followed by kx_qk_norm_rope_batch_bf16 (row input), every sequence at its own position."""
    heads = n_q + 2 * n_kv
    N = heads * 128
    max_pos = 96
    qw, sc, qz = weights(torch, f"sb_rope_{K}_{N}", K, N, group)
    ws = capi.make_workspace(M, K, N)
    x = bf16_rand(torch, (M, K), 7 * M + K)
    q_gain = bf16_rand(torch, (128,), 2, 0.1) + 1.0
    k_gain = bf16_rand(torch, (128,), 3, 0.1) + 1.0
    positions = [(29 * m + 5) % max_pos for m in range(M)]
    positions[0], positions[-1] = 0, max_pos - 1
    pos = torch.tensor(positions, dtype=torch.int32, device="cuda")
    kc = bf16_rand(torch, (M, max_pos, n_kv, 128), 4)
    vc = bf16_rand(torch, (M, max_pos, n_kv, 128), 5)
    kc1, vc1 = kc.clone(), vc.clone()

    qkv = torch.empty((M, N), dtype=torch.bfloat16, device="cuda")
    capi.gemv_awq_bf16(x, qw, sc, qz, qkv, group, ws)
    q_sep = torch.empty((M, n_q * 128), dtype=torch.bfloat16, device="cuda")
    capi.qk_norm_rope_batch_bf16(qkv, q_gain, k_gain, q_sep, kc1, vc1, n_q, n_kv, pos, 1e6, 1e-6)

    q = torch.full((M, n_q * 128), float("nan"), dtype=torch.bfloat16, device="cuda")
    capi.gemv_awq_chain_bf16({"in_kind": capi.IN_ROW, "x": x, "out_kind": capi.OUT_QKV_ROPE, "q_gain": q_gain,
                              "k_gain": k_gain, "q_out": q, "k_cache": kc, "v_cache": vc, "pos": pos,
                              "rope_n_q_heads": n_q, "rope_n_kv_heads": n_kv, "rope_theta": 1e6, "qk_eps": 1e-6,
                              "cache_positions": max_pos, "cache_stride": kc.stride(0), "rows": M},
                             qw, sc, qz, K, N, group, ws)
    torch.cuda.synchronize()
    assert torch.equal(bits(q, torch), bits(q_sep, torch))
    assert torch.equal(bits(kc, torch), bits(kc1, torch))
    assert torch.equal(bits(vc, torch), bits(vc1, torch))
    # caches closer together than they are long are refused
    with pytest.raises(capi.KxError) as e:
        capi.gemv_awq_chain_bf16({"in_kind": capi.IN_ROW, "x": x, "out_kind": capi.OUT_QKV_ROPE, "q_gain": q_gain,
                                  "k_gain": k_gain, "q_out": q, "k_cache": kc, "v_cache": vc, "pos": pos,
                                  "rope_n_q_heads": n_q, "rope_n_kv_heads": n_kv, "rope_theta": 1e6, "qk_eps": 1e-6,
                                  "cache_positions": max_pos, "cache_stride": kc.stride(0) - 128, "rows": M},
                                 qw, sc, qz, K, N, group, ws)
    assert e.value.code == -2


def test_what_several_rows_refuse(capi, torch):
    K, N, group, M = 512, 256, 128, 4
    qw, sc, qz = weights(torch, "sb_refuse", K, N, group)
    ws = capi.make_workspace(M, K, N)
    x = bf16_rand(torch, (M, K), 1)
    y = torch.empty((M, N), dtype=torch.bfloat16, device="cuda")

    def code(desc, n=N, g=group, w=None):
        with pytest.raises(capi.KxError) as e:
            capi.gemv_awq_chain_bf16(desc, qw, sc, qz, K, n, g, ws if w is None else w)
        return e.value.code

    base = {"in_kind": capi.IN_ROW, "x": x, "out_kind": capi.OUT_ROW, "y": y}
    assert code(dict(base, rows=17)) == -2
    # the attention merge and the rotary output serve one row
    attn_ws = capi.attn_decode_workspace(4, 128)
    assert code({"in_kind": capi.IN_ATTN, "attn_workspace": attn_ws, "attn_workspace_bytes": attn_ws.numel() * 4,
                 "n_q_heads": 4, "n_kv_heads": 2, "max_positions": 128, "out_kind": capi.OUT_ROW, "y": y,
                 "rows": M}) == -2
    # gate / up that cannot be read 16 bytes at a time
    gu = bf16_rand(torch, (M, 2 * K + 8), 2)
    flat = gu.view(-1)
    shifted_gate = flat[1:1 + M * K].view(M, K)
    assert code({"in_kind": capi.IN_SWIGLU, "gate": shifted_gate, "up": gu[:, :K], "out_kind": capi.OUT_ROW, "y": y,
                 "rows": M}) == -4
    assert code({"in_kind": capi.IN_SWIGLU, "gate": gu[:, :K], "up": gu[:, K:2 * K], "act_ld": 2 * K + 4,
                 "out_kind": capi.OUT_ROW, "y": y, "rows": M}) == -2
    assert code({"in_kind": capi.IN_SWIGLU, "gate": gu[:, :K], "up": gu[:, K:2 * K], "act_ld": K - 8,
                 "out_kind": capi.OUT_ROW, "y": y, "rows": M}) == -2
    # a workspace sized for one row
    small = capi.make_workspace(1, K, N)
    if small.numel() < ws.numel():
        assert code(dict(base, rows=M), w=small) == -3
    # the plain combination still works and equals the plain entry point
    expected = torch.empty_like(y)
    capi.gemv_awq_bf16(x, qw, sc, qz, expected, group, ws)
    capi.gemv_awq_chain_bf16(dict(base, rows=M), qw, sc, qz, K, N, group, ws)
    torch.cuda.synchronize()
    assert torch.equal(bits(y, torch), bits(expected, torch))
