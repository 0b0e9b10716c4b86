"""GPU parity of the chained GEMV entry point (kx_gemv_awq_chain_bf16): every input kind and every
output kind against the stand-alone kernels run back to back.

Bitwise wherever the arithmetic is the same (residual add, SwiGLU and attention-merge inputs, rotary
output); the RMSNorm input works from per-tile sums of squares, an order of its own, so its results
are compared within the GEMV's tolerance (relative L2 <= 1e-3) and a few bf16 ulp on O(1) outputs.
"""
import numpy as np
import pytest

from mykuiperllama_amd import synth
from tests import helpers as H

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


@pytest.fixture(autouse=True)
def vector_kernel_for_the_unfused_side(capi):
    capi.set_awq_kernel_policy(1)
    yield
    capi.set_awq_kernel_policy(0)


def weights(torch, name, K, N, group):
    p = synth.make_awq_problem(name, 1, K, N, group)
    return H.to_dev_i32(p["qweight"], torch), H.to_dev_f16(p["scales"], torch), H.to_dev_i32(p["qzeros"], torch)


def bf16_rand(torch, shape, seed, scale=1.0):
    g = torch.Generator(device="cuda")
    g.manual_seed(seed)
    return (torch.randn(shape, device="cuda", generator=g) * scale).bfloat16()


def tile_sums(torch, row):
    """fp64 sums of squares of a bf16 row per quarter (64 columns) of every tile of 256 columns: [tiles, 4]."""
    v = row.double().flatten()
    n = v.numel()
    pad = (-n) % 256
    v = torch.cat([v, torch.zeros(pad, dtype=torch.float64, device=v.device)])
    return (v * v).view(-1, 4, 64).sum(dim=2)


def rel_l2(a, b):
    a, b = a.double(), b.double()
    return float((a - b).norm() / b.norm())


RESIDUAL_CASES = [(4096, 4096, 128), (12288, 4096, 128), (8192, 5120, 128), (256, 520, 32), (64, 40, 32)]


@pytest.mark.parametrize("K,N,group", RESIDUAL_CASES)
@pytest.mark.parametrize("in_place", [False, True])
def test_residual_output_equals_gemv_then_add(capi, torch, K, N, group, in_place):
    qw, sc, qz = weights(torch, f"chain_res_{K}_{N}", K, N, group)
    x = bf16_rand(torch, (1, K), K + N)
    resid = bf16_rand(torch, (1, N), N, 2.0)
    ws = capi.make_workspace(1, K, N)
    y = torch.empty((1, N), dtype=torch.bfloat16, device="cuda")
    capi.gemv_awq_bf16(x, qw, sc, qz, y, group, ws)
    expected = (resid.float() + y.float()).bfloat16()

    parts = (N + 255) // 256
    sumsq = torch.full((parts, 4), float("nan"), dtype=torch.float32, device="cuda")
    out = resid.clone() if in_place else torch.full((1, N), float("nan"), dtype=torch.bfloat16, device="cuda")
    capi.gemv_awq_chain_bf16({"in_kind": capi.IN_ROW, "x": x, "out_kind": capi.OUT_RESIDUAL,
                              "residual_in": out if in_place else resid, "residual_out": out, "sumsq_out": sumsq},
                             qw, sc, qz, K, N, group, ws)
    torch.cuda.synchronize()
    assert torch.equal(out.view(torch.int16), expected.view(torch.int16))
    ref = tile_sums(torch, expected)
    live = (ref > 0) | (torch.arange(parts * 4, device="cuda").view(parts, 4) * 64 < N)  # quarters that hold columns
    assert torch.allclose(sumsq.double()[live], ref[live], rtol=1e-5, atol=0)


def test_swiglu_and_attention_inputs_with_residual_output(capi, torch):
    # SwiGLU in, residual out
    K, N, group = 1024, 512, 128
    qw, sc, qz = weights(torch, "chain_swiglu", K, N, group)
    gu = bf16_rand(torch, (1, 2 * K), 3, 1.5)
    resid = bf16_rand(torch, (1, N), 4)
    ws = capi.make_workspace(1, K, N)
    y = torch.empty((1, N), dtype=torch.bfloat16, device="cuda")
    capi.gemv_awq_swiglu_bf16(gu[:, :K], gu[:, K:], qw, sc, qz, y, group, ws)
    expected = (resid.float() + y.float()).bfloat16()
    sumsq = torch.empty((N // 256, 4), dtype=torch.float32, device="cuda")
    out = torch.empty_like(resid)
    capi.gemv_awq_chain_bf16({"in_kind": capi.IN_SWIGLU, "gate": gu[:, :K], "up": gu[:, K:],
                              "out_kind": capi.OUT_RESIDUAL, "residual_in": resid, "residual_out": out,
                              "sumsq_out": sumsq}, qw, sc, qz, K, N, group, ws)
    torch.cuda.synchronize()
    assert torch.equal(out.view(torch.int16), expected.view(torch.int16))

    # attention merge in, residual out
    n_q, n_kv, pos_value, max_pos, N = 4, 2, 100, 192, 512
    K = n_q * 128
    qw, sc, qz = weights(torch, "chain_attn", K, N, group)
    q = bf16_rand(torch, (n_q, 128), 5)
    kc = bf16_rand(torch, (max_pos, n_kv, 128), 6)
    vc = bf16_rand(torch, (max_pos, n_kv, 128), 7)
    pos = torch.tensor([pos_value], dtype=torch.int32, device="cuda")
    ws = capi.make_workspace(1, K, N)
    attn_ws = capi.attn_decode_workspace(n_q, max_pos)
    attn = torch.empty((1, K), dtype=torch.bfloat16, device="cuda")
    capi.attn_decode_bf16(q, kc, vc, attn, n_q, n_kv, pos, max_pos, attn_ws)
    capi.gemv_awq_bf16(attn, qw, sc, qz, y, group, ws)
    expected = (resid.float() + y.float()).bfloat16()
    capi.attn_decode_partial_bf16(q, kc, vc, n_q, n_kv, pos, max_pos, attn_ws)
    out.fill_(float("nan"))
    capi.gemv_awq_chain_bf16({"in_kind": capi.IN_ATTN, "attn_workspace": attn_ws, "attn_workspace_bytes": attn_ws.numel(),
                              "n_q_heads": n_q, "n_kv_heads": n_kv, "max_positions": max_pos,
                              "out_kind": capi.OUT_RESIDUAL, "residual_in": resid, "residual_out": out,
                              "sumsq_out": sumsq}, qw, sc, qz, K, N, group, ws)
    torch.cuda.synchronize()
    assert torch.equal(out.view(torch.int16), expected.view(torch.int16))
    assert torch.allclose(sumsq.double(), tile_sums(torch, expected), rtol=1e-5, atol=0)


NORM_CASES = [(4096, 24576, 128), (4096, 6144, 128), (5120, 10240, 128), (256, 520, 32), (320, 64, 32)]


@pytest.mark.parametrize("K,N,group", NORM_CASES)
def test_norm_input_matches_rmsnorm_then_gemv(capi, torch, oracle, K, N, group):
    eps = 1e-6
    p = synth.make_awq_problem(f"chain_norm_{K}_{N}", 1, K, N, group)
    qw, sc, qz = H.to_dev_i32(p["qweight"], torch), H.to_dev_f16(p["scales"], torch), H.to_dev_i32(p["qzeros"], torch)
    row = bf16_rand(torch, (1, K), K, 2.0)
    gain = (1 + 0.1 * torch.randn((K,), device="cuda")).bfloat16()
    ws = capi.make_workspace(1, K, N)
    h = torch.empty((1, K), dtype=torch.bfloat16, device="cuda")
    y_sep = torch.empty((1, N), dtype=torch.bfloat16, device="cuda")
    capi.rmsnorm_bf16(row.clone(), gain, h, eps)
    capi.gemv_awq_bf16(h, qw, sc, qz, y_sep, group, ws)

    sumsq = tile_sums(torch, row).float()   # what a residual output would have left, to fp32 rounding
    y = torch.full((1, N), float("nan"), dtype=torch.bfloat16, device="cuda")
    capi.gemv_awq_chain_bf16({"in_kind": capi.IN_NORM, "norm_row": row, "norm_sumsq": sumsq, "norm_parts": sumsq.shape[0],
                              "norm_gain": gain, "norm_eps": eps, "out_kind": capi.OUT_ROW, "y": y},
                             qw, sc, qz, K, N, group, ws)
    torch.cuda.synchronize()
    assert torch.isfinite(y.float()).all()
    assert rel_l2(y, y_sep) <= 1e-3
    # and against the oracle's GEMV on the normalised row
    ref64 = oracle.gemv_awq_f64(H.bf16_bits(h, torch), p["qweight"], p["scales"], p["qzeros"], group)
    ref_rounded = H.bf16_to_f64(oracle.f32_to_bf16(ref64.astype(np.float32)))
    assert H.rel_l2(H.bf16_to_f64(H.bf16_bits(y, torch)), ref_rounded) <= 1.5e-3


def test_residual_sums_feed_the_norm_input_of_the_next_launch(capi, torch):
    """Two links: o projection with residual output, then gate|up with the norm input."""
    K1, H_, N2, group, eps = 512, 1024, 2048, 128, 1e-6
    qw1, sc1, qz1 = weights(torch, "chain_link1", K1, H_, group)
    qw2, sc2, qz2 = weights(torch, "chain_link2", H_, N2, group)
    x = bf16_rand(torch, (1, K1), 1)
    resid = bf16_rand(torch, (1, H_), 2, 2.0)
    gain = (1 + 0.1 * torch.randn((H_,), device="cuda")).bfloat16()
    ws = capi.make_workspace(1, max(K1, H_), max(H_, N2))
    # separate launches
    o = torch.empty((1, H_), dtype=torch.bfloat16, device="cuda")
    capi.gemv_awq_bf16(x, qw1, sc1, qz1, o, group, ws)
    r_sep = resid.clone()
    h = torch.empty_like(r_sep)
    capi.add_rmsnorm_bf16(r_sep, o, gain, h, eps)
    y_sep = torch.empty((1, N2), dtype=torch.bfloat16, device="cuda")
    capi.gemv_awq_bf16(h, qw2, sc2, qz2, y_sep, group, ws)
    # chained
    r = resid.clone()
    sumsq = torch.empty((H_ // 256, 4), dtype=torch.float32, device="cuda")
    capi.gemv_awq_chain_bf16({"in_kind": capi.IN_ROW, "x": x, "out_kind": capi.OUT_RESIDUAL, "residual_in": r,
                              "residual_out": r, "sumsq_out": sumsq}, qw1, sc1, qz1, K1, H_, group, ws)
    y = torch.empty((1, N2), dtype=torch.bfloat16, device="cuda")
    capi.gemv_awq_chain_bf16({"in_kind": capi.IN_NORM, "norm_row": r, "norm_sumsq": sumsq, "norm_parts": H_ // 256,
                              "norm_gain": gain, "norm_eps": eps, "out_kind": capi.OUT_ROW, "y": y},
                             qw2, sc2, qz2, H_, N2, group, ws)
    torch.cuda.synchronize()
    assert torch.equal(r.view(torch.int16), r_sep.view(torch.int16))
    assert rel_l2(y, y_sep) <= 1e-3


def test_norm_input_with_rotary_output(capi, torch):
    K, n_q, n_kv, group, eps, theta, pos_value, max_pos = 512, 4, 2, 128, 1e-6, 1e6, 21, 32
    N = (n_q + 2 * n_kv) * 128
    qw, sc, qz = weights(torch, "chain_rope", K, N, group)
    row = bf16_rand(torch, (1, K), 9, 2.0)
    gain = (1 + 0.1 * torch.randn((K,), device="cuda")).bfloat16()
    hg = (1 + 0.1 * torch.randn((128,), device="cuda")).bfloat16()
    pos = torch.tensor([pos_value], dtype=torch.int32, device="cuda")
    ws = capi.make_workspace(1, K, N)
    h = torch.empty((1, K), dtype=torch.bfloat16, device="cuda")
    qkv = torch.empty((1, N), dtype=torch.bfloat16, device="cuda")
    capi.rmsnorm_bf16(row.clone(), gain, h, eps)
    capi.gemv_awq_bf16(h, qw, sc, qz, qkv, group, ws)
    q_sep = torch.empty((1, n_q * 128), dtype=torch.bfloat16, device="cuda")
    k_sep = torch.zeros((max_pos, n_kv, 128), dtype=torch.bfloat16, device="cuda")
    v_sep = torch.zeros_like(k_sep)
    capi.qk_norm_rope_bf16(qkv, hg, hg, q_sep, k_sep, v_sep, n_q, n_kv, pos, theta, eps)

    q_one = torch.full_like(q_sep, float("nan"))
    k_one, v_one = torch.zeros_like(k_sep), torch.zeros_like(v_sep)
    sumsq = tile_sums(torch, row).float()
    capi.gemv_awq_chain_bf16({"in_kind": capi.IN_NORM, "norm_row": row, "norm_sumsq": sumsq, "norm_parts": sumsq.shape[0],
                              "norm_gain": gain, "norm_eps": eps, "out_kind": capi.OUT_QKV_ROPE, "q_gain": hg,
                              "k_gain": hg, "q_out": q_one, "k_cache": k_one, "v_cache": v_one, "pos": pos,
                              "rope_n_q_heads": n_q, "rope_n_kv_heads": n_kv, "rope_theta": theta, "qk_eps": eps},
                             qw, sc, qz, K, N, group, ws)
    torch.cuda.synchronize()
    # normalised, rotated heads are O(1): a last-bit difference in the normalised input moves an output by
    # at most a few bf16 ulp (2^-7 at magnitude 1..2)
    for a, b in ((q_one, q_sep), (k_one[pos_value], k_sep[pos_value]), (v_one[pos_value], v_sep[pos_value])):
        assert torch.isfinite(a.float()).all()
        assert (a.float() - b.float()).abs().max().item() <= 0.05
        assert rel_l2(a, b) <= 5e-3


@pytest.mark.parametrize("K", [8192, 12288])
def test_row_input_with_rotary_output_on_tall_k(capi, torch, K):
    """32 and 48 K tiles per column: the finishing wave of a head adds the even and the odd tiles separately, in one
    and in two batches of each, and must return the bits of the plain launch followed by the per-head kernel."""
    n_q, n_kv, group, eps, theta, pos_value, max_pos = 2, 1, 128, 1e-6, 1e6, 5, 8
    N = (n_q + 2 * n_kv) * 128
    qw, sc, qz = weights(torch, f"chain_rope_tall_{K}", K, N, group)
    x = bf16_rand(torch, (1, K), K)
    hg = (1 + 0.1 * torch.randn((128,), device="cuda")).bfloat16()
    pos = torch.tensor([pos_value], dtype=torch.int32, device="cuda")
    ws = capi.make_workspace(1, K, N)
    qkv = torch.empty((1, N), dtype=torch.bfloat16, device="cuda")
    capi.gemv_awq_bf16(x, qw, sc, qz, qkv, group, ws)
    q_sep = torch.empty((1, n_q * 128), dtype=torch.bfloat16, device="cuda")
    k_sep = torch.zeros((max_pos, n_kv, 128), dtype=torch.bfloat16, device="cuda")
    v_sep = torch.zeros_like(k_sep)
    capi.qk_norm_rope_bf16(qkv, hg, hg, q_sep, k_sep, v_sep, n_q, n_kv, pos, theta, eps)

    for _ in range(2):  # the second launch finds the counters as the first one left them
        q_one = torch.full_like(q_sep, float("nan"))
        k_one, v_one = torch.zeros_like(k_sep), torch.zeros_like(v_sep)
        capi.gemv_awq_chain_bf16({"in_kind": capi.IN_ROW, "x": x, "out_kind": capi.OUT_QKV_ROPE, "q_gain": hg,
                                  "k_gain": hg, "q_out": q_one, "k_cache": k_one, "v_cache": v_one, "pos": pos,
                                  "rope_n_q_heads": n_q, "rope_n_kv_heads": n_kv, "rope_theta": theta, "qk_eps": eps},
                                 qw, sc, qz, K, N, group, ws)
        torch.cuda.synchronize()
        for a, b in ((q_one, q_sep), (k_one, k_sep), (v_one, v_sep)):
            assert torch.equal(a.view(torch.int16), b.view(torch.int16))
    # and the plain launch still works on the same workspace
    again = torch.empty_like(qkv)
    capi.gemv_awq_bf16(x, qw, sc, qz, again, group, ws)
    torch.cuda.synchronize()
    assert torch.equal(again.view(torch.int16), qkv.view(torch.int16))


def test_chain_rejects_bad_descriptors(capi, torch):
    K, N, group = 512, 512, 128
    qw, sc, qz = weights(torch, "chain_bad", K, N, group)
    x = torch.zeros((1, K), dtype=torch.bfloat16, device="cuda")
    y = torch.zeros((1, N), dtype=torch.bfloat16, device="cuda")
    s2 = torch.zeros((2, 4), dtype=torch.float32, device="cuda")
    ws = capi.make_workspace(1, K, N)

    def code(desc):
        with pytest.raises(capi.KxError) as e:
            capi.gemv_awq_chain_bf16(desc, qw, sc, qz, K, N, group, ws)
        return e.value.code

    assert code({"in_kind": 9, "out_kind": capi.OUT_ROW, "y": y}) == -2
    assert code({"in_kind": capi.IN_ROW, "x": x, "out_kind": 7}) == -2
    assert code({"in_kind": capi.IN_ROW, "out_kind": capi.OUT_ROW, "y": y}) == -1                      # no x
    assert code({"in_kind": capi.IN_ROW, "x": x, "out_kind": capi.OUT_RESIDUAL, "residual_in": y}) == -1  # no out
    assert code({"in_kind": capi.IN_NORM, "norm_row": x, "norm_sumsq": s2, "norm_parts": 3, "norm_gain": x,
                 "out_kind": capi.OUT_ROW, "y": y}) == -2                                                # parts != K / 256
    assert code({"in_kind": capi.IN_NORM, "norm_row": x, "norm_sumsq": s2, "norm_parts": 2, "norm_gain": x,
                 "out_kind": capi.OUT_RESIDUAL, "residual_in": x, "residual_out": x, "sumsq_out": s2}) == -5
    # overlap is judged on byte ranges, not on base pointers: an outgoing row that starts inside the activations
    # (or inside a shifted copy of the incoming residual row) is refused as well
    big = torch.zeros((1, 2 * K), dtype=torch.bfloat16, device="cuda")
    inside = big[:, 64:64 + N]
    r_in = torch.zeros((1, N), dtype=torch.bfloat16, device="cuda")
    assert code({"in_kind": capi.IN_ROW, "x": big[:, :K], "out_kind": capi.OUT_RESIDUAL, "residual_in": r_in,
                 "residual_out": inside, "sumsq_out": s2}) == -5
    assert code({"in_kind": capi.IN_SWIGLU, "gate": big[:, :K], "up": x, "out_kind": capi.OUT_RESIDUAL,
                 "residual_in": r_in, "residual_out": inside, "sumsq_out": s2}) == -5
    assert code({"in_kind": capi.IN_SWIGLU, "gate": x, "up": big[:, :K], "out_kind": capi.OUT_RESIDUAL,
                 "residual_in": r_in, "residual_out": inside, "sumsq_out": s2}) == -5
    assert code({"in_kind": capi.IN_ROW, "x": x, "out_kind": capi.OUT_RESIDUAL, "residual_in": big[:, :N],
                 "residual_out": inside, "sumsq_out": s2}) == -5
    # in place (the same row in and out) stays allowed
    capi.gemv_awq_chain_bf16({"in_kind": capi.IN_ROW, "x": x, "out_kind": capi.OUT_RESIDUAL, "residual_in": r_in,
                              "residual_out": r_in, "sumsq_out": s2}, qw, sc, qz, K, N, group, ws)
    torch.cuda.synchronize()
    assert code({"in_kind": capi.IN_ATTN, "attn_workspace": ws, "attn_workspace_bytes": 16, "n_q_heads": 4,
                 "n_kv_heads": 2, "max_positions": 64, "out_kind": capi.OUT_ROW, "y": y}) == -3
