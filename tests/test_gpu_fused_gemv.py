"""GPU parity of the AWQ GEMV entry points that produce their activations on the way in.

Two independent checks per entry point:
  * against the stand-alone kernels run back to back (SwiGLU or add+RMSNorm, then the GEMV on the
    vector kernel): bitwise for the SwiGLU prologue and for the norm prologue on workgroups of eight
    waves, whose sum of squares is added in the stand-alone kernel's order; otherwise the
    normalised row may differ by an ulp in a few places and the tolerance of the GEMV applies;
  * against the CPU oracle's fp64 GEMV fed with activations computed by torch in fp32 with the
    same rounding points (relative L2 <= 1e-3 against the rounded result).
"""
import numpy as np
import pytest

from mykuiperllama_amd import synth
from tests import helpers as H

pytestmark = pytest.mark.gpu

REL_L2_ROUNDED = 1e-3


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


def weights(torch, name, M, K, N, group):
    p = synth.make_awq_problem(name, M, K, N, group)
    dev = (H.to_dev_i32(p["qweight"], torch), H.to_dev_f16(p["scales"], torch), H.to_dev_i32(p["qzeros"], torch))
    return p, dev


def oracle_check(oracle, torch, p, x_dev, y_dev):
    x_bits = H.bf16_bits(x_dev, torch)
    ref64 = oracle.gemv_awq_f64(x_bits, p["qweight"], p["scales"], p["qzeros"], p["group"])
    ref_rounded = H.bf16_to_f64(oracle.f32_to_bf16(ref64.astype(np.float32)))
    got = H.bf16_to_f64(H.bf16_bits(y_dev, torch))
    assert np.isfinite(got).all()
    assert H.rel_l2(got, ref_rounded) <= REL_L2_ROUNDED
    assert np.abs(got - ref_rounded).max() <= 2 * H.bf16_ulp_of(np.abs(ref64).max())


SWIGLU_CASES = [
    # M, K, N, group, gate and up as halves of one tensor?
    (1, 12288, 4096, 128, True),    # Qwen3-8B down_proj
    (1, 25600, 5120, 128, True),    # Qwen3-32B down_proj
    (1, 256, 512, 128, False),
    (1, 128, 264, 32, False),       # K below one full workgroup, ragged N
    (1, 96, 40, 32, True),
    (2, 1024, 2048, 128, True),
    (3, 4096, 1024, 128, False),
    (5, 2048, 512, 64, True),
    (16, 512, 256, 128, True),
]


@pytest.mark.parametrize("M,K,N,group,halves", SWIGLU_CASES)
def test_swiglu_prologue_equals_separate_launches(capi, torch, oracle, M, K, N, group, halves):
    p, (qw, sc, qz) = weights(torch, f"fused_swiglu_{M}_{K}_{N}", M, K, N, group)
    g = torch.Generator(device="cuda")
    g.manual_seed(K * 31 + N + M)
    if halves:
        gu = (torch.randn((M, 2 * K), device="cuda", generator=g) * 1.5).bfloat16()
        gate, up = gu[:, :K], gu[:, K:]
    else:
        gate = (torch.randn((M, K), device="cuda", generator=g) * 1.5).bfloat16()
        up = torch.randn((M, K), device="cuda", generator=g).bfloat16()
    ws = capi.make_workspace(M, K, N)
    act = torch.empty((M, K), dtype=torch.bfloat16, device="cuda")
    y_sep = torch.full((M, N), float("nan"), dtype=torch.bfloat16, device="cuda")
    y_fused = torch.full((M, N), float("nan"), dtype=torch.bfloat16, device="cuda")
    capi.swiglu_bf16(gate.contiguous(), up.contiguous(), act)
    # several rows: the fused launch runs on the kernel the plain entry point picks by shape
    capi.set_awq_kernel_policy(1 if M == 1 else 0)
    capi.gemv_awq_bf16(act, qw, sc, qz, y_sep, group, ws)
    capi.gemv_awq_swiglu_bf16(gate, up, qw, sc, qz, y_fused, group, ws)
    torch.cuda.synchronize()
    assert np.array_equal(H.bf16_bits(y_fused, torch), H.bf16_bits(y_sep, torch))
    # activations recomputed by torch with the same rounding points feed the oracle
    silu = torch.nn.functional.silu(gate.float()).bfloat16().float()
    act_ref = (silu * up.float()).bfloat16()
    # expf of the kernel and torch's sigmoid may round an activation differently once in a while
    assert (act_ref.view(torch.int16).int() - act.view(torch.int16).int()).abs().max().item() <= 1
    oracle_check(oracle, torch, p, act, y_fused)


ADDNORM_CASES = [
    # M, K, N, group, with delta, with residual_out
    (1, 4096, 6144, 128, True, True),    # Qwen3-8B fused q/k/v
    (1, 4096, 24576, 128, True, True),   # Qwen3-8B fused gate/up
    (1, 5120, 10240, 128, True, True),   # Qwen3-32B fused q/k/v: two pieces of the row per thread
    (1, 8192, 512, 128, True, False),
    (1, 4096, 1024, 128, False, False),  # plain RMSNorm (first layer)
    (1, 4096, 1024, 128, False, True),
    (1, 256, 512, 32, True, True),
    (1, 128, 264, 32, True, True),       # four waves per workgroup
    (1, 64, 40, 32, True, True),
    (2, 1024, 2048, 128, True, True),
    (5, 2048, 520, 64, True, True),
]


@pytest.mark.parametrize("M,K,N,group,with_delta,with_out", ADDNORM_CASES)
def test_addnorm_prologue_equals_separate_launches(capi, torch, oracle, M, K, N, group, with_delta, with_out):
    eps = 1e-6
    p, (qw, sc, qz) = weights(torch, f"fused_addnorm_{M}_{K}_{N}", M, K, N, group)
    g = torch.Generator(device="cuda")
    g.manual_seed(K * 17 + N + M)
    resid = (torch.randn((M, K), device="cuda", generator=g) * 2.0).bfloat16()
    delta = torch.randn((M, K), device="cuda", generator=g).bfloat16() if with_delta else None
    gain = (1 + 0.1 * torch.randn((K,), device="cuda", generator=g)).bfloat16()
    ws = capi.make_workspace(M, K, N)

    x_sep = resid.clone()
    h_sep = torch.empty((M, K), dtype=torch.bfloat16, device="cuda")
    y_sep = torch.full((M, N), float("nan"), dtype=torch.bfloat16, device="cuda")
    if with_delta:
        capi.add_rmsnorm_bf16(x_sep, delta, gain, h_sep, eps)
    else:
        capi.rmsnorm_bf16(x_sep, gain, h_sep, eps)
    capi.gemv_awq_bf16(h_sep, qw, sc, qz, y_sep, group, ws)

    resid_before = resid.clone()
    r_out = torch.full((M, K), float("nan"), dtype=torch.bfloat16, device="cuda") if with_out else None
    y_fused = torch.full((M, N), float("nan"), dtype=torch.bfloat16, device="cuda")
    capi.gemv_awq_addnorm_bf16(resid, delta, gain, eps, r_out, qw, sc, qz, y_fused, group, ws)
    torch.cuda.synchronize()

    assert torch.equal(resid, resid_before), "the incoming residual stream is read only"
    if with_out:
        assert np.array_equal(H.bf16_bits(r_out, torch), H.bf16_bits(x_sep, torch))
    if K >= 256:
        assert np.array_equal(H.bf16_bits(y_fused, torch), H.bf16_bits(y_sep, torch))
    else:
        a, b = y_fused.float().cpu().numpy(), y_sep.float().cpu().numpy()
        assert H.rel_l2(a, b) <= REL_L2_ROUNDED
    # fp32 torch restatement of the prologue, then the oracle's GEMV
    r = (resid.float() + delta.float()).bfloat16().float() if with_delta else resid.float()
    inv = torch.rsqrt((r * r).mean(dim=-1, keepdim=True) + eps)
    h_ref = (gain.float() * (r * inv).bfloat16().float()).bfloat16()
    assert (h_ref.view(torch.int16).int() - h_sep.view(torch.int16).int()).abs().max().item() <= 1
    oracle_check(oracle, torch, p, h_sep, y_fused)


QKV_CASES = [
    # hidden K, n_q, n_kv, group, with delta
    (4096, 32, 8, 128, True),    # Qwen3-8B
    (5120, 64, 8, 128, True),    # Qwen3-32B
    (4096, 32, 8, 128, False),   # first layer: no delta
    (512, 4, 2, 128, True),
    (128, 2, 1, 32, True),       # four waves per workgroup
    (64, 2, 2, 32, True),        # K in one workgroup: no split, every workgroup finishes its own tile
    (8192, 4, 2, 128, True),     # 32 K tiles: the read-back adds the even and the odd tiles separately
]


@pytest.mark.parametrize("K,n_q,n_kv,group,with_delta", QKV_CASES)
def test_qkv_rope_launch_equals_separate_launches(capi, torch, K, n_q, n_kv, group, with_delta):
    eps, theta, pos_value, max_pos = 1e-6, 1e6, 37, 48
    N = (n_q + 2 * n_kv) * 128
    _, (qw, sc, qz) = weights(torch, f"fused_qkv_{K}_{n_q}_{n_kv}", 1, K, N, group)
    g = torch.Generator(device="cuda")
    g.manual_seed(K + n_q)
    resid = (torch.randn((1, K), device="cuda", generator=g) * 2.0).bfloat16()
    delta = torch.randn((1, K), device="cuda", generator=g).bfloat16() if with_delta else None
    gain = (1 + 0.1 * torch.randn((K,), device="cuda", generator=g)).bfloat16()
    q_gain = (1 + 0.1 * torch.randn((128,), device="cuda", generator=g)).bfloat16()
    k_gain = (1 + 0.1 * torch.randn((128,), device="cuda", generator=g)).bfloat16()
    pos = torch.tensor([pos_value], dtype=torch.int32, device="cuda")
    ws = capi.make_workspace(1, K, N)

    def caches():
        return (torch.full((max_pos, n_kv, 128), 3.0, dtype=torch.bfloat16, device="cuda"),
                torch.full((max_pos, n_kv, 128), 5.0, dtype=torch.bfloat16, device="cuda"))

    # separate: add + norm + GEMV, then the stand-alone per-head kernel
    k_sep, v_sep = caches()
    qkv = torch.empty((1, N), dtype=torch.bfloat16, device="cuda")
    r_sep = torch.empty((1, K), dtype=torch.bfloat16, device="cuda")
    q_sep = torch.empty((1, n_q * 128), dtype=torch.bfloat16, device="cuda")
    capi.gemv_awq_addnorm_bf16(resid, delta, gain, eps, r_sep, qw, sc, qz, qkv, group, ws)
    capi.qk_norm_rope_bf16(qkv, q_gain, k_gain, q_sep, k_sep, v_sep, n_q, n_kv, pos, theta, eps)
    # one launch
    k_one, v_one = caches()
    r_one = torch.empty((1, K), dtype=torch.bfloat16, device="cuda")
    q_one = torch.full((1, n_q * 128), float("nan"), dtype=torch.bfloat16, device="cuda")
    capi.gemv_awq_qkv_rope_bf16(resid, delta, gain, eps, r_one, qw, sc, qz, q_gain, k_gain, q_one, k_one, v_one,
                                n_q, n_kv, pos, theta, eps, group, ws)
    torch.cuda.synchronize()
    for a, b in ((q_one, q_sep), (k_one, k_sep), (v_one, v_sep), (r_one, r_sep)):
        assert torch.equal(a.view(torch.int16), b.view(torch.int16))
    # only row `pos` of the caches was touched
    assert (k_one[:pos_value] == 3.0).all() and (k_one[pos_value + 1:] == 3.0).all()
    assert (v_one[:pos_value] == 5.0).all() and (v_one[pos_value + 1:] == 5.0).all()
    assert torch.isfinite(q_one.float()).all()
    # a position the caches have no row for: nothing is appended
    k_off, v_off = caches()
    for bad in (max_pos, -1):
        capi.gemv_awq_qkv_rope_bf16(resid, delta, gain, eps, r_one, qw, sc, qz, q_gain, k_gain, q_one, k_off, v_off,
                                    n_q, n_kv, torch.tensor([bad], dtype=torch.int32, device="cuda"), theta, eps,
                                    group, ws)
    torch.cuda.synchronize()
    assert (k_off == 3.0).all() and (v_off == 5.0).all()


def test_qkv_rope_launch_rejects_bad_arguments(capi, torch):
    K, n_q, n_kv, group = 256, 3, 1, 128  # five heads do not fill column tiles of two heads
    N = (n_q + 2 * n_kv) * 128
    _, (qw, sc, qz) = weights(torch, "fused_qkv_bad", 1, K, N, group)
    x = torch.zeros((1, K), dtype=torch.bfloat16, device="cuda")
    gain = torch.ones((K,), dtype=torch.bfloat16, device="cuda")
    hg = torch.ones((128,), dtype=torch.bfloat16, device="cuda")
    q = torch.zeros((1, n_q * 128), dtype=torch.bfloat16, device="cuda")
    kc = torch.zeros((4, n_kv, 128), dtype=torch.bfloat16, device="cuda")
    pos = torch.zeros(1, dtype=torch.int32, device="cuda")
    ws = capi.make_workspace(1, K, N)
    with pytest.raises(capi.KxError) as e:
        capi.gemv_awq_qkv_rope_bf16(x, None, gain, 1e-6, None, qw, sc, qz, hg, hg, q, kc, kc.clone(), n_q, n_kv, pos,
                                    1e6, 1e-6, group, ws)
    assert e.value.code == -2
    with pytest.raises(capi.KxError) as e:
        capi.gemv_awq_qkv_rope_bf16(x, None, gain, 1e-6, x, qw, sc, qz, hg, hg, q, kc, kc.clone(), 2, 1, pos,
                                    1e6, 1e-6, group, ws)
    assert e.value.code == -5
    with pytest.raises(capi.KxError) as e:
        capi.gemv_awq_qkv_rope_bf16(x, None, gain, 1e-6, None, qw, sc, qz, hg, hg, q, kc, kc.clone(), 2, 1, None,
                                    1e6, 1e-6, group, ws)
    assert e.value.code == -1


MERGE_CASES = [
    # n_q, n_kv, pos, max_positions, N, group
    (32, 8, 4096, 4224, 4096, 128),   # Qwen3-8B at the benchmark's context
    (32, 8, 0, 4224, 4096, 128),      # a single cached position
    (32, 8, 63, 5120, 1024, 128),     # the longest cache walked in chunks of 64 positions
    (64, 8, 8192, 8320, 5120, 128),   # Qwen3-32B at its benchmark context: chunks of 128 positions
    (8, 2, 10239, 10240, 512, 128),   # the longest context the merging projection takes
    (8, 2, 5000, 5121, 512, 128),     # just past the switch to chunks of 128
    (64, 8, 1000, 1100, 5120, 128),   # eight query heads per KV head
    (4, 2, 37, 48, 512, 128),
    (40, 8, 700, 768, 1024, 128),     # Qwen3-14B's grouping: five query heads per KV head
    (6, 2, 300, 6000, 264, 64),       # three per KV head, chunks of 128 positions
    (2, 1, 100, 128, 264, 32),        # K = 256, ragged N
    (1, 1, 5, 64, 64, 32),            # K = 128: four waves, one head
    (4, 4, 127, 128, 256, 64),        # no grouping, context ends on a chunk boundary
]


@pytest.mark.parametrize("n_q,n_kv,pos_value,max_pos,N,group", MERGE_CASES)
def test_attention_merge_in_the_o_projection_equals_separate_launches(capi, torch, n_q, n_kv, pos_value, max_pos, N,
                                                                      group):
    K = n_q * 128
    _, (qw, sc, qz) = weights(torch, f"fused_merge_{n_q}_{n_kv}_{N}", 1, K, N, group)
    g = torch.Generator(device="cuda")
    g.manual_seed(n_q * 1000 + pos_value)
    q = torch.randn((n_q, 128), device="cuda", generator=g).bfloat16()
    kc = torch.randn((max_pos, n_kv, 128), device="cuda", generator=g).bfloat16()
    vc = torch.randn((max_pos, n_kv, 128), device="cuda", generator=g).bfloat16()
    kc[pos_value + 1:] = float("nan")  # rows past the context must not matter
    vc[pos_value + 1:] = float("nan")
    pos = torch.tensor([pos_value], dtype=torch.int32, device="cuda")
    ws = capi.make_workspace(1, K, N)

    attn_ws = capi.attn_decode_workspace(n_q, max_pos)
    attn_ws.view(torch.float32)[: attn_ws.numel() // 4].fill_(float("nan"))  # nothing stale may be read
    attn = torch.empty((1, K), dtype=torch.bfloat16, device="cuda")
    y_sep = torch.full((1, N), float("nan"), dtype=torch.bfloat16, device="cuda")
    capi.attn_decode_bf16(q, kc, vc, attn, n_q, n_kv, pos, max_pos, attn_ws)
    capi.gemv_awq_bf16(attn, qw, sc, qz, y_sep, group, ws)

    attn_ws2 = capi.attn_decode_workspace(n_q, max_pos)
    attn_ws2.view(torch.float32)[: attn_ws2.numel() // 4].fill_(float("nan"))
    y_one = torch.full((1, N), float("nan"), dtype=torch.bfloat16, device="cuda")
    capi.attn_decode_partial_bf16(q, kc, vc, n_q, n_kv, pos, max_pos, attn_ws2)
    capi.gemv_awq_attn_merge_bf16(attn_ws2, n_q, n_kv, max_pos, qw, sc, qz, y_one, group, ws)
    torch.cuda.synchronize()
    assert torch.isfinite(y_sep.float()).all()
    assert torch.equal(y_one.view(torch.int16), y_sep.view(torch.int16))


def test_attention_merge_rejects_long_contexts_and_bad_arguments(capi, torch):
    n_q, n_kv, N, group = 2, 1, 256, 128
    _, (qw, sc, qz) = weights(torch, "fused_merge_bad", 1, n_q * 128, N, group)
    y = torch.zeros((1, N), dtype=torch.bfloat16, device="cuda")
    ws = capi.make_workspace(1, n_q * 128, N)
    long_ws = capi.attn_decode_workspace(n_q, 10241)
    with pytest.raises(capi.KxError) as e:
        capi.gemv_awq_attn_merge_bf16(long_ws, n_q, n_kv, 10241, qw, sc, qz, y, group, ws)
    assert e.value.code == -2
    small_ws = capi.attn_decode_workspace(n_q, 64)
    with pytest.raises(capi.KxError) as e:
        capi.gemv_awq_attn_merge_bf16(small_ws, n_q, n_kv, 4096, qw, sc, qz, y, group, ws)
    assert e.value.code == -3
    rc = capi.load().kx_gemv_awq_attn_merge_bf16(None, 1 << 20, n_q, n_kv, 128, 64, qw.data_ptr(), sc.data_ptr(),
                                                 qz.data_ptr(), y.data_ptr(), N, group, ws.data_ptr(), ws.numel(),
                                                 None)
    assert rc == -1


def test_fused_launches_are_deterministic_and_leave_the_workspace_reusable(capi, torch):
    M, K, N, group = 1, 4096, 6144, 128
    _, (qw, sc, qz) = weights(torch, "fused_repeat", M, K, N, group)
    g = torch.Generator(device="cuda")
    g.manual_seed(5)
    resid = torch.randn((M, K), device="cuda", generator=g).bfloat16()
    delta = torch.randn((M, K), device="cuda", generator=g).bfloat16()
    gain = torch.ones((K,), device="cuda").bfloat16()
    ws = capi.make_workspace(M, K, N)
    outs = []
    for _ in range(4):
        y = torch.empty((M, N), dtype=torch.bfloat16, device="cuda")
        r = torch.empty((M, K), dtype=torch.bfloat16, device="cuda")
        capi.gemv_awq_addnorm_bf16(resid, delta, gain, 1e-6, r, qw, sc, qz, y, group, ws)
        outs.append(y)
    torch.cuda.synchronize()
    for y in outs[1:]:
        assert torch.equal(y.view(torch.int16), outs[0].view(torch.int16))


def test_fused_entry_points_reject_bad_arguments(capi, torch):
    M, K, N, group = 1, 1024, 512, 128
    _, (qw, sc, qz) = weights(torch, "fused_bad", M, K, N, group)
    x = torch.zeros((M, K), dtype=torch.bfloat16, device="cuda")
    gain = torch.ones((K,), dtype=torch.bfloat16, device="cuda")
    y = torch.zeros((M, N), dtype=torch.bfloat16, device="cuda")
    ws = capi.make_workspace(M, K, N)
    with pytest.raises(capi.KxError) as e:
        capi.gemv_awq_addnorm_bf16(x, None, gain, 1e-6, x, qw, sc, qz, y, group, ws)  # in place
    assert e.value.code == -5
    with pytest.raises(capi.KxError) as e:
        capi.gemv_awq_addnorm_bf16(x, x, gain, 1e-6, None, qw, sc, qz, y, group, None)  # split K, no workspace
    assert e.value.code == -3
    with pytest.raises(capi.KxError) as e:
        capi.gemv_awq_addnorm_bf16(x, None, None, 1e-6, None, qw, sc, qz, y, group, ws)
    assert e.value.code == -1
    rc = capi.load().kx_gemv_awq_swiglu_bf16(x.data_ptr(), None, K, qw.data_ptr(), sc.data_ptr(), qz.data_ptr(),
                                             y.data_ptr(), M, K, N, group, ws.data_ptr(), ws.numel(), None)
    assert rc == -1  # up missing
    rc = capi.load().kx_gemv_awq_swiglu_bf16(x.data_ptr(), x.data_ptr(), K - 8, qw.data_ptr(), sc.data_ptr(),
                                             qz.data_ptr(), y.data_ptr(), M, K, N, group, ws.data_ptr(),
                                             ws.numel(), None)
    assert rc == -2  # rows closer together than they are long
    # a row longer than the norm prologue holds in registers
    Kbig = 8192 + 128
    _, (qw2, sc2, qz2) = weights(torch, "fused_bad_big", 1, Kbig, 256, 128)
    xb = torch.zeros((1, Kbig), dtype=torch.bfloat16, device="cuda")
    gb = torch.ones((Kbig,), dtype=torch.bfloat16, device="cuda")
    yb = torch.zeros((1, 256), dtype=torch.bfloat16, device="cuda")
    wsb = capi.make_workspace(1, Kbig, 256)
    with pytest.raises(capi.KxError) as e:
        capi.gemv_awq_addnorm_bf16(xb, None, gb, 1e-6, None, qw2, sc2, qz2, yb, 128, wsb)
    assert e.value.code == -2
