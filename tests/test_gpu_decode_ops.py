"""GPU parity of the decode-step supporting kernels against fp32 torch references on the CPU.

These are floating-point kernels with bf16 storage, so the reference is the closed form evaluated
in fp32 by torch and rounded where the kernel rounds; tolerances are stated per test.  The
conventions that a closed form cannot pin by itself (rotate-half pairing, norm before rotation,
rounding points of RMSNorm) are checked against the Qwen3 modelling code that ships with the
installed transformers package (a library oracle; nothing is downloaded).
"""
import math

import numpy as np
import pytest

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def torch():
    import torch as _t
    assert _t.cuda.is_available()
    _t.manual_seed(1234)
    return _t


@pytest.fixture(scope="module")
def capi():
    from mykuiperllama_amd import capi as _c
    _c.load()
    return _c


def ulp_diff(torch, a, b):
    """Distance in bf16 units-in-the-last-place between two bf16 tensors (same sign region)."""
    ia = a.view(torch.int16).to(torch.int32)
    ib = b.view(torch.int16).to(torch.int32)
    return (ia - ib).abs()


def ref_rmsnorm(torch, x, gain, eps):
    xf = x.float()
    normed = (xf * torch.rsqrt(xf.pow(2).mean(-1, keepdim=True) + eps)).to(torch.bfloat16)
    return gain * normed  # bf16 * bf16 -> bf16, the rounding points of Qwen3RMSNorm


@pytest.mark.parametrize("rows,n", [(1, 4096), (1, 5120), (3, 1024), (2, 128), (1, 8)])
def test_rmsnorm_matches_reference_and_transformers(capi, torch, rows, n):
    eps = 1e-6
    x = (torch.randn(rows, n) * 3).bfloat16()
    gain = (1 + 0.1 * torch.randn(n)).bfloat16()
    y = torch.empty(rows, n, dtype=torch.bfloat16, device="cuda")
    capi.rmsnorm_bf16(x.cuda(), gain.cuda(), y, eps)
    torch.cuda.synchronize()
    ref = ref_rmsnorm(torch, x, gain, eps)
    d = ulp_diff(torch, y.cpu(), ref)
    assert d.max() <= 1 and (d == 0).float().mean() > 0.99  # rsqrt vs 1/sqrt may flip a rounding
    from transformers.models.qwen3.modeling_qwen3 import Qwen3RMSNorm
    mod = Qwen3RMSNorm(n, eps=eps).to(torch.bfloat16)
    with torch.no_grad():
        mod.weight.copy_(gain)
        hf = mod(x)
    assert ulp_diff(torch, y.cpu(), hf).max() <= 1


def test_add_rmsnorm_updates_the_residual_in_place(capi, torch):
    n, eps = 4096, 1e-6
    x = torch.randn(1, n).bfloat16()
    delta = torch.randn(1, n).bfloat16()
    gain = (1 + 0.1 * torch.randn(n)).bfloat16()
    xd = x.cuda().clone()
    y = torch.empty(1, n, dtype=torch.bfloat16, device="cuda")
    capi.add_rmsnorm_bf16(xd, delta.cuda(), gain.cuda(), y, eps)
    torch.cuda.synchronize()
    x_new = x + delta  # bf16 addition rounds once, like the kernel
    assert torch.equal(xd.cpu(), x_new)
    assert ulp_diff(torch, y.cpu(), ref_rmsnorm(torch, x_new, gain, eps)).max() <= 1


@pytest.mark.parametrize("n_q,n_kv,pos", [(32, 8, 0), (32, 8, 4096), (64, 8, 8191), (4, 2, 17), (2, 2, 1)])
def test_qk_norm_rope_and_cache_append(capi, torch, n_q, n_kv, pos):
    theta, eps, D = 1e6, 1e-6, 128
    max_pos = pos + 3
    qkv = torch.randn((n_q + 2 * n_kv) * D).bfloat16()
    qg = (1 + 0.1 * torch.randn(D)).bfloat16()
    kg = (1 + 0.1 * torch.randn(D)).bfloat16()
    q_out = torch.zeros(n_q, D, dtype=torch.bfloat16, device="cuda")
    kc = torch.zeros(max_pos, n_kv, D, dtype=torch.bfloat16, device="cuda")
    vc = torch.zeros(max_pos, n_kv, D, dtype=torch.bfloat16, device="cuda")
    pos_t = torch.tensor([pos], dtype=torch.int32, device="cuda")
    capi.qk_norm_rope_bf16(qkv.cuda(), qg.cuda(), kg.cuda(), q_out, kc, vc, n_q, n_kv, pos_t, theta, eps)
    torch.cuda.synchronize()

    q = qkv[: n_q * D].view(n_q, D)
    k = qkv[n_q * D:(n_q + n_kv) * D].view(n_kv, D)
    v = qkv[(n_q + n_kv) * D:].view(n_kv, D)
    qn = ref_rmsnorm(torch, q, qg, eps).float()
    kn = ref_rmsnorm(torch, k, kg, eps).float()
    inv_freq = 1.0 / (theta ** (torch.arange(0, D, 2, dtype=torch.float32) / D))
    ang = pos * inv_freq
    cos = torch.cat([ang, ang]).cos()
    sin = torch.cat([ang, ang]).sin()

    def rot(t):
        return torch.cat([-t[..., D // 2:], t[..., : D // 2]], dim=-1)

    q_ref = qn * cos + rot(qn) * sin
    k_ref = kn * cos + rot(kn) * sin
    # fp32 reference, one bf16 rounding at the end: within one ulp of the output scale
    scale_q = q_ref.abs().max().item()
    assert (q_out.cpu().float() - q_ref).abs().max() <= 2.0 ** (math.floor(math.log2(scale_q)) - 7)
    assert (kc[pos].cpu().float() - k_ref).abs().max() <= 2.0 ** (math.floor(math.log2(k_ref.abs().max().item())) - 7)
    assert torch.equal(vc[pos].cpu(), v)
    other = [p for p in range(max_pos) if p != pos]
    assert not kc[other].any() and not vc[other].any()  # only row `pos` is written

    # convention check against the library: bf16 cos/sin there, so a looser bound
    from transformers.models.qwen3.modeling_qwen3 import apply_rotary_pos_emb
    qh, kh = apply_rotary_pos_emb(qn.bfloat16()[None, :, None, :], kn.bfloat16()[None, :, None, :],
                                  cos.bfloat16()[None, None, :], sin.bfloat16()[None, None, :])
    assert (q_out.cpu().float() - qh[0, :, 0].float()).abs().max() <= 0.03 * max(scale_q, 1.0)
    assert (kc[pos].cpu().float() - kh[0, :, 0].float()).abs().max() <= 0.03 * max(k_ref.abs().max().item(), 1.0)


@pytest.mark.parametrize("pos", [4, 5, 1 << 20, -1, -(1 << 31)])
def test_cache_append_skips_positions_outside_the_cache(capi, torch, pos):
    """A position the caches have no row for writes nothing into them (memory on either side of the
    caches keeps its contents); the query heads are still produced."""
    n_q, n_kv, D, rows = 4, 2, 128, 4
    qkv = torch.randn((n_q + 2 * n_kv) * D).bfloat16().cuda()
    g = torch.ones(D, dtype=torch.bfloat16, device="cuda")
    q_out = torch.full((n_q, D), float("nan"), dtype=torch.bfloat16, device="cuda")
    # the caches sit in the middle of a larger buffer: rows before and after them must stay as they are
    pool = torch.full((2, rows + 4, n_kv, D), 7.0, dtype=torch.bfloat16, device="cuda")
    kc, vc = pool[0, 2:2 + rows], pool[1, 2:2 + rows]
    capi.qk_norm_rope_bf16(qkv, g, g, q_out, kc, vc, n_q, n_kv,
                           torch.tensor([pos], dtype=torch.int32, device="cuda"), 1e6, 1e-6)
    torch.cuda.synchronize()
    assert (pool == 7.0).all()
    assert torch.isfinite(q_out.float()).all()


@pytest.mark.parametrize("n_q,n_kv", [(32, 8), (64, 8), (8, 4), (4, 4), (40, 8), (12, 4), (16, 1)])
@pytest.mark.parametrize("ctx,max_pos", [(1, 4224), (5, 4224), (128, 4224), (129, 4224), (1000, 4224), (4097, 4224),
                                         # caches past 5120 positions are walked in chunks of 128
                                         (1, 5121), (127, 8320), (128, 8320), (129, 8320), (8193, 8320),
                                         (12000, 12032)])
def test_attention_decode_matches_fp32_softmax(capi, torch, n_q, n_kv, ctx, max_pos):
    D = 128
    G = n_q // n_kv
    q = torch.randn(n_q, D).bfloat16()
    kc = torch.randn(max_pos, n_kv, D).bfloat16()
    vc = torch.randn(max_pos, n_kv, D).bfloat16()
    out = torch.full((n_q, D), float("nan"), dtype=torch.bfloat16, device="cuda")
    pos_t = torch.tensor([ctx - 1], dtype=torch.int32, device="cuda")
    ws = capi.attn_decode_workspace(n_q, max_pos)
    capi.attn_decode_bf16(q.cuda(), kc.cuda(), vc.cuda(), out, n_q, n_kv, pos_t, max_pos, ws)
    torch.cuda.synchronize()
    kf = kc[:ctx].float().repeat_interleave(G, dim=1)  # [ctx, n_q, D]
    vf = vc[:ctx].float().repeat_interleave(G, dim=1)
    scores = torch.einsum("hd,phd->hp", q.float(), kf) / math.sqrt(D)
    ref = torch.einsum("hp,phd->hd", torch.softmax(scores, dim=-1), vf)
    got = out.cpu().float()
    assert torch.isfinite(got).all()
    err = (got - ref).norm() / ref.norm()
    assert err <= 3e-3  # the bf16 store alone is ~1.6e-3
    assert (got - ref).abs().max() <= 2 * 2.0 ** (math.floor(math.log2(ref.abs().max().item())) - 7)


def test_swiglu_add_embedding_argmax(capi, torch):
    n = 12288
    g = (torch.randn(n) * 2).bfloat16()
    u = torch.randn(n).bfloat16()
    out = torch.empty(n, dtype=torch.bfloat16, device="cuda")
    capi.swiglu_bf16(g.cuda(), u.cuda(), out)
    torch.cuda.synchronize()
    ref = torch.nn.functional.silu(g.float()).bfloat16() * u
    d = ulp_diff(torch, out.cpu(), ref)
    assert d.max() <= 1 and (d == 0).float().mean() > 0.98  # expf vs torch's exp may flip a rounding

    a = torch.randn(4096).bfloat16()
    b = torch.randn(4096).bfloat16()
    capi.add_bf16(a.cuda(), b.cuda(), out[:4096])
    torch.cuda.synchronize()
    assert torch.equal(out[:4096].cpu(), a + b)

    table = torch.randn(1000, 512).bfloat16().cuda()
    row = torch.empty(512, dtype=torch.bfloat16, device="cuda")
    for tok in (0, 7, 999, 5000, -3):  # out-of-range tokens clamp
        capi.embedding_bf16(table, torch.tensor([tok], dtype=torch.int32, device="cuda"), row)
        torch.cuda.synchronize()
        assert torch.equal(row, table[min(max(tok, 0), 999)])

    logits = torch.randn(151936).bfloat16()
    logits[77777] = 50.0
    idx = torch.zeros(1, dtype=torch.int32, device="cuda")
    capi.argmax_bf16(logits.cuda(), idx)
    torch.cuda.synchronize()
    assert idx.item() == 77777
    logits[123] = 50.0  # a tie: the first index wins
    capi.argmax_bf16(logits.cuda(), idx)
    torch.cuda.synchronize()
    assert idx.item() == 123
    logits[5] = float("nan")  # NaN is ignored
    capi.argmax_bf16(logits.cuda(), idx)
    torch.cuda.synchronize()
    assert idx.item() == 123
    for fill, want in ((float("nan"), 0), (float("-inf"), 0), (-0.0, 0)):
        flat = torch.full((4099,), fill).bfloat16()
        capi.argmax_bf16(flat.cuda(), idx)
        torch.cuda.synchronize()
        assert idx.item() == want
    flat = torch.full((4099,), -1.0).bfloat16()
    flat[4000], flat[4098] = -0.0, 0.0  # the two zeros are one value: the first of them wins
    capi.argmax_bf16(flat.cuda(), idx)
    torch.cuda.synchronize()
    assert idx.item() == 4000
    # ragged lengths (shorter than one 16-byte piece, not a multiple of eight, the maximum in the
    # last element) and a pointer off the 16-byte grid
    g = torch.Generator().manual_seed(5)
    for n in (1, 7, 8, 9, 1000, 8193, 65537):
        for shift in (0, 1):
            buf = torch.randn(n + shift, generator=g).bfloat16()
            view = buf[shift:]
            for where in (n - 1, n // 2, 0):
                vals = view.clone()
                vals[where] = 60.0
                dev = torch.empty(n + shift, dtype=torch.bfloat16, device="cuda")
                dev[shift:] = vals.cuda()
                capi.argmax_bf16(dev[shift:], idx)
                torch.cuda.synchronize()
                assert idx.item() == where, (n, shift, where)
