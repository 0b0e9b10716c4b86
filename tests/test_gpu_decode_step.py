"""End-to-end parity of the decode step on a small Qwen3-shaped model.

The model under test takes fused QKV and gate+up tensors; the reference below keeps the five
projections separate, dequantises them with the CPU oracle and evaluates the layer formulas in fp32
with torch on the CPU, rounding to bf16 where the GPU path stores bf16.  Accumulation order differs,
so single-ulp flips propagate through the layers: logits are compared at 2e-2 relative L2, the
greedy token must agree whenever the reference's top-2 margin is clear.
"""
import math

import numpy as np
import pytest

from mykuiperllama_amd import synth
from tests import helpers as H

pytestmark = pytest.mark.gpu

CFG = dict(layers=2, hidden=512, intermediate=1024, n_q=4, n_kv=2, vocab=1024)
CTX = 37
MAXPOS = 48


@pytest.fixture(scope="module")
def torch():
    import torch as _t
    assert _t.cuda.is_available()
    return _t


def make_weights(torch, oracle, cfg):
    """Seeded weights: packed numpy tensors per projection, their fp32 dequantisation, bf16 extras."""
    D = 128
    rng_names = ["q", "k", "v", "o", "gate", "up", "down"]
    shapes = {"q": (cfg.hidden, cfg.n_q * D), "k": (cfg.hidden, cfg.n_kv * D), "v": (cfg.hidden, cfg.n_kv * D),
              "o": (cfg.n_q * D, cfg.hidden), "gate": (cfg.hidden, cfg.intermediate),
              "up": (cfg.hidden, cfg.intermediate), "down": (cfg.intermediate, cfg.hidden)}
    layers_np, layers_ref = [], []
    g = torch.Generator().manual_seed(99)
    for li in range(cfg.layers):
        packed, deq = {}, {}
        for name in rng_names:
            K, N = shapes[name]
            p = synth.make_awq_problem(f"e2e_l{li}_{name}", 1, K, N)
            # rescale so that activations stay O(1): scales ~ 1 / (4.6 sqrt(K))
            s = synth.f16_bits_to_f32(p["scales"]) / 0.0105 / (4.6 * math.sqrt(K))
            p["scales"] = synth.f32_to_f16_bits(s.astype(np.float32))
            packed[name] = p
            w = oracle.awq_dequant_bf16(p["qweight"], p["scales"], p["qzeros"], 128)
            # the GEMV uses the unrounded product (q - z) * s; rebuild it exactly in fp32
            codes = oracle.awq_unpack(p["qweight"]).astype(np.float32)
            zeros = np.repeat(oracle.awq_unpack(p["qzeros"]).astype(np.float32), 128, axis=0)
            sc = np.repeat(synth.f16_bits_to_f32(p["scales"]), 128, axis=0)
            deq[name] = torch.from_numpy((codes - zeros) * sc)
            del w
        norms = {k: (1 + 0.05 * torch.randn(n, generator=g)).bfloat16()
                 for k, n in (("in_norm", cfg.hidden), ("post_norm", cfg.hidden), ("q_norm", D), ("k_norm", D))}
        layers_np.append((packed, norms))
        layers_ref.append((deq, norms))
    embed = torch.randn(cfg.vocab, cfg.hidden, generator=g).bfloat16()
    lm_head = (0.05 * torch.randn(cfg.vocab, cfg.hidden, generator=g)).bfloat16()
    final_norm = (1 + 0.05 * torch.randn(cfg.hidden, generator=g)).bfloat16()
    return layers_np, layers_ref, embed, lm_head, final_norm


def to_model_weights(torch, layers_np, embed, lm_head, final_norm):
    def fuse(parts):
        qw = np.concatenate([p["qweight"] for p in parts], axis=1)
        sc = np.concatenate([p["scales"] for p in parts], axis=1)
        qz = np.concatenate([p["qzeros"] for p in parts], axis=1)
        return (H.to_dev_i32(qw, torch), H.to_dev_f16(sc, torch), H.to_dev_i32(qz, torch))

    layers = []
    for packed, norms in layers_np:
        L = {"qkv": fuse([packed["q"], packed["k"], packed["v"]]), "o": fuse([packed["o"]]),
             "gateup": fuse([packed["gate"], packed["up"]]), "down": fuse([packed["down"]])}
        L.update({k: v.cuda() for k, v in norms.items()})
        layers.append(L)
    return {"layers": layers, "embed": embed.cuda(), "lm_head": lm_head.cuda(), "final_norm": final_norm.cuda()}


class Reference:
    def __init__(self, torch, cfg, layers_ref, embed, lm_head, final_norm, k0, v0):
        self.t, self.cfg, self.layers = torch, cfg, layers_ref
        self.embed, self.lm_head, self.final_norm = embed, lm_head, final_norm
        self.k = [k.clone() for k in k0]
        self.v = [v.clone() for v in v0]

    def norm(self, x, gain):
        t = self.t
        xf = x.float()
        return gain * (xf * t.rsqrt(xf.pow(2).mean(-1, keepdim=True) + self.cfg.eps)).to(t.bfloat16)

    def lin(self, x, w):
        return (x.float() @ w).to(self.t.bfloat16)

    def step(self, token, pos):
        t, c, D = self.t, self.cfg, 128
        G = c.n_q // c.n_kv
        x = self.embed[token].clone()
        inv_freq = 1.0 / (c.rope_theta ** (t.arange(0, D, 2, dtype=t.float32) / D))
        ang = pos * inv_freq
        cos, sin = t.cat([ang, ang]).cos(), t.cat([ang, ang]).sin()

        def rope(v):
            return v * cos + t.cat([-v[..., D // 2:], v[..., : D // 2]], dim=-1) * sin

        for li, (w, n) in enumerate(self.layers):
            h = self.norm(x, n["in_norm"])
            q = self.norm(self.lin(h, w["q"]).view(c.n_q, D), n["q_norm"]).float()
            k = self.norm(self.lin(h, w["k"]).view(c.n_kv, D), n["k_norm"]).float()
            v = self.lin(h, w["v"]).view(c.n_kv, D)
            q = rope(q).to(t.bfloat16)
            self.k[li][pos] = rope(k).to(t.bfloat16)
            self.v[li][pos] = v
            kf = self.k[li][: pos + 1].float().repeat_interleave(G, dim=1)
            vf = self.v[li][: pos + 1].float().repeat_interleave(G, dim=1)
            sc = t.einsum("hd,phd->hp", q.float(), kf) / math.sqrt(D)
            a = t.einsum("hp,phd->hd", t.softmax(sc, dim=-1), vf).to(t.bfloat16).reshape(-1)
            x = x + self.lin(a, w["o"])
            h = self.norm(x, n["post_norm"])
            act = t.nn.functional.silu(self.lin(h, w["gate"]).float()).to(t.bfloat16) * self.lin(h, w["up"])
            x = x + self.lin(act, w["down"])
        logits = self.lin(self.norm(x, self.final_norm), self.lm_head.float().T)
        return x, logits


@pytest.mark.parametrize("fused", [True, "prologue", False])
def test_decode_steps_match_the_fp32_reference(torch, oracle, fused):
    from mykuiperllama_amd import decode
    cfg = decode.ModelConfig(**CFG)
    layers_np, layers_ref, embed, lm_head, final_norm = make_weights(torch, oracle, cfg)
    model = decode.DecodeModel(cfg, MAXPOS, weights=to_model_weights(torch, layers_np, embed, lm_head, final_norm))
    model.prefill_cache_random(CTX)
    ref = Reference(torch, cfg, layers_ref, embed, lm_head, final_norm,
                    [k.cpu() for k in model.k_cache], [v.cpu() for v in model.v_cache])
    token = 17
    agreed = 0
    for stepno in range(4):
        pos = CTX + stepno
        model.set_input(token, pos)
        model.step(fused=fused)
        torch.cuda.synchronize()
        x_ref, logits_ref = ref.step(token, pos)
        got_logits = model.logits[0].cpu().float()
        assert torch.isfinite(got_logits).all()
        err = (got_logits - logits_ref.float()).norm() / logits_ref.float().norm()
        assert err <= 2e-2, f"step {stepno}: logits relative L2 {err}"
        xerr = (model.x[0].cpu().float() - x_ref.float()).norm() / x_ref.float().norm()
        assert xerr <= 2e-2
        for li in range(cfg.layers):
            kerr = (model.k_cache[li][pos].cpu().float() - ref.k[li][pos].float()).abs().max()
            assert kerr <= 0.06  # rotated, normalised keys are O(1): a few bf16 ulps
        top2 = logits_ref.float().topk(2).values
        ref_token = int(logits_ref.float().argmax())
        if (top2[0] - top2[1]) > 0.05 * top2[0].abs():
            assert int(model.next_token.item()) == ref_token
            agreed += 1
        token = ref_token
    assert agreed >= 1


# a second head layout: five query heads per KV head (Qwen3-14B's grouping), ten heads of 128 on hidden 512
CFG_G5 = dict(CFG, n_q=10, n_kv=2)


@pytest.mark.parametrize("fused,max_pos,shape", [(True, MAXPOS, CFG), ("prologue", MAXPOS, CFG), (False, MAXPOS, CFG),
                                                 (True, 6000, CFG), (True, 10368, CFG),  # chunks of 128; separate merge
                                                 (True, MAXPOS, CFG_G5), (False, MAXPOS, CFG_G5)])
def test_decode_from_an_empty_cache_matches_the_transformers_qwen3_model(torch, oracle, fused, max_pos, shape):
    """An independent implementation of the architecture: the installed `transformers` Qwen3 model (eager
    attention, fp32, on the CPU) is given the dequantised weights and run over a token sequence in one pass;
    the decode step here is fed the same tokens one by one from an empty KV cache.  This pins what the
    in-file fp32 restatement could share a misreading with: where the norms sit, the rotate-half convention
    and its frequencies, which query heads go with which KV head, the residual wiring and SwiGLU."""
    from transformers import Qwen3Config, Qwen3ForCausalLM
    from mykuiperllama_amd import decode
    cfg = decode.ModelConfig(**shape)
    layers_np, layers_ref, embed, lm_head, final_norm = make_weights(torch, oracle, cfg)
    hf_cfg = Qwen3Config(vocab_size=cfg.vocab, hidden_size=cfg.hidden, intermediate_size=cfg.intermediate,
                         num_hidden_layers=cfg.layers, num_attention_heads=cfg.n_q, num_key_value_heads=cfg.n_kv,
                         head_dim=128, rms_norm_eps=cfg.eps, rope_theta=cfg.rope_theta, tie_word_embeddings=False,
                         attention_bias=False, max_position_embeddings=MAXPOS, attn_implementation="eager")
    hf = Qwen3ForCausalLM(hf_cfg).eval().float()
    sd = {"model.embed_tokens.weight": embed.float(), "model.norm.weight": final_norm.float(),
          "lm_head.weight": lm_head.float()}
    for li, (w, n) in enumerate(layers_ref):
        pre = f"model.layers.{li}."
        for name in ("q", "k", "v", "o"):
            sd[pre + f"self_attn.{name}_proj.weight"] = w[name].T.contiguous()  # Linear keeps [out, in]
        for name in ("gate", "up", "down"):
            sd[pre + f"mlp.{name}_proj.weight"] = w[name].T.contiguous()
        sd[pre + "self_attn.q_norm.weight"] = n["q_norm"].float()
        sd[pre + "self_attn.k_norm.weight"] = n["k_norm"].float()
        sd[pre + "input_layernorm.weight"] = n["in_norm"].float()
        sd[pre + "post_attention_layernorm.weight"] = n["post_norm"].float()
    missing, unexpected = hf.load_state_dict(sd, strict=False)
    assert not unexpected and all("rotary" in m or "inv_freq" in m for m in missing), (missing, unexpected)

    tokens = [17, 3, 900, 41, 512, 7, 1023, 64, 5, 250, 77, 12]
    with torch.no_grad():
        hf_logits = hf(torch.tensor([tokens])).logits[0]  # [len, vocab], causal: row p sees tokens 0..p

    model = decode.DecodeModel(cfg, max_pos, weights=to_model_weights(torch, layers_np, embed, lm_head, final_norm))
    agreed = 0
    for pos, token in enumerate(tokens):
        model.set_input(token, pos)
        model.step(fused=fused)
        torch.cuda.synchronize()
        got = model.logits[0].cpu().float()
        ref = hf_logits[pos]
        assert torch.isfinite(got).all()
        # the GPU path stores bf16 after every operator, the library computes in fp32 throughout
        err = ((got - ref).norm() / ref.norm()).item()
        assert err <= 3e-2, f"position {pos}: logits relative L2 {err}"
        top2 = ref.topk(2).values
        if (top2[0] - top2[1]) > 0.05 * top2[0].abs():
            assert int(model.next_token.item()) == int(ref.argmax())
            agreed += 1
    assert agreed >= 3


def test_fused_and_separate_launches_give_the_same_step(torch):
    """SwiGLU and add+RMSNorm in the GEMV prologue change nothing, bit for bit."""
    from mykuiperllama_amd import decode
    cfg = decode.ModelConfig(**CFG)
    model = decode.DecodeModel(cfg, MAXPOS)
    model.prefill_cache_random(CTX)
    results = []
    for fused in (False, "prologue"):
        model.set_input(9, CTX)
        model.step(fused=fused)
        torch.cuda.synchronize()
        results.append((model.logits.clone(), model.x.clone(), model.k_cache[-1][CTX].clone()))
    for a, b in zip(*results):
        assert torch.equal(a.view(torch.int16), b.view(torch.int16))


def test_chained_step_agrees_with_the_prologue_step_to_rounding(torch):
    """The chained launches add the RMSNorm's sum of squares tile by tile: same step up to that rounding."""
    from mykuiperllama_amd import decode
    cfg = decode.ModelConfig(**CFG)
    model = decode.DecodeModel(cfg, MAXPOS)
    model.prefill_cache_random(CTX)
    results = []
    for fused in ("prologue", "chain"):
        model.set_input(9, CTX)
        model.step(fused=fused)
        torch.cuda.synchronize()
        results.append((model.logits.float().clone(), model.x.float().clone(), model.k_cache[-1][CTX].float().clone()))
    (la, xa, ka), (lb, xb, kb) = results
    assert torch.isfinite(lb).all()
    assert ((la - lb).norm() / la.norm()).item() <= 5e-3
    assert ((xa - xb).norm() / xa.norm()).item() <= 5e-3
    assert (ka - kb).abs().max().item() <= 0.05


@pytest.mark.parametrize("max_pos,ctx", [(48, 37), (6000, 5500), (10240, 10239), (10368, 7000)])
def test_merge_inside_the_o_projection_or_as_a_launch_of_its_own_is_the_same_step(torch, max_pos, ctx):
    """Where the attention chunks are merged changes nothing, bit for bit; caches past 5120 positions are
    walked in chunks of 128, past 10240 the merge is always a launch of its own."""
    from mykuiperllama_amd import decode
    cfg = decode.ModelConfig(**CFG)
    results = []
    for merge_in_o in (True, False):
        model = decode.DecodeModel(cfg, max_pos, merge_in_o=merge_in_o)
        assert model.merge_in_o == (merge_in_o and max_pos <= 10240)
        model.prefill_cache_random(ctx)
        model.set_input(9, ctx)
        model.step(fused="chain")
        torch.cuda.synchronize()
        assert torch.isfinite(model.logits.float()).all()
        results.append((model.logits.clone(), model.x.clone()))
        assert model.launches_per_step(True) == 4 + cfg.layers * (5 if model.merge_in_o else 6)
    for a, b in zip(*results):
        assert torch.equal(a.view(torch.int16), b.view(torch.int16))


@pytest.mark.parametrize("fused", [True, "prologue", False])
def test_step_is_capturable_in_a_graph_and_replays_identically(torch, fused):
    """A captured step replayed with the same inputs gives bitwise the same logits as eager."""
    from mykuiperllama_amd import decode
    cfg = decode.ModelConfig(**CFG)
    model = decode.DecodeModel(cfg, MAXPOS)
    model.prefill_cache_random(CTX)
    model.set_input(5, CTX)
    model.step(fused=fused)
    torch.cuda.synchronize()
    eager = model.logits.clone()
    side = torch.cuda.Stream()
    with torch.cuda.stream(side):
        g = torch.cuda.CUDAGraph()
        with torch.cuda.graph(g):
            model.step(fused=fused)
        for _ in range(3):
            model.logits.zero_()
            torch.cuda.synchronize()
            g.replay()
            side.synchronize()
            assert torch.equal(model.logits, eager)
    torch.cuda.synchronize()
