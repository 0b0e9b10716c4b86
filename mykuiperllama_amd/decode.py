"""Qwen3-shaped decode step (batch 1) assembled from the C ABI entry points.

Plumbing for the benchmark and for the end-to-end parity test: random-init (or caller-supplied)
INT4 AWQ weights, bf16 KV cache, and the launch sequence of one token.  The reference has no model
code (its model/ directory is absent), so this is not a port of anything; the operator order is
the usual pre-norm decoder with per-head QK-norm:

  x = embed[token]
  per layer:  h = rmsnorm(x);  qkv = Wqkv h;  q,k <- head-norm + rope, k,v -> cache;  a = attn(q);
              x += Wo a;  h = rmsnorm(x);  x += Wdown( silu(Wgate h) * (Wup h) )
  logits = lm_head rmsnorm(x);  next = argmax(logits)

q/k/v share one fused GEMV (N = (n_q + 2 n_kv) * 128) and gate/up another (N = 2 * intermediate): the
packed tensors of the separate projections are concatenated along N when the weights are loaded
(rows are laid end to end; the nibble order inside a word is untouched).  The residual add is fused
into the next RMSNorm, and by default (`fused=True`) both ride in the prologue of the GEMV that
consumes the normalised row, as does SwiGLU in front of the down projection, and the per-head
norm, rotation and cache append ride in the epilogue of the q/k/v GEMV, and the o projection
merges the chunks of the attention itself (contexts up to 5120 positions): five launches per
layer instead of ten.  The residual stream then alternates between two buffers, because a fused
launch reads the whole incoming row in every workgroup while it writes the updated one.
Every launch goes to torch's current stream, so a step can be captured in a HIP graph; token and
position live in device memory for that reason.
"""
from dataclasses import dataclass

from . import capi


@dataclass
class ModelConfig:
    layers: int
    hidden: int
    intermediate: int
    n_q: int
    n_kv: int
    vocab: int
    head_dim: int = 128
    rope_theta: float = 1e6
    eps: float = 1e-6
    group: int = 128

    @property
    def qkv_out(self):
        return (self.n_q + 2 * self.n_kv) * self.head_dim


QWEN3_8B = ModelConfig(layers=36, hidden=4096, intermediate=12288, n_q=32, n_kv=8, vocab=151936)
QWEN3_32B = ModelConfig(layers=64, hidden=5120, intermediate=25600, n_q=64, n_kv=8, vocab=151936)


def _rand_awq(torch, K, N, group, gen):
    qw = torch.randint(-2**31, 2**31 - 1, (K, N // 8), dtype=torch.int32, device="cuda", generator=gen)
    qz = torch.randint(-2**31, 2**31 - 1, (K // group, N // 8), dtype=torch.int32, device="cuda", generator=gen)
    # scales sized so that activations keep O(1) magnitude through the layers: |w| ~ 4.6 s, fan-in K
    s = (torch.rand((K // group, N), device="cuda", generator=gen) * 0.5 + 0.75) * (1.0 / (4.6 * K ** 0.5))
    return qw, s.half(), qz


class DecodeModel:
    """Weights, caches and scratch buffers of one model on the GPU."""

    def __init__(self, cfg, max_positions, weights=None, seed=20251125, merge_in_o=None):
        import torch
        self.torch = torch
        self.cfg = cfg
        self.max_positions = max_positions
        # Where the attention chunks are merged: in the prologue of the o projection (one launch
        # fewer per layer) when the cache is short enough for it.  Every workgroup of that projection
        # repeats the merge of its two heads, so it pays while the projection has about one round of
        # workgroups (Qwen3-8B: 256 of them, 1.5 us per layer faster; Qwen3-32B: 640, 2 us slower
        # than the separate merge kernel).  The caller can decide otherwise.
        fits = max_positions <= capi.FUSED_MERGE_MAX_POSITIONS
        o_workgroups = -(-cfg.hidden // 256) * max(1, cfg.n_q * cfg.head_dim // 256)
        self.merge_in_o = fits and (o_workgroups <= 512 if merge_in_o is None else bool(merge_in_o))
        c = cfg
        gen = torch.Generator(device="cuda")
        gen.manual_seed(seed)
        bf = torch.bfloat16

        def rand_bf16(shape, std):
            return (torch.randn(shape, device="cuda", generator=gen) * std).to(bf)

        if weights is None:
            self.layers = []
            for _ in range(c.layers):
                self.layers.append({
                    "qkv": _rand_awq(torch, c.hidden, c.qkv_out, c.group, gen),
                    "o": _rand_awq(torch, c.n_q * c.head_dim, c.hidden, c.group, gen),
                    "gateup": _rand_awq(torch, c.hidden, 2 * c.intermediate, c.group, gen),
                    "down": _rand_awq(torch, c.intermediate, c.hidden, c.group, gen),
                    "in_norm": 1 + rand_bf16((c.hidden,), 0.02),
                    "post_norm": 1 + rand_bf16((c.hidden,), 0.02),
                    "q_norm": 1 + rand_bf16((c.head_dim,), 0.02),
                    "k_norm": 1 + rand_bf16((c.head_dim,), 0.02),
                })
            self.embed = rand_bf16((c.vocab, c.hidden), 1.0)
            self.lm_head = rand_bf16((c.vocab, c.hidden), 0.02)
            self.final_norm = 1 + rand_bf16((c.hidden,), 0.02)
        else:
            self.layers = weights["layers"]
            self.embed = weights["embed"]
            self.lm_head = weights["lm_head"]
            self.final_norm = weights["final_norm"]

        self.k_cache = [torch.zeros((max_positions, c.n_kv, c.head_dim), dtype=bf, device="cuda") for _ in range(c.layers)]
        self.v_cache = [torch.zeros((max_positions, c.n_kv, c.head_dim), dtype=bf, device="cuda") for _ in range(c.layers)]

        def buf(n):
            return torch.zeros((1, n), dtype=bf, device="cuda")

        self.x = buf(c.hidden)
        self.x2 = buf(c.hidden)
        self.h = buf(c.hidden)
        self.qkv = buf(c.qkv_out)
        self.q = buf(c.n_q * c.head_dim)
        self.attn = buf(c.n_q * c.head_dim)
        self.o = buf(c.hidden)
        self.gu = buf(2 * c.intermediate)
        self.act = buf(c.intermediate)
        self.down = buf(c.hidden)
        self.logits = buf(c.vocab)
        self.ssq = torch.zeros(((c.hidden + 255) // 256, 4), dtype=torch.float32, device="cuda")  # quarter sums per tile
        self.token = torch.zeros(1, dtype=torch.int32, device="cuda")
        self.pos = torch.zeros(1, dtype=torch.int32, device="cuda")
        self.next_token = torch.zeros(1, dtype=torch.int32, device="cuda")
        big_k = max(c.hidden, c.intermediate, c.n_q * c.head_dim)
        big_n = max(c.qkv_out, 2 * c.intermediate, c.hidden)
        self.gemv_ws = capi.make_workspace(1, big_k, big_n)
        self.attn_ws = capi.attn_decode_workspace(c.n_q, max_positions)

    def prefill_cache_random(self, ctx, seed=7):
        """Fill cache rows 0 .. ctx-1 with N(0,1), as the benchmark configurations ask."""
        torch = self.torch
        gen = torch.Generator(device="cuda")
        gen.manual_seed(seed)
        for kc, vc in zip(self.k_cache, self.v_cache):
            kc[:ctx] = torch.randn(kc[:ctx].shape, device="cuda", generator=gen).to(torch.bfloat16)
            vc[:ctx] = torch.randn(vc[:ctx].shape, device="cuda", generator=gen).to(torch.bfloat16)

    def set_input(self, token, pos):
        self.token.fill_(token)
        self.pos.fill_(pos)

    def _awq(self, x, w, y):
        capi.gemv_awq_bf16(x, w[0], w[1], w[2], y, self.cfg.group, self.gemv_ws)

    def step(self, with_lm_head=True, fused=True):
        """Enqueue one decode step on torch's current stream (no synchronisation).

        fused=False       every operator a launch of its own (ten per layer)
        fused="prologue"  the small operators inside the GEMV launches, arithmetic unchanged: bit for bit
                          the result of fused=False when that step's plain GEMVs add their K tiles in the
                          same order (capi.set_awq_kernel_policy(1)); the product's plain GEMV adds them
                          exactly, in fixed point, and agrees to rounding
        fused=True        ("chain") additionally the residual add and the sum of squares of the RMSNorm
                          leave with the epilogue of the producing GEMV, which saves every workgroup of the
                          consuming GEMV a pass over the whole row; the sum is added in another order, so
                          results agree with the other two modes to rounding, not bit for bit
        """
        if fused is True or fused == "chain":
            return self._step_chain(with_lm_head)
        if fused == "prologue":
            return self._step_fused(with_lm_head)
        c = self.cfg
        capi.embedding_bf16(self.embed, self.token, self.x)
        for li, L in enumerate(self.layers):
            if li == 0:
                capi.rmsnorm_bf16(self.x, L["in_norm"], self.h, c.eps)
            else:
                capi.add_rmsnorm_bf16(self.x, self.down, L["in_norm"], self.h, c.eps)
            self._awq(self.h, L["qkv"], self.qkv)
            capi.qk_norm_rope_bf16(self.qkv, L["q_norm"], L["k_norm"], self.q, self.k_cache[li], self.v_cache[li],
                                   c.n_q, c.n_kv, self.pos, c.rope_theta, c.eps)
            capi.attn_decode_bf16(self.q, self.k_cache[li], self.v_cache[li], self.attn, c.n_q, c.n_kv, self.pos,
                                  self.max_positions, self.attn_ws)
            self._awq(self.attn, L["o"], self.o)
            capi.add_rmsnorm_bf16(self.x, self.o, L["post_norm"], self.h, c.eps)
            self._awq(self.h, L["gateup"], self.gu)
            capi.swiglu_bf16(self.gu[:, : c.intermediate], self.gu[:, c.intermediate:], self.act)
            self._awq(self.act, L["down"], self.down)
        capi.add_rmsnorm_bf16(self.x, self.down, self.final_norm, self.h, c.eps)
        if with_lm_head:
            capi.gemv_bf16(self.h, self.lm_head, self.logits)
            capi.argmax_bf16(self.logits, self.next_token)

    def _step_fused(self, with_lm_head):
        c = self.cfg
        g, ws = c.group, self.gemv_ws
        capi.embedding_bf16(self.embed, self.token, self.x)
        xa, xb = self.x, self.x2
        for li, L in enumerate(self.layers):
            qw, sc, qz = L["qkv"]
            capi.gemv_awq_qkv_rope_bf16(xa, None if li == 0 else self.down, L["in_norm"], c.eps, xb, qw, sc, qz,
                                        L["q_norm"], L["k_norm"], self.q, self.k_cache[li], self.v_cache[li],
                                        c.n_q, c.n_kv, self.pos, c.rope_theta, c.eps, g, ws)
            if self.merge_in_o:
                capi.attn_decode_partial_bf16(self.q, self.k_cache[li], self.v_cache[li], c.n_q, c.n_kv, self.pos,
                                              self.max_positions, self.attn_ws)
                qw, sc, qz = L["o"]
                capi.gemv_awq_attn_merge_bf16(self.attn_ws, c.n_q, c.n_kv, self.max_positions, qw, sc, qz, self.o,
                                              g, ws)
            else:
                capi.attn_decode_bf16(self.q, self.k_cache[li], self.v_cache[li], self.attn, c.n_q, c.n_kv,
                                      self.pos, self.max_positions, self.attn_ws)
                self._awq(self.attn, L["o"], self.o)
            qw, sc, qz = L["gateup"]
            capi.gemv_awq_addnorm_bf16(xb, self.o, L["post_norm"], c.eps, xa, qw, sc, qz, self.gu, g, ws)
            qw, sc, qz = L["down"]
            capi.gemv_awq_swiglu_bf16(self.gu[:, : c.intermediate], self.gu[:, c.intermediate:], qw, sc, qz,
                                      self.down, g, ws)
        capi.add_rmsnorm_bf16(xa, self.down, self.final_norm, self.h, c.eps)
        if with_lm_head:
            capi.gemv_bf16(self.h, self.lm_head, self.logits)
            capi.argmax_bf16(self.logits, self.next_token)

    def _step_chain(self, with_lm_head):
        c = self.cfg
        g, ws = c.group, self.gemv_ws
        H, I = c.hidden, c.intermediate
        merge_in_o = self.merge_in_o
        capi.embedding_bf16(self.embed, self.token, self.x)
        x, ssq = self.x, self.ssq
        rope = {"out_kind": capi.OUT_QKV_ROPE, "q_out": self.q, "pos": self.pos, "rope_n_q_heads": c.n_q,
                "rope_n_kv_heads": c.n_kv, "rope_theta": c.rope_theta, "qk_eps": c.eps}
        into_residual = {"out_kind": capi.OUT_RESIDUAL, "residual_in": x, "residual_out": x, "sumsq_out": ssq}
        for li, L in enumerate(self.layers):
            qw, sc, qz = L["qkv"]
            if li == 0:  # the embedding row comes without its sums of squares
                capi.gemv_awq_qkv_rope_bf16(x, None, L["in_norm"], c.eps, None, qw, sc, qz, L["q_norm"], L["k_norm"],
                                            self.q, self.k_cache[li], self.v_cache[li], c.n_q, c.n_kv, self.pos,
                                            c.rope_theta, c.eps, g, ws)
            else:
                capi.gemv_awq_chain_bf16(dict(rope, in_kind=capi.IN_NORM, norm_row=x, norm_sumsq=ssq,
                                              norm_parts=ssq.shape[0], norm_gain=L["in_norm"], norm_eps=c.eps,
                                              q_gain=L["q_norm"], k_gain=L["k_norm"], k_cache=self.k_cache[li],
                                              v_cache=self.v_cache[li]), qw, sc, qz, H, c.qkv_out, g, ws)
            qw, sc, qz = L["o"]
            if merge_in_o:
                capi.attn_decode_partial_bf16(self.q, self.k_cache[li], self.v_cache[li], c.n_q, c.n_kv, self.pos,
                                              self.max_positions, self.attn_ws)
                capi.gemv_awq_chain_bf16(dict(into_residual, in_kind=capi.IN_ATTN, attn_workspace=self.attn_ws,
                                              attn_workspace_bytes=self.attn_ws.numel(), n_q_heads=c.n_q,
                                              n_kv_heads=c.n_kv, max_positions=self.max_positions),
                                         qw, sc, qz, c.n_q * c.head_dim, H, g, ws)
            else:
                capi.attn_decode_bf16(self.q, self.k_cache[li], self.v_cache[li], self.attn, c.n_q, c.n_kv,
                                      self.pos, self.max_positions, self.attn_ws)
                capi.gemv_awq_chain_bf16(dict(into_residual, in_kind=capi.IN_ROW, x=self.attn),
                                         qw, sc, qz, c.n_q * c.head_dim, H, g, ws)
            qw, sc, qz = L["gateup"]
            capi.gemv_awq_chain_bf16({"in_kind": capi.IN_NORM, "norm_row": x, "norm_sumsq": ssq,
                                      "norm_parts": ssq.shape[0], "norm_gain": L["post_norm"], "norm_eps": c.eps,
                                      "out_kind": capi.OUT_ROW, "y": self.gu}, qw, sc, qz, H, 2 * I, g, ws)
            qw, sc, qz = L["down"]
            capi.gemv_awq_chain_bf16(dict(into_residual, in_kind=capi.IN_SWIGLU, gate=self.gu[:, :I],
                                          up=self.gu[:, I:]), qw, sc, qz, I, H, g, ws)
        capi.rmsnorm_bf16(x, self.final_norm, self.h, c.eps)
        if with_lm_head:
            capi.gemv_bf16(self.h, self.lm_head, self.logits)
            capi.argmax_bf16(self.logits, self.next_token)

    def launches_per_step(self, with_lm_head=True, fused=True):
        per_layer = 10
        if fused:
            per_layer = 5 if self.merge_in_o else 6
        return 1 + self.cfg.layers * per_layer + 1 + (2 if with_lm_head else 0)


class BatchDecodeModel:
    """B sequences decoded together, one token each per step: the weights of a DecodeModel, a KV cache per
    sequence ([B, positions, n_kv, 128] per layer) and activations of B rows.  The GEMVs run on the matrix-core
    kernel (2 <= B <= 16 rows), rotation and attention take the sequence as a grid dimension.

    fused=True   six or seven launches per layer: q|k|v with the RMSNorm on the way in (and, for up to four
                 sequences, rotation + cache append on the way out; a launch of its own otherwise), attention
                 (two stages), o with the residual add on the way out, gate|up with the RMSNorm on the way in,
                 down with SwiGLU on the way in and the residual add on the way out
    fused=False  every operator a launch of its own (SwiGLU one per sequence)
    The two agree to the rounding of the RMSNorm's sum of squares (added per 256 columns when fused).
    """

    def __init__(self, single, batch, rope_in_qkv=None):
        torch = single.torch
        if not 2 <= batch <= 16:
            raise ValueError("2 <= batch <= 16")
        # Rotation and cache append ride in the epilogue of the q|k|v GEMV for up to four sequences: the
        # workgroup that finishes a column tile runs the per-head routine for two heads of every row, which
        # takes longer than the launch it saves from eight rows on (measured, tokens/s at 2 / 8 / 16 sequences:
        # 909 / 2243 / 3051 with the epilogue, 886 / 2254 / 3111 with the separate launch).
        self.rope_in_qkv = batch <= 4 if rope_in_qkv is None else bool(rope_in_qkv)
        self.torch = torch
        self.cfg = c = single.cfg
        self.batch = B = batch
        self.max_positions = single.max_positions
        self.layers, self.embed, self.lm_head, self.final_norm = single.layers, single.embed, single.lm_head, single.final_norm
        bf = torch.bfloat16
        self.k_cache = [torch.zeros((B, self.max_positions, c.n_kv, c.head_dim), dtype=bf, device="cuda")
                        for _ in range(c.layers)]
        self.v_cache = [torch.zeros((B, self.max_positions, c.n_kv, c.head_dim), dtype=bf, device="cuda")
                        for _ in range(c.layers)]

        def buf(n):
            return torch.zeros((B, n), dtype=bf, device="cuda")

        self.x = buf(c.hidden)
        self.h = buf(c.hidden)
        self.qkv = buf(c.qkv_out)
        self.q = buf(c.n_q * c.head_dim)
        self.attn = buf(c.n_q * c.head_dim)
        self.o = buf(c.hidden)
        self.gu = buf(2 * c.intermediate)
        self.act = buf(c.intermediate)
        self.down = buf(c.hidden)
        self.logits = buf(c.vocab)
        self.ssq = torch.zeros((B, (c.hidden + 255) // 256, 4), dtype=torch.float32, device="cuda")  # quarter sums per tile
        self.token = torch.zeros(B, dtype=torch.int32, device="cuda")
        self.pos = torch.zeros(B, dtype=torch.int32, device="cuda")
        self.next_token = torch.zeros(B, dtype=torch.int32, device="cuda")
        big_k = max(c.hidden, c.intermediate, c.n_q * c.head_dim)
        big_n = max(c.qkv_out, 2 * c.intermediate, c.hidden)
        self.gemv_ws = capi.make_workspace(B, big_k, big_n)
        self.attn_ws = capi.attn_decode_batch_workspace(B, c.n_q, self.max_positions)

    def prefill_cache_random(self, ctx, seed=7):
        """Rows 0 .. ctx[b]-1 of sequence b's caches get N(0,1); `ctx` is one length or one per sequence."""
        torch = self.torch
        lengths = [ctx] * self.batch if isinstance(ctx, int) else list(ctx)
        gen = torch.Generator(device="cuda")
        gen.manual_seed(seed)
        for kc, vc in zip(self.k_cache, self.v_cache):
            for b, n in enumerate(lengths):
                kc[b, :n] = torch.randn(kc[b, :n].shape, device="cuda", generator=gen).to(torch.bfloat16)
                vc[b, :n] = torch.randn(vc[b, :n].shape, device="cuda", generator=gen).to(torch.bfloat16)

    def set_input(self, tokens, positions):
        torch = self.torch
        self.token.copy_(torch.as_tensor(tokens, dtype=torch.int32))
        self.pos.copy_(torch.as_tensor(positions, dtype=torch.int32))

    def _awq(self, x, w, y):
        capi.gemv_awq_bf16(x, w[0], w[1], w[2], y, self.cfg.group, self.gemv_ws)

    def _attention(self, li, L):
        c = self.cfg
        capi.qk_norm_rope_batch_bf16(self.qkv, L["q_norm"], L["k_norm"], self.q, self.k_cache[li], self.v_cache[li],
                                     c.n_q, c.n_kv, self.pos, c.rope_theta, c.eps)
        capi.attn_decode_batch_bf16(self.q, self.k_cache[li], self.v_cache[li], self.attn, c.n_q, c.n_kv, self.pos,
                                    self.max_positions, self.attn_ws)

    def _head(self, with_lm_head):
        if with_lm_head:
            capi.gemv_bf16(self.h, self.lm_head, self.logits)
            capi.argmax_rows_bf16(self.logits, self.next_token)

    def step(self, with_lm_head=True, fused=True):
        """Enqueue one step for all sequences on torch's current stream (no synchronisation)."""
        c, B = self.cfg, self.batch
        H, I, g, ws = c.hidden, c.intermediate, c.group, self.gemv_ws
        capi.embedding_rows_bf16(self.embed, self.token, self.x)
        if not fused:
            for li, L in enumerate(self.layers):
                if li == 0:
                    capi.rmsnorm_bf16(self.x, L["in_norm"], self.h, c.eps)
                else:
                    capi.add_rmsnorm_bf16(self.x, self.down, L["in_norm"], self.h, c.eps)
                self._awq(self.h, L["qkv"], self.qkv)
                self._attention(li, L)
                self._awq(self.attn, L["o"], self.o)
                capi.add_rmsnorm_bf16(self.x, self.o, L["post_norm"], self.h, c.eps)
                self._awq(self.h, L["gateup"], self.gu)
                for b in range(B):  # gate and up of a row are the two halves of one gate|up output row
                    capi.swiglu_bf16(self.gu[b, :I], self.gu[b, I:], self.act[b])
                self._awq(self.act, L["down"], self.down)
            capi.add_rmsnorm_bf16(self.x, self.down, self.final_norm, self.h, c.eps)
            return self._head(with_lm_head)

        x, ssq = self.x, self.ssq
        parts = ssq.shape[1]
        into_residual = {"out_kind": capi.OUT_RESIDUAL, "residual_in": x, "residual_out": x, "sumsq_out": ssq, "rows": B}
        for li, L in enumerate(self.layers):
            qw, sc, qz = L["qkv"]
            if self.rope_in_qkv:
                out = {"out_kind": capi.OUT_QKV_ROPE, "q_out": self.q, "pos": self.pos, "rope_n_q_heads": c.n_q,
                       "rope_n_kv_heads": c.n_kv, "rope_theta": c.rope_theta, "qk_eps": c.eps, "q_gain": L["q_norm"],
                       "k_gain": L["k_norm"], "k_cache": self.k_cache[li], "v_cache": self.v_cache[li],
                       "cache_positions": self.max_positions, "cache_stride": self.k_cache[li].stride(0), "rows": B}
            else:
                out = {"out_kind": capi.OUT_ROW, "y": self.qkv, "rows": B}
            if li == 0:  # the embedding rows come without their sums of squares
                capi.rmsnorm_bf16(x, L["in_norm"], self.h, c.eps)
                capi.gemv_awq_chain_bf16(dict(out, in_kind=capi.IN_ROW, x=self.h), qw, sc, qz, H, c.qkv_out, g, ws)
            else:
                capi.gemv_awq_chain_bf16(dict(out, in_kind=capi.IN_NORM, norm_row=x, norm_sumsq=ssq, norm_parts=parts,
                                              norm_gain=L["in_norm"], norm_eps=c.eps), qw, sc, qz, H, c.qkv_out, g, ws)
            if not self.rope_in_qkv:
                capi.qk_norm_rope_batch_bf16(self.qkv, L["q_norm"], L["k_norm"], self.q, self.k_cache[li],
                                             self.v_cache[li], c.n_q, c.n_kv, self.pos, c.rope_theta, c.eps)
            capi.attn_decode_batch_bf16(self.q, self.k_cache[li], self.v_cache[li], self.attn, c.n_q, c.n_kv, self.pos,
                                        self.max_positions, self.attn_ws)
            qw, sc, qz = L["o"]
            capi.gemv_awq_chain_bf16(dict(into_residual, in_kind=capi.IN_ROW, x=self.attn),
                                     qw, sc, qz, c.n_q * c.head_dim, H, g, ws)
            qw, sc, qz = L["gateup"]
            capi.gemv_awq_chain_bf16({"in_kind": capi.IN_NORM, "norm_row": x, "norm_sumsq": ssq, "norm_parts": parts,
                                      "norm_gain": L["post_norm"], "norm_eps": c.eps, "out_kind": capi.OUT_ROW,
                                      "y": self.gu, "rows": B}, qw, sc, qz, H, 2 * I, g, ws)
            qw, sc, qz = L["down"]
            capi.gemv_awq_chain_bf16(dict(into_residual, in_kind=capi.IN_SWIGLU, gate=self.gu[:, :I], up=self.gu[:, I:],
                                          act_ld=2 * I), qw, sc, qz, I, H, g, ws)
        capi.rmsnorm_bf16(x, self.final_norm, self.h, c.eps)
        return self._head(with_lm_head)

    def launches_per_step(self, with_lm_head=True, fused=True):
        per_layer = (6 if self.rope_in_qkv else 7) if fused else 10 + self.batch
        return 1 + self.cfg.layers * per_layer + (1 if fused else 0) + 1 + (2 if with_lm_head else 0)


def step_bytes(cfg, ctx, with_lm_head=True):
    """Algorithmic HBM bytes of one decode step: packed projections + KV read (+ bf16 lm_head)."""
    from .synth import awq_gemv_bytes
    per_layer = (awq_gemv_bytes(1, cfg.hidden, cfg.n_q * cfg.head_dim, cfg.group)
                 + 2 * awq_gemv_bytes(1, cfg.hidden, cfg.n_kv * cfg.head_dim, cfg.group)
                 + awq_gemv_bytes(1, cfg.n_q * cfg.head_dim, cfg.hidden, cfg.group)
                 + 2 * awq_gemv_bytes(1, cfg.hidden, cfg.intermediate, cfg.group)
                 + awq_gemv_bytes(1, cfg.intermediate, cfg.hidden, cfg.group))
    kv = 2 * ctx * cfg.n_kv * cfg.head_dim * 2
    total = cfg.layers * (per_layer + kv)
    if with_lm_head:
        total += cfg.vocab * cfg.hidden * 2
    return total
