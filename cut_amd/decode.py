"""One decode step of a Llama-style dense transformer on GGUF weights: the
chain the reference's runner encodes per token (interface/runner/llama/
llama.cpp, runLayer: RMSNorm -> q/k/v matmuls -> RoPE + KV write ->
attention -> wo + residual -> RMSNorm -> fused gate+up -> SiLU * up ->
w_down + residual; then the output norm, the head matmul and arg-max).

Every launch goes through the C ABI on the current stream and allocates
nothing, so `step()` can be captured once into a HIP graph and replayed:
the position and sequence length live in a device buffer, as the reference's
runtimeParams do.  The residual stream is fp32; matmul inputs are fp16.
"""
from __future__ import annotations

import dataclasses
import math

import torch

from . import ops


@dataclasses.dataclass
class DecodeConfig:
    hidden: int = 4096
    n_layers: int = 32
    n_heads: int = 32
    n_kv_heads: int = 8
    head_dim: int = 128
    ffn: int = 14336
    vocab: int = 128256
    max_ctx: int = 2048
    rope_theta: float = 500000.0
    eps: float = 1e-5
    fmt_attn: str = "Q4_K"
    fmt_v: str = "Q6_K"
    fmt_ffn: str = "Q4_K"
    fmt_head: str = "Q6_K"
    fmt_embd: str = "Q4_K"

    @property
    def q_dim(self) -> int:
        return self.n_heads * self.head_dim

    @property
    def kv_dim(self) -> int:
        return self.n_kv_heads * self.head_dim


def interleave_gate_up(gate_up: torch.Tensor, ffn: int) -> torch.Tensor:
    """[gate rows | up rows] of GGUF blocks -> rows gate_0, up_0, gate_1, up_1, ... (the layout the SwiGLU row-pair
    epilogue reads); rows are whole numbers of blocks, so this is a permutation of byte ranges."""
    rb = gate_up.numel() // (2 * ffn)
    g = gate_up.view(2, ffn, rb)
    return torch.stack((g[0], g[1]), dim=1).reshape(-1).contiguous()


class DecodeStep:
    """weights: per layer a dict with GGUF-block device tensors 'qk' ([q_dim + kv_dim, hidden], q rows first),
    'v', 'o', 'gate_up' ([2 * ffn, hidden], gate rows first), 'down' and fp32 'attn_norm', 'ffn_norm';
    plus 'out_norm' (fp32) and 'head' at the top level."""

    def __init__(self, cfg: DecodeConfig, layers: list[dict], out_norm: torch.Tensor, head: torch.Tensor, device="cuda:0",
                 fuse: int = 4, embedding: torch.Tensor | None = None, penalty_window: int = 0):
        """embedding: the token-embedding table as GGUF blocks [vocab, hidden] (cfg.fmt_embd); with it a step starts from
        self.token (the id the previous step sampled, on the device) instead of a caller-filled self.x, so a replayed
        graph feeds itself.  penalty_window: entries of the repetition-penalty list (self.pen_tokens / self.pen_factors,
        set by set_penalties; unused entries hold token -1); 0 = plain greedy sampling.
        fuse: 4 (default) = 3 plus RMSNorm carried across the matmuls (see _step_carry): the producer of the
        residual stream stores x * norm_weight and partial sums of x^2, the consumer scales its result, so neither
        repeats the norm per workgroup and the RMSNorm launches disappear; 3 = SiLU(gate) * up runs in the epilogue of the gate+up matmul (the producer), whose rows
        are interleaved gate_0, up_0, gate_1, ... for it: 'gate_up' is re-laid out once, here, and the layer dicts are
        copied; 0 = every operator is its own launch; 1 = SiLU(gate) * up runs inside the staging of w_down;
        2 = RMSNorm is fused into the following matmuls as well.  Level 2 saves three more launches per layer but
        every workgroup of those matmuls then stages fp32 x and the norm weights (4x the bytes of fp16 x), which
        lengthens their start-up; likewise every workgroup of w_down recomputes SiLU * up for its whole input.  On
        MI355X neither level gains over separate launches (2.05 / 2.07 / 2.09 ms per token for 0 / 1 / 2 at the 8B
        shape, 1.96 / 1.72 for 3 / 4); fusing into the producer has no such cost.  The fused entry point stays for
        shapes where launches dominate."""
        if fuse >= 3:
            layers = [dict(L, gate_up=interleave_gate_up(L["gate_up"], cfg.ffn)) for L in layers]
        if fuse == 5 and cfg.head_dim != 128:
            raise ValueError("fuse = 5 needs head_dim 128 (the wide-split attention kernel)")
        if fuse >= 4:   # rows of q | k interleaved inside every head for the RoPE epilogue
            layers = [dict(L, qk=ops.interleave_rope_rows(L["qk"], cfg.q_dim + cfg.kv_dim, cfg.head_dim)) for L in layers]
        self.cfg, self.layers, self.out_norm, self.head, self.fuse = cfg, layers, out_norm, head, fuse
        dev = torch.device(device)
        c = cfg
        f16, f32 = torch.float16, torch.float32
        self.x = torch.zeros(c.hidden, dtype=f32, device=dev)            # residual stream
        self.xn = torch.empty(c.hidden, dtype=f16, device=dev)
        self.qk = torch.empty(c.q_dim + c.kv_dim, dtype=f32, device=dev)
        self.v = torch.empty(c.kv_dim, dtype=f32, device=dev)
        self.q_rot = torch.empty(c.q_dim, dtype=f32, device=dev)
        self.attn = torch.empty(c.q_dim, dtype=f16, device=dev)
        self.gu = torch.empty(2 * c.ffn, dtype=f16, device=dev)
        self.act = torch.empty(c.ffn, dtype=f16, device=dev)
        self.logits = torch.empty(c.vocab, dtype=f32, device=dev)
        self.token = torch.zeros(1, dtype=torch.int32, device=dev)
        self.params = torch.zeros(2, dtype=torch.int32, device=dev)      # {position, sequence length}
        self.sumsq_parts = torch.zeros((c.hidden + 7) // 8, dtype=f32, device=dev)   # carried RMSNorm: sum(x^2) per 8 outputs
        self.k_cache = [torch.zeros((c.max_ctx, c.kv_dim), dtype=f16, device=dev) for _ in layers]
        self.v_cache = [torch.zeros((c.max_ctx, c.kv_dim), dtype=f16, device=dev) for _ in layers]
        half = c.head_dim // 2
        inv = 1.0 / (c.rope_theta ** (torch.arange(half, dtype=torch.float64) * 2.0 / c.head_dim))
        ang = torch.arange(c.max_ctx, dtype=torch.float64)[:, None] * inv[None, :]
        self.cos_t = torch.cos(ang).to(f32).to(dev).contiguous()
        self.sin_t = torch.sin(ang).to(f32).to(dev).contiguous()
        self.ws = ops.attn_decode_workspace(c.n_heads, c.head_dim, c.max_ctx, dev)
        self.records = ops.attn_partial_records(c.n_heads, c.head_dim, c.max_ctx, dev) if fuse == 5 else None
        self.scale = 1.0 / math.sqrt(c.head_dim)
        self.embedding = embedding
        self.head_ws = ops.lm_head_workspace(c.vocab, dev)
        self.pen_tokens = torch.full((penalty_window,), -1, dtype=torch.int32, device=dev) if penalty_window else None
        self.pen_factors = torch.ones(penalty_window, dtype=f32, device=dev) if penalty_window else None

    def set_penalties(self, tokens: list[int], penalty: float, suppressed: list[int] = ()) -> None:
        """Host-side update between graph replays: the recent window at `penalty`, then `suppressed` tokens (end of
        sequence while a minimum length is enforced) at 1e9, the non-unit entries of the dense factor vector the
        reference's runner uploads (interface/runner/llama/llama.cpp:2566-2592).  The most recent entries are kept
        when the list is longer than the window."""
        cap = self.pen_tokens.numel()
        pairs = ([(t, penalty) for t in tokens] + [(t, 1e9) for t in suppressed])[-cap:]
        toks = [t for t, _ in pairs] + [-1] * (cap - len(pairs))
        facs = [f for _, f in pairs] + [1.0] * (cap - len(pairs))
        self.pen_tokens.copy_(torch.tensor(toks, dtype=torch.int32))
        self.pen_factors.copy_(torch.tensor(facs, dtype=torch.float32))

    def set_position(self, pos: int) -> None:
        """Host-side update between graph replays (a 8-byte copy; the kernels read it on the device)."""
        self.params.copy_(torch.tensor([pos, pos + 1], dtype=torch.int32))

    def _sample(self) -> None:
        """Penalty on the listed tokens (if a window was asked for) and the arg-max of the logits."""
        if self.pen_tokens is not None:
            ops.argmax_penalized(self.logits, self.token, self.pen_tokens, self.pen_factors)
        else:
            ops.argmax(self.logits, self.token)

    def step(self) -> None:
        """Consumes self.token through the embedding table (or, without a table, a caller-filled self.x), leaves the
        logits and the sampled token."""
        c = self.cfg
        if self.embedding is not None:
            ops.embedding_rows(self.embedding, c.fmt_embd, self.token, c.vocab, c.hidden, self.x.view(1, -1))
        if self.fuse == 2:
            return self._step_fused()
        if self.fuse >= 4:
            return self._step_carry()
        for i, L in enumerate(self.layers):
            ops.rmsnorm(self.x, L["attn_norm"], c.eps, out=self.xn.view(1, -1))
            # (running v beside q+k on a second stream was measured slower: the fork / join nodes of the graph cost
            # more than the 6 us the small matmul takes)
            # q | k and v in one launch although their formats differ
            ops.matmul_gguf_pair(self.xn, L["qk"], c.fmt_attn, c.q_dim + c.kv_dim, self.qk, L["v"], c.fmt_v, c.kv_dim, self.v,
                                 c.hidden)
            ops.rope_kv_write(self.qk[:c.q_dim], self.qk[c.q_dim:], self.v, self.params, self.cos_t, self.sin_t,
                              self.k_cache[i], self.v_cache[i], c.head_dim, self.q_rot)
            ops.attn_decode(self.q_rot, self.k_cache[i], self.v_cache[i], self.params, c.n_heads, c.n_kv_heads, c.head_dim,
                            self.scale, self.ws, self.attn)
            ops.matmul_gguf(self.attn, L["o"], c.fmt_attn, c.hidden, c.q_dim, out=self.x.view(1, -1), binary="add",
                            d=self.x.view(1, -1))
            ops.rmsnorm(self.x, L["ffn_norm"], c.eps, out=self.xn.view(1, -1))
            if self.fuse == 3:
                ops.matmul_gguf(self.xn, L["gate_up"], c.fmt_ffn, 2 * c.ffn, c.hidden, out=self.act.view(1, -1),
                                swiglu_pairs=True)
                ops.matmul_gguf(self.act, L["down"], c.fmt_ffn, c.hidden, c.ffn, out=self.x.view(1, -1), binary="add",
                                d=self.x.view(1, -1))
                continue
            ops.matmul_gguf(self.xn, L["gate_up"], c.fmt_ffn, 2 * c.ffn, c.hidden, out=self.gu.view(1, -1))
            if self.fuse >= 1:
                ops.matmul_gguf_pro(self.gu, L["down"], c.fmt_ffn, c.hidden, c.ffn, self.x, "swiglu", binary="add", d=self.x)
            else:
                ops.silu_mul(self.gu, self.act)
                ops.matmul_gguf(self.act, L["down"], c.fmt_ffn, c.hidden, c.ffn, out=self.x.view(1, -1), binary="add",
                                d=self.x.view(1, -1))
        ops.rmsnorm(self.x, self.out_norm, c.eps, out=self.xn.view(1, -1))
        ops.matmul_gguf(self.xn, self.head, c.fmt_head, c.vocab, c.hidden, out=self.logits.view(1, -1))
        self._sample()

    def _step_carry(self) -> None:
        """Six launches per layer (q|k|v with RoPE and cache append, attention, merge, wo, gate+up with SwiGLU, down);
        only the first RMSNorm of the step is a kernel, and the arg-max rides in the epilogue of the head matmul.  Every matmul that forms the
        residual stream (wo, w_down) also stores x * next_norm_weight as fp16 and the sum of x^2 over each group of 8
        outputs; the matmul that consumes it adds those partial sums (fixed order) and scales its result by
        rsqrt(sum / hidden + eps).  Producers and consumers alternate, so one array of partial sums serves all."""
        c = self.cfg
        n_layers = len(self.layers)
        consume = ops.norm_carry(sumsq_parts=self.sumsq_parts, eps=c.eps)
        ops.rmsnorm(self.x, self.layers[0]["attn_norm"], c.eps, out=self.xn.view(1, -1))
        for i, L in enumerate(self.layers):
            # layer 0 reads the output of the RMSNorm kernel (already scaled); the others the carried form
            # q | k | v projections, RoPE and the cache append in one launch
            ops.matmul_gguf_pair(self.xn, L["qk"], c.fmt_attn, c.q_dim + c.kv_dim, None, L["v"], c.fmt_v, c.kv_dim, None,
                                 c.hidden, carry=consume if i > 0 else None,
                                 rope=ops.rope_append(self.params, self.cos_t, self.sin_t, self.q_rot, self.k_cache[i],
                                                      self.v_cache[i], c.q_dim, c.head_dim))
            produce = ops.norm_carry(next_norm_weight=L["ffn_norm"], next_x16=self.xn, next_sumsq_parts=self.sumsq_parts)
            if self.fuse == 5:
                # five launches per layer: the attention leaves at most 8 records per head, wo folds them while it
                # stages its activations
                ops.attn_decode_partial(self.q_rot, self.k_cache[i], self.v_cache[i], self.params, c.n_heads, c.n_kv_heads,
                                        c.head_dim, self.scale, self.records)
                ops.matmul_gguf_attn_merge(self.records, L["o"], c.fmt_attn, c.hidden, self.x, carry=produce, binary="add",
                                           d=self.x)
            else:
                ops.attn_decode(self.q_rot, self.k_cache[i], self.v_cache[i], self.params, c.n_heads, c.n_kv_heads,
                                c.head_dim, self.scale, self.ws, self.attn)
                ops.matmul_gguf_carry(self.attn, L["o"], c.fmt_attn, c.hidden, c.q_dim, self.x, binary="add", d=self.x,
                                      carry=produce)
            ops.matmul_gguf_carry(self.xn, L["gate_up"], c.fmt_ffn, 2 * c.ffn, c.hidden, self.act, swiglu_pairs=True, carry=consume)
            nxt = self.layers[i + 1]["attn_norm"] if i + 1 < n_layers else self.out_norm
            ops.matmul_gguf_carry(self.act, L["down"], c.fmt_ffn, c.hidden, c.ffn, self.x, binary="add", d=self.x,
                                  carry=ops.norm_carry(next_norm_weight=nxt, next_x16=self.xn, next_sumsq_parts=self.sumsq_parts))
        ops.matmul_gguf_argmax(self.xn, self.head, c.fmt_head, c.vocab, c.hidden, self.logits, self.token, carry=consume,
                               pen_tokens=self.pen_tokens, pen_factors=self.pen_factors, workspace=self.head_ws)

    def _step_fused(self) -> None:
        c = self.cfg
        for i, L in enumerate(self.layers):
            ops.matmul_gguf_pro(self.x, L["qk"], c.fmt_attn, c.q_dim + c.kv_dim, c.hidden, self.qk, "rmsnorm", L["attn_norm"], c.eps)
            ops.matmul_gguf_pro(self.x, L["v"], c.fmt_v, c.kv_dim, c.hidden, self.v, "rmsnorm", L["attn_norm"], c.eps)
            ops.rope_kv_write(self.qk[:c.q_dim], self.qk[c.q_dim:], self.v, self.params, self.cos_t, self.sin_t,
                              self.k_cache[i], self.v_cache[i], c.head_dim, self.q_rot)
            ops.attn_decode(self.q_rot, self.k_cache[i], self.v_cache[i], self.params, c.n_heads, c.n_kv_heads, c.head_dim,
                            self.scale, self.ws, self.attn)
            ops.matmul_gguf(self.attn, L["o"], c.fmt_attn, c.hidden, c.q_dim, out=self.x.view(1, -1), binary="add",
                            d=self.x.view(1, -1))
            ops.matmul_gguf_pro(self.x, L["gate_up"], c.fmt_ffn, 2 * c.ffn, c.hidden, self.gu, "rmsnorm", L["ffn_norm"], c.eps)
            ops.matmul_gguf_pro(self.gu, L["down"], c.fmt_ffn, c.hidden, c.ffn, self.x, "swiglu", binary="add", d=self.x)
        ops.matmul_gguf_pro(self.x, self.head, c.fmt_head, c.vocab, c.hidden, self.logits, "rmsnorm", self.out_norm, c.eps)
        self._sample()
