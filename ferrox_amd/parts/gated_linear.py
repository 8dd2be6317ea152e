"""Mixers whose memory of a sequence is a linear recurrence with gates that do not depend on the state: a state of
fixed size per request (a state slot), no pages.  Everything that enters a recurrence is float32.

`decay_attention`: linear attention with one constant decay per head.  Per token, with h the mixer's input row:
    q, k, v = act(W_q h), act(W_k h), act(W_v h)                              heads x dim, heads x dim, heads x v_dim
    S <- decay_h S + k v^T;  o = S^T q                                        S: [D, V] per head
    y = W_o (o / rms(o) * w_norm * sigmoid(W_g h))                            one norm over all heads together

`matrix_memory`: a matrix memory with exponential gates kept in range by a running maximum.  Per head:
    q = W_q h * D^-1/2,  k = W_k h,  v = W_v h
    i = cap tanh((W_i h + b_i) / cap),  f = logsigmoid(cap tanh((W_f h + b_f) / cap))          two logarithms
    m <- max(f + m, i);  S <- exp(f + m_old - m) S + exp(i - m) k v^T;  n likewise with k alone      m, S, n from zero
    o = S^T q / (max(|n . q|, exp(-m)) + 1e-6)
    y = W_o (o / rms(o) per head * w_norm * sigmoid(W_g h))                   w_norm: one weight per head and channel

`rglru`: a recurrent block around a real-gated linear recurrent unit.  Two branches of `width` channels:
    b = gelu_tanh(W_y h + b_y);  u = conv(W_x h + b_x)                        short causal convolution with bias, no activation
    r = sigmoid(A_r[j] u_j + b_r[j]),  i = sigmoid(A_i[j] u_j + b_i[j])       u cut into `blocks` parts j, a square matrix each
    a = exp(-rate r softplus(lam));  S <- a S + sqrt(1 - a^2) i u              per channel
    y = W_o (S b)
"""
from __future__ import annotations

import torch

from .. import debug, ops
from .base import MIXERS, Mixer, ParamSpec
from .latent import head_groups
from .linear import Linear, matmul, same_dtype
from .recurrent import sequence_starts


def longest_portion(ctx) -> int:
    """The most tokens that one sequence brings to this step (1 in a recorded step)."""
    if ctx.recorded:
        return 1
    return max((ctx.q_starts[s + 1] - ctx.q_starts[s] for s in range(ctx.n_seqs)), default=0)


def _add_out(o_proj, y, ctx, residual, out_scale, fresh=False):
    """The output projection into `residual`: added, or, where the caller says that `residual` holds nothing yet
    (`fresh`), stored."""
    debug.region("o_proj")
    if fresh and (out_scale is None or out_scale == 1.0):
        o_proj(y, epilogue=ops.EPI_STORE_F32, out=residual)
        return
    if fresh:
        ops.fill_u32(residual, 0)
    scale = ops.constant_rows(y.device, out_scale, ctx.n_tokens) if out_scale is not None and out_scale != 1.0 else None
    o_proj(y, epilogue=ops.EPI_RESID, out=residual, row_scale=scale)


@MIXERS.register("decay_attention")
class DecayAttention(Mixer):
    kernel_libraries = ("elementwise", "gemm", "recurrent")
    graph_safe = True
    TENSORS = {"q": "q", "k": "k", "v": "v", "gate": "g", "norm": "norm", "o": "o"}

    def __init__(self, hidden_size: int, n_heads: int, key_dim: int, v_dim: int, decay, norm_eps: float,
                 activation: str = "silu", names: dict | None = None):
        """`decay`: n_heads numbers in (0, 1], the factor a head's state is multiplied by at every token.
        `activation`: what q, k and v go through after their projections (one of ops.STORED_ACTIVATIONS, or None)."""
        self.hidden_size, self.n_heads, self.key_dim, self.v_dim = int(hidden_size), int(n_heads), int(key_dim), int(v_dim)
        self.decay = tuple(float(d) for d in decay)
        if len(self.decay) != self.n_heads or not all(0.0 < d <= 1.0 for d in self.decay):
            raise ValueError(f"{len(self.decay)} decays for {n_heads} heads, each in (0, 1]: {self.decay}")
        if not 1 <= self.key_dim <= 256:
            raise ValueError(f"key_dim {key_dim}: the recurrence kernel holds up to 256 key channels a head")
        if activation not in ops.STORED_ACTIVATIONS:
            raise ValueError(f"activation '{activation}' is not one of {sorted(a for a in ops.STORED_ACTIVATIONS if a)}")
        self.activation, self.norm_eps = activation, float(norm_eps)
        self.names = dict(self.TENSORS, **(names or {}))
        self.qk_width, self.v_width = self.n_heads * self.key_dim, self.n_heads * self.v_dim
        self.w_qkv = self.w_gate = self.norm_w = self.o_proj = self.decays = None

    def param_specs(self):
        W, n = self.hidden_size, self.names
        return {n["q"]: ParamSpec((self.qk_width, W)), n["k"]: ParamSpec((self.qk_width, W)),
                n["v"]: ParamSpec((self.v_width, W)), n["gate"]: ParamSpec((self.v_width, W)),
                n["norm"]: ParamSpec((self.v_width,), init="ones"), n["o"]: ParamSpec((W, self.v_width))}

    def load(self, fetch):
        n = self.names
        self.w_qkv = torch.cat(same_dtype([fetch(n[x]) for x in ("q", "k", "v")]), dim=0).contiguous()
        self.w_gate = fetch(n["gate"]).contiguous()
        self.norm_w = fetch(n["norm"]).float().contiguous()
        self.o_proj = Linear(fetch(n["o"]))
        self.decays = torch.tensor(self.decay, dtype=torch.float64).to(torch.float32).to(self.w_qkv.device)

    def state_shapes(self) -> dict:
        return {"S": ((self.n_heads, self.v_dim, self.key_dim), torch.float32)}      # transposed: [head][value][key]

    takes_fresh = True       # forward(..., fresh=True): `residual` holds nothing yet, the output is stored into it

    def forward(self, x, ctx, cache, residual, out_scale: float | None = None, fresh: bool = False) -> None:
        H, D, V, QK = self.n_heads, self.key_dim, self.v_dim, self.qk_width
        debug.region("linear in")
        # the activation is applied to the float32 sums as they are stored: what the recurrence reads is float32
        qkv = matmul(x, self.w_qkv, epilogue=ops.EPI_STORE_F32, store_activation=self.activation)
        gate = matmul(x, self.w_gate, epilogue=ops.EPI_STORE_F32)
        debug.region("linear recurrence")
        o = ops.gated_outer(qkv[:, :QK], qkv[:, QK:2 * QK], qkv[:, 2 * QK:], self.decays, None, cache.state["S"],
                            sequence_starts(ctx), ctx.slot_ids, ctx.n_seqs, H, H, D, V)
        debug.region("linear out")
        y = ops.gated_head_norm(o, gate, self.norm_w, self.norm_eps, 1, H * V, ctx.act_dtype)      # all heads as one row
        _add_out(self.o_proj, y, ctx, residual, out_scale, fresh)


@MIXERS.register("matrix_memory")
class MatrixMemory(Mixer):
    kernel_libraries = ("elementwise", "gemm", "recurrent")
    graph_safe = True
    TENSORS = {"q": "q", "k": "k", "v": "v", "in": "i", "in_bias": "i.b", "forget": "f", "forget_bias": "f.b", "gate": "g",
               "norm": "norm", "o": "o"}

    def __init__(self, hidden_size: int, n_heads: int, key_dim: int, v_dim: int, gate_cap: float, norm_eps: float,
                 names: dict | None = None):
        """`gate_cap`: both gates' projections go through cap tanh(x / cap) before they become logarithms."""
        self.hidden_size, self.n_heads, self.key_dim, self.v_dim = int(hidden_size), int(n_heads), int(key_dim), int(v_dim)
        if not 1 <= self.key_dim <= 256:
            raise ValueError(f"key_dim {key_dim}: the recurrence kernel holds up to 256 key channels a head")
        self.gate_cap, self.norm_eps = float(gate_cap), float(norm_eps)
        if not self.gate_cap > 0.0:
            raise ValueError(f"a gate cap of {gate_cap}")
        self.names = dict(self.TENSORS, **(names or {}))
        self.qk_width, self.v_width = self.n_heads * self.key_dim, self.n_heads * self.v_dim
        self.w_in = self.norm_w = self.o_proj = None

    def param_specs(self):
        W, n, H = self.hidden_size, self.names, self.n_heads
        return {n["q"]: ParamSpec((self.qk_width, W)), n["k"]: ParamSpec((self.qk_width, W)),
                n["v"]: ParamSpec((self.v_width, W)), n["gate"]: ParamSpec((self.v_width, W)),
                n["in"]: ParamSpec((H, W)), n["in_bias"]: ParamSpec((H,), init="zeros"),
                n["forget"]: ParamSpec((H, W)), n["forget_bias"]: ParamSpec((H,), init="zeros"),
                n["norm"]: ParamSpec((self.v_width,), init="ones"), n["o"]: ParamSpec((W, self.v_width))}

    def load(self, fetch):
        n, H = self.names, self.n_heads
        # one product makes everything that reads the input row: q | k | v | output gate | input gate | forget gate
        w = torch.cat(same_dtype([fetch(n[x]) for x in ("q", "k", "v", "gate", "in", "forget")]), dim=0).contiguous()
        bias = torch.zeros(w.shape[0], dtype=torch.float32, device=w.device)
        bias[-2 * H:-H] = fetch(n["in_bias"]).float()
        bias[-H:] = fetch(n["forget_bias"]).float()
        self.w_in = Linear(w, bias)
        self.norm_w = fetch(n["norm"]).float().contiguous()
        self.o_proj = Linear(fetch(n["o"]))

    def state_shapes(self) -> dict:
        return {"S": ((self.n_heads, self.v_dim + 1, self.key_dim), torch.float32),      # transposed; the last column is n
                "m": ((self.n_heads,), torch.float32)}

    takes_fresh = True

    def forward(self, x, ctx, cache, residual, out_scale: float | None = None, fresh: bool = False) -> None:
        H, D, V, QK, VW = self.n_heads, self.key_dim, self.v_dim, self.qk_width, self.v_width
        debug.region("memory in")
        proj = self.w_in(x, epilogue=ops.EPI_STORE_F32)
        g0 = 2 * QK + VW          # the output gate's columns begin
        i0 = g0 + VW              # the input gate's
        starts = sequence_starts(ctx)
        debug.region("memory gates")
        keep, take, m = ops.exp_gate_scan(proj[:, i0:i0 + H], proj[:, i0 + H:i0 + 2 * H], self.gate_cap, cache.state["m"],
                                          starts, ctx.slot_ids, ctx.n_seqs, H)
        debug.region("linear recurrence")
        o, nq = ops.gated_outer(proj[:, :QK], proj[:, QK:2 * QK], proj[:, 2 * QK:g0], keep, take, cache.state["S"], starts,
                                ctx.slot_ids, ctx.n_seqs, H, H, D, V, q_scale=D ** -0.5, normalizer=True)
        debug.region("memory out")
        y = ops.gated_head_norm(o, proj[:, g0:i0], self.norm_w, self.norm_eps, H, V, ctx.act_dtype, denominators=(nq, m))
        _add_out(self.o_proj, y, ctx, residual, out_scale, fresh)


@MIXERS.register("rglru")
class RGLRU(Mixer):
    kernel_libraries = ("elementwise", "gemm", "recurrent")
    graph_safe = True
    RATE = 8.0               # log a = -RATE * r * softplus(lam)
    TENSORS = {"branch": "y", "branch_bias": "y.b", "in": "x", "in_bias": "x.b", "conv": "conv", "conv_bias": "conv.b",
               "rec_gate": "ra", "rec_gate_bias": "ra.b", "in_gate": "ri", "in_gate_bias": "ri.b", "lam": "lam", "o": "o"}

    def __init__(self, hidden_size: int, width: int, n_blocks: int, conv_taps: int, names: dict | None = None):
        self.hidden_size, self.width, self.n_blocks, self.conv_taps = int(hidden_size), int(width), int(n_blocks), int(conv_taps)
        if self.n_blocks < 1 or self.width % self.n_blocks:
            raise ValueError(f"a width of {width} is not cut into {n_blocks} equal parts")
        if not 1 <= self.conv_taps <= 16:
            raise ValueError(f"conv_taps {conv_taps}: the convolution kernel takes 1..16 taps")
        self.names = dict(self.TENSORS, **(names or {}))
        self.w_in = self.taps = self.conv_bias = self.w_gates = self.w_gates_t = self.gate_bias = self.lam = self.o_proj = None

    def param_specs(self):
        W, C, B, n = self.hidden_size, self.width, self.n_blocks, self.names
        cb = C // B
        return {n["branch"]: ParamSpec((C, W)), n["branch_bias"]: ParamSpec((C,), init="zeros"),
                n["in"]: ParamSpec((C, W)), n["in_bias"]: ParamSpec((C,), init="zeros"),
                n["conv"]: ParamSpec((C, self.conv_taps)), n["conv_bias"]: ParamSpec((C,), init="zeros"),
                n["rec_gate"]: ParamSpec((B, cb, cb)), n["rec_gate_bias"]: ParamSpec((B, cb), init="zeros"),
                n["in_gate"]: ParamSpec((B, cb, cb)), n["in_gate_bias"]: ParamSpec((B, cb), init="zeros"),
                n["lam"]: ParamSpec((C,)), n["o"]: ParamSpec((W, C))}

    def load(self, fetch):
        n = self.names
        w = torch.cat(same_dtype([fetch(n["branch"]), fetch(n["in"])]), dim=0).contiguous()
        self.w_in = Linear(w, torch.cat([fetch(n["branch_bias"]).float(), fetch(n["in_bias"]).float()]).contiguous())
        # what feeds the recurrence stays float32: taps, the gates' matrices and biases, the rates
        self.taps = fetch(n["conv"]).float().contiguous()
        self.conv_bias = fetch(n["conv_bias"]).float().contiguous()
        # per part j one matrix [2 cb, cb]: the recurrence gate's rows, then the input gate's
        self.w_gates = torch.cat([fetch(n["rec_gate"]).float(), fetch(n["in_gate"]).float()], dim=1).contiguous()
        self.gate_bias = torch.cat([fetch(n["rec_gate_bias"]).float(), fetch(n["in_gate_bias"]).float()], dim=1).contiguous()
        # (a transposed copy for the few rows of a decode step, where the parts' products are one small launch)
        self.w_gates_t = self.w_gates.transpose(1, 2).contiguous()
        self.lam = fetch(n["lam"]).float().contiguous()
        self.o_proj = Linear(fetch(n["o"]))

    def state_shapes(self) -> dict:
        return {"S": ((self.width,), torch.float32), "conv": ((self.width, self.conv_taps - 1), torch.float32)}

    takes_fresh = True

    def forward(self, x, ctx, cache, residual, out_scale: float | None = None, fresh: bool = False) -> None:
        C, B, T = self.width, self.n_blocks, ctx.n_tokens
        cb = C // B
        debug.region("lru in")
        proj = self.w_in(x, epilogue=ops.EPI_STORE_F32)                 # [T, C | C]: the gelu branch, then the recurrent one
        starts = sequence_starts(ctx)
        debug.region("lru conv")
        u = ops.short_conv(proj[:, C:], self.taps, cache.state["conv"], ctx.token_seq, starts, ctx.slot_ids, ctx.n_seqs,
                           activation=None, bias=self.conv_bias)
        debug.region("lru gates")
        # the gates' products, a part of the channels each: part j of token t is row t*B + j of [T*B, cb]
        if T <= ops.SMALL_ROWS_MAX and cb <= ops.SMALL_ROWS_MAX_K:
            logits = ops.small_rows_parts(u, self.w_gates_t)
        else:
            rows, offsets = head_groups(u.device, T, B)
            logits = torch.empty((T * B, 2 * cb), dtype=torch.float32, device=u.device)
            ops.gemm(u.view(T * B, cb), self.w_gates, a_rows=rows, c_rows=rows, expert_offsets=offsets, n_rows=T * B,
                     epilogue=ops.EPI_STORE_F32, out=logits)
        debug.region("linear recurrence")
        # (the gates' biases join inside: the grouped product has one bias for all groups)
        y = ops.rglru(u, logits, self.gate_bias, B, self.lam, proj[:, :C], cache.state["S"], starts, ctx.slot_ids, ctx.n_seqs,
                      longest_portion(ctx), ctx.act_dtype, rate=self.RATE)
        _add_out(self.o_proj, y, ctx, residual, out_scale, fresh)
