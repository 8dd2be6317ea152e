"""Recurrent mixers: their memory of a sequence is a state of fixed size per request (a state slot), not pages.

`channel_delta`: the gated delta rule with one decay per head and key channel.  Per token, with h the mixer's
input row:
    q, k, v = silu(conv(W_q h)), silu(conv(W_k h)), silu(conv(W_v h))       short causal convolution per channel
    q <- q / |q| / sqrt(D),  k <- k / |k|                                     per head, |x| = sqrt(sum x^2 + 1e-6)
    beta = sigmoid(W_b h)                                                     one step size per head
    d = exp(-exp(A_log) * softplus(W_a2 (W_a1 h) + dt_bias))                  one decay per head and key channel
    S <- diag(d) S;  u = beta (v - S^T k);  S <- S + k u^T;  o = S^T q        S: [D, V] per head, float32
    y = W_o (o / rms(o) * w_norm * sigmoid(W_g2 (W_g1 h)))                    norm and gate per head
Value head j reads q/k head j // (heads / kv_heads).  The state S and the convolution's last taps - 1 inputs
are carried in the request's slot; everything from the convolution to the norm is float32.

`head_delta`: the same rule with one decay per head and full-rank gates:
    d = exp(-exp(A_log) * softplus(W_a h + dt_bias))                          one decay per head, S <- d S
    y = W_o (o / rms(o) * w_norm * silu(W_g h))
"""
from __future__ import annotations

import torch

from .. import debug, ops
from .base import MIXERS, Mixer, ParamSpec
from .linear import Linear, matmul, same_dtype

_aranges: dict = {}


def sequence_starts(ctx) -> torch.Tensor:
    """int32 [n_seqs + 1] on the device: sequence s owns tokens [starts[s], starts[s + 1]) of the step.  One upload
    per step, shared by the layers; a recorded step (token t is sequence t) reads a table that never changes."""
    if ctx.recorded:
        key = (ctx.device, ctx.n_seqs)
        if key not in _aranges:       # kept for the life of the process: recorded steps hold the address
            _aranges[key] = torch.arange(ctx.n_seqs + 1, dtype=torch.int32, device=ctx.device)
        return _aranges[key]
    return ctx.memo("sequence starts", lambda: torch.tensor(ctx.q_starts, dtype=torch.int32).pin_memory()
                    .to(ctx.device, non_blocking=True))


@MIXERS.register("channel_delta")
class ChannelDelta(Mixer):
    kernel_libraries = ("elementwise", "gemm", "recurrent")
    graph_safe = True          # every index comes from the context's device tensors; launches depend on sizes alone
    takes_post_norm = True
    TENSORS = {"q": "q", "k": "k", "v": "v", "q_conv": "q.conv", "k_conv": "k.conv", "v_conv": "v.conv", "beta": "b",
               "A_log": "A_log", "dt_bias": "dt_bias", "decay_in": "a1", "decay_out": "a2", "gate_in": "g1",
               "gate_out": "g2", "norm": "norm", "o": "o"}

    def __init__(self, hidden_size: int, n_heads: int, n_kv_heads: int, key_dim: int, v_dim: int, conv_taps: int,
                 norm_eps: float, decay_rank: int, gate_rank: int, names: dict | None = None):
        """`decay_rank`, `gate_rank`: inner sizes of the two low-rank projections (decay and output gate)."""
        if n_heads % n_kv_heads:
            raise ValueError(f"n_heads {n_heads} is not a multiple of n_kv_heads {n_kv_heads}")
        if not 1 <= key_dim <= 256:
            raise ValueError(f"key_dim {key_dim}: the recurrence kernel holds up to 256 key channels a head")
        if not 1 <= conv_taps <= 16:
            raise ValueError(f"conv_taps {conv_taps}: the convolution kernel takes 1..16 taps")
        self.hidden_size, self.n_heads, self.n_kv_heads = int(hidden_size), int(n_heads), int(n_kv_heads)
        self.key_dim, self.v_dim, self.conv_taps = int(key_dim), int(v_dim), int(conv_taps)
        self.norm_eps, self.decay_rank, self.gate_rank = float(norm_eps), int(decay_rank), int(gate_rank)
        self.names = dict(self.TENSORS, **(names or {}))
        self.qk_width, self.v_width = self.n_kv_heads * self.key_dim, self.n_heads * self.v_dim
        self.conv_channels = 2 * self.qk_width + self.v_width
        self.w_in = self.taps = self.decay_out = self.gate_out = self.decay_out_t = self.gate_out_t = self.A_log = self.dt_bias = self.norm_w = self.o_proj = None

    def param_specs(self):
        W, n = self.hidden_size, self.names
        H, D, t = self.n_heads, self.key_dim, self.conv_taps
        return {
            n["q"]: ParamSpec((self.qk_width, W)), n["q_conv"]: ParamSpec((self.qk_width, t)),
            n["k"]: ParamSpec((self.qk_width, W)), n["k_conv"]: ParamSpec((self.qk_width, t)),
            n["v"]: ParamSpec((self.v_width, W)), n["v_conv"]: ParamSpec((self.v_width, t)),
            n["beta"]: ParamSpec((H, W)), n["A_log"]: ParamSpec((H,)), n["norm"]: ParamSpec((self.v_dim,), init="ones"),
            n["decay_in"]: ParamSpec((self.decay_rank, W)), n["decay_out"]: ParamSpec((H * D, self.decay_rank)),
            n["dt_bias"]: ParamSpec((H * D,)),
            n["gate_in"]: ParamSpec((self.gate_rank, W)), n["gate_out"]: ParamSpec((self.v_width, self.gate_rank)),
            n["o"]: ParamSpec((W, self.v_width)),
        }

    def load(self, fetch):
        n = self.names
        # one product makes everything that reads the input row: q | k | v | beta | decay_in | gate_in
        self.w_in = torch.cat(same_dtype([fetch(n[x]) for x in ("q", "k", "v", "beta", "decay_in", "gate_in")]), dim=0).contiguous()
        # what feeds the recurrence stays float32: taps, the second halves of the low-rank projections, rates and biases
        self.taps = torch.cat([fetch(n[x]).float() for x in ("q_conv", "k_conv", "v_conv")], dim=0).contiguous()
        self.decay_out = fetch(n["decay_out"]).float().contiguous()
        self.gate_out = fetch(n["gate_out"]).float().contiguous()
        # (transposed copies for the few rows of a decode step, where both products are one launch)
        self.decay_out_t, self.gate_out_t = self.decay_out.t().contiguous(), self.gate_out.t().contiguous()
        self.A_log = fetch(n["A_log"]).float().contiguous()
        self.dt_bias = fetch(n["dt_bias"]).float().contiguous()
        self.norm_w = fetch(n["norm"]).contiguous()
        self.o_proj = Linear(fetch(n["o"]))

    def state_shapes(self) -> dict:
        return {"conv": ((self.conv_channels, self.conv_taps - 1), torch.float32),
                "S": ((self.n_heads, self.v_dim, self.key_dim), torch.float32)}      # kept transposed: [head][value][key]

    def forward(self, x, ctx, cache, residual, post_norm=None) -> None:
        H, G, D, V = self.n_heads, self.n_kv_heads, self.key_dim, self.v_dim
        C, QK = self.conv_channels, self.qk_width
        debug.region("delta in")
        proj = matmul(x, self.w_in, epilogue=ops.EPI_STORE_F32)
        starts = sequence_starts(ctx)
        o1 = C + H
        o2 = o1 + self.decay_rank
        debug.region("delta conv")
        conv = ops.short_conv(proj[:, :C], self.taps, cache.state["conv"], ctx.token_seq, starts, ctx.slot_ids, ctx.n_seqs)
        debug.region("delta gates")
        if ctx.n_tokens <= ops.SMALL_ROWS_MAX and max(self.decay_rank, self.gate_rank) <= ops.SMALL_ROWS_MAX_K:
            a, gate = ops.small_rows_pair(proj[:, o1:o2], self.decay_out_t, proj[:, o2:o2 + self.gate_rank], self.gate_out_t)
        else:
            a = ops.gemm(proj[:, o1:o2], self.decay_out, epilogue=ops.EPI_STORE_F32)
            gate = ops.gemm(proj[:, o2:o2 + self.gate_rank], self.gate_out, epilogue=ops.EPI_STORE_F32)
        qn, kn, decay, beta, kq = ops.delta_prepare(conv[:, :QK], conv[:, QK:2 * QK], a, proj[:, C:o1], self.A_log, self.dt_bias,
                                                H, G, D)
        debug.region("delta rule")
        o = ops.channel_delta(qn, kn, decay, beta, kq, conv[:, 2 * QK:], cache.state["S"], starts, ctx.slot_ids, ctx.n_seqs,
                              H, G, D, V)
        debug.region("delta out")
        y = ops.gated_head_norm(o, gate, self.norm_w, self.norm_eps, H, V, ctx.act_dtype)
        debug.region("o_proj")
        if post_norm is None:
            self.o_proj(y, epilogue=ops.EPI_RESID, out=residual)
        else:
            ops.rmsnorm_add(residual, self.o_proj(y, epilogue=ops.EPI_STORE_F32), post_norm[0], post_norm[1])


@MIXERS.register("head_delta")
class HeadDelta(ChannelDelta):
    """The gated delta rule with one decay per head (W_a: [heads, hidden], dt_bias: [heads]) and an output gate
    silu(W_g h) of full rank (W_g: [heads * v_dim, hidden]).  State, convolution, unit vectors, step sizes and the
    recurrence are `channel_delta`'s, through the same kernels: the decay of a head is handed to all its key channels."""
    TENSORS = {"q": "q", "k": "k", "v": "v", "q_conv": "q.conv", "k_conv": "k.conv", "v_conv": "v.conv", "beta": "b",
               "A_log": "A_log", "dt_bias": "dt_bias", "decay": "a", "gate": "g", "norm": "norm", "o": "o"}

    def __init__(self, hidden_size: int, n_heads: int, n_kv_heads: int, key_dim: int, v_dim: int, conv_taps: int,
                 norm_eps: float, gate_activation: str = "silu", names: dict | None = None):
        super().__init__(hidden_size, n_heads, n_kv_heads, key_dim, v_dim, conv_taps, norm_eps, decay_rank=1, gate_rank=1)
        if gate_activation not in ops.HEAD_GATES:
            raise ValueError(f"gate activation '{gate_activation}' is not one of {sorted(ops.HEAD_GATES)}")
        self.gate_activation = gate_activation
        self.names = dict(self.TENSORS, **(names or {}))

    def param_specs(self):
        W, n = self.hidden_size, self.names
        H, t = self.n_heads, self.conv_taps
        return {
            n["q"]: ParamSpec((self.qk_width, W)), n["q_conv"]: ParamSpec((self.qk_width, t)),
            n["k"]: ParamSpec((self.qk_width, W)), n["k_conv"]: ParamSpec((self.qk_width, t)),
            n["v"]: ParamSpec((self.v_width, W)), n["v_conv"]: ParamSpec((self.v_width, t)),
            n["beta"]: ParamSpec((H, W)), n["A_log"]: ParamSpec((H,)), n["norm"]: ParamSpec((self.v_dim,), init="ones"),
            n["decay"]: ParamSpec((H, W)), n["dt_bias"]: ParamSpec((H,)),
            n["gate"]: ParamSpec((self.v_width, W)), n["o"]: ParamSpec((W, self.v_width)),
        }

    def load(self, fetch):
        n = self.names
        # one product makes everything that reads the input row: q | k | v | beta | decay | gate
        self.w_in = torch.cat(same_dtype([fetch(n[x]) for x in ("q", "k", "v", "beta", "decay", "gate")]), dim=0).contiguous()
        self.taps = torch.cat([fetch(n[x]).float() for x in ("q_conv", "k_conv", "v_conv")], dim=0).contiguous()
        self.A_log = fetch(n["A_log"]).float().contiguous()
        self.dt_bias = fetch(n["dt_bias"]).float().contiguous()
        self.norm_w = fetch(n["norm"]).contiguous()
        self.o_proj = Linear(fetch(n["o"]))

    def forward(self, x, ctx, cache, residual, post_norm=None, out_scale: float | None = None) -> None:
        H, G, D, V = self.n_heads, self.n_kv_heads, self.key_dim, self.v_dim
        C, QK = self.conv_channels, self.qk_width
        debug.region("delta in")
        proj = matmul(x, self.w_in, epilogue=ops.EPI_STORE_F32)
        starts = sequence_starts(ctx)
        o1 = C + H          # beta ends
        o2 = o1 + H         # decay ends; the gate's rows follow
        debug.region("delta conv")
        conv = ops.short_conv(proj[:, :C], self.taps, cache.state["conv"], ctx.token_seq, starts, ctx.slot_ids, ctx.n_seqs)
        debug.region("delta gates")
        qn, kn, decay, beta, kq = ops.delta_prepare(conv[:, :QK], conv[:, QK:2 * QK], proj[:, o1:o2], proj[:, C:o1], self.A_log,
                                                    self.dt_bias, H, G, D, per_head=True)
        debug.region("delta rule")
        o = ops.channel_delta(qn, kn, decay, beta, kq, conv[:, 2 * QK:], cache.state["S"], starts, ctx.slot_ids, ctx.n_seqs,
                              H, G, D, V)
        debug.region("delta out")
        y = ops.gated_head_norm(o, proj[:, o2:o2 + self.v_width], self.norm_w, self.norm_eps, H, V, ctx.act_dtype,
                                gate_activation=self.gate_activation)
        debug.region("o_proj")
        if post_norm is None:
            scale = ops.constant_rows(y.device, out_scale, ctx.n_tokens) if out_scale is not None and out_scale != 1.0 else None
            self.o_proj(y, epilogue=ops.EPI_RESID, out=residual, row_scale=scale)
        else:
            ops.rmsnorm_add(residual, self.o_proj(y, epilogue=ops.EPI_STORE_F32), post_norm[0], post_norm[1])
