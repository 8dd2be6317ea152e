"""Arrangements of a mixer, a feed-forward and norms in one layer."""
from __future__ import annotations

import torch

from .. import debug
from .base import BLOCKS, FEED_FORWARDS, MIXERS, NORMS, Block, ParamSpec
from .linear import Linear


@BLOCKS.register("prenorm")
class PreNormBlock(Block):
    """h += mixer(norm1(h)); h += ffn(norm2(h))   (ferrox-models/src/decoder.rs:1-5, 2155-2173).
    A layer without a feed-forward has the first half only."""
    slots = {"norm1": NORMS, "mixer": MIXERS, "norm2": NORMS, "ffn": FEED_FORWARDS}
    optional_slots = ("norm2", "ffn")

    def __init__(self, parts: dict, prefixes: dict):
        self.norm1, self.mixer, self.norm2, self.ffn = parts["norm1"], parts["mixer"], parts.get("norm2"), parts.get("ffn")
        if (self.ffn is None) != (self.norm2 is None):
            raise ValueError("a pre-norm block has a feed-forward and its norm, or neither")
        self._prefixes = prefixes

    def children(self):
        return [(self._prefixes[s], getattr(self, s)) for s in ("norm1", "mixer", "norm2", "ffn") if getattr(self, s) is not None]

    chains_norms = True     # forward takes `normed` and `then` and returns what the next block may take as `normed`

    @property
    def first_norm(self):
        return self.norm1

    def takes_scale_later(self, act_dtype) -> bool:
        return bool(self.mixer.takes_scale_later(act_dtype))

    def forward(self, h, ctx, cache, normed=None, then=None):
        """`normed`: norm1(h), if the block before has already made it (a tensor, or an ops.ScaleLater if this
        block's mixer takes one).  `then`: (the norm that the next block applies first, whether its mixer
        takes an ops.ScaleLater); a feed-forward that says `norms_after` may apply that norm to the rows it
        has just finished and leave the result in ctx.carry, which is returned (else None)."""
        # a part may offer `forward_from_residual(norm, ...)`: it then applies the norm itself, fused
        # into its first kernel, and says False when it cannot for this step
        if normed is not None:
            self.mixer.forward(normed, ctx, cache, h)
        elif not self.mixer.forward_from_residual(self.norm1, ctx, cache, h):
            debug.region("norm")
            self.mixer.forward(self.norm1.forward(h, ctx), ctx, cache, h)
        ctx.carry = None
        if self.ffn is None:
            return None
        more = {"then_norm": then} if then is not None and self.ffn.norms_after else {}
        if not self.ffn.forward_from_residual(self.norm2, ctx, h, **more):
            debug.region("norm")
            self.ffn.forward(self.norm2.forward(h, ctx), ctx, h, **more)
        out, ctx.carry = ctx.carry, None
        return out


@BLOCKS.register("sandwich")
class SandwichBlock(Block):
    """h += norm1b(mixer(norm1(h))); h += norm2b(ffn(norm2(h))): a norm before and after each sublayer.
    A layer without a feed-forward has the first half only.

    A sublayer's output is normed before it joins the residual stream, so it cannot be added there by the
    sublayer's last product.  A part that sets `takes_post_norm` is called with `post_norm=(weight, eps)` and
    ends with one kernel that norms its float32 output rows and adds them; any other part adds into a zeroed
    float32 buffer in place of the stream, which is then normed and added."""
    slots = {"norm1": NORMS, "mixer": MIXERS, "norm1b": NORMS, "norm2": NORMS, "ffn": FEED_FORWARDS, "norm2b": NORMS}
    optional_slots = ("norm2", "ffn", "norm2b")

    def __init__(self, parts: dict, prefixes: dict):
        self.norm1, self.mixer, self.norm1b = parts["norm1"], parts["mixer"], parts["norm1b"]
        self.ffn = parts.get("ffn")
        self.norm2, self.norm2b = parts.get("norm2"), parts.get("norm2b")
        if self.ffn is not None and (self.norm2 is None or self.norm2b is None):
            raise ValueError("a sandwich block with a feed-forward needs norm2 and norm2b")
        self._prefixes = prefixes

    def children(self):
        return [(self._prefixes[s], getattr(self, s)) for s in self.slots if getattr(self, s, None) is not None]

    @staticmethod
    def _sublayer(part, post, x, ctx, h, *cache):
        rms = post.rms_params()
        if rms is not None and getattr(part, "takes_post_norm", False):
            part.forward(x, ctx, *cache, h, post_norm=rms)
            return
        from .. import ops
        out = torch.empty_like(h)
        ops.fill_u32(out, 0)
        part.forward(x, ctx, *cache, out)
        debug.region("norm")
        if rms is not None:
            ops.rmsnorm_add(h, out, rms[0], rms[1])
        else:
            ops.residual_add(h, post.forward(out, ctx))

    def forward(self, h, ctx, cache):
        debug.region("norm")
        self._sublayer(self.mixer, self.norm1b, self.norm1.forward(h, ctx), ctx, h, cache)
        if self.ffn is not None:
            debug.region("norm")
            self._sublayer(self.ffn, self.norm2b, self.norm2.forward(h, ctx), ctx, h)


@BLOCKS.register("parallel")
class ParallelBlock(Block):
    """h += mixer(norm1(h)) + ffn(norm1(h)): one norm, and both sublayers read its output.  A layer without a
    feed-forward has the mixer only.  Both sublayers end with a product that adds into the float32 stream; the
    normed rows are made before either has added, so the order of the two additions changes rounding alone."""
    slots = {"norm1": NORMS, "mixer": MIXERS, "ffn": FEED_FORWARDS}
    optional_slots = ("ffn",)

    def __init__(self, parts: dict, prefixes: dict):
        self.norm1, self.mixer, self.ffn = parts["norm1"], parts["mixer"], parts.get("ffn")
        self._prefixes = prefixes

    def children(self):
        return [(self._prefixes[s], getattr(self, s)) for s in self.slots if getattr(self, s, None) is not None]

    def forward(self, h, ctx, cache):
        debug.region("norm")
        x = self.norm1.forward(h, ctx)
        self.mixer.forward(x, ctx, cache, h)
        if self.ffn is not None:
            self.ffn.forward(x, ctx, h)


@BLOCKS.register("gated_prenorm")
class GatedPreNormBlock(Block):
    """h += G1 * mixer(C(x1)),  x1 = norm1(h);  h += G2 * ffn(x2),  x2 = norm2(h), with two optional additions to the
    pre-norm block:
      * an input convolution, C(x) = x + conv(x): a short causal convolution over time on each channel of what the
        mixer reads (`conv_taps` >= 1; weights [hidden, taps], the last column meets the current token; no bias, no
        activation).  The last taps - 1 normed rows of every request are part of its state (`block.conv`).
      * a gated residual, G = sigmoid(W x + b) element by element, x being the normed rows the sublayer was handed
        (before the input convolution): a sublayer's float32 output rows pass the gate as they join the stream.
    A layer without a feed-forward has the first half only.  A sublayer leaves its output in a float32 buffer in
    place of the stream (stored by its last product if it says `takes_fresh`, else added into a zeroed buffer),
    which one kernel then gates and adds."""
    slots = {"norm1": NORMS, "mixer": MIXERS, "norm2": NORMS, "ffn": FEED_FORWARDS}
    optional_slots = ("norm2", "ffn")
    kernel_libraries = ("elementwise", "gemm", "recurrent")
    TENSORS = {"conv": "conv1", "gate1": "gate1.weight", "gate1_bias": "gate1.bias", "gate2": "gate2.weight",
               "gate2_bias": "gate2.bias"}

    def __init__(self, parts: dict, prefixes: dict, hidden_size: int, conv_taps: int = 0, residual_gates: bool = True,
                 names: dict | None = None):
        self.norm1, self.mixer, self.norm2, self.ffn = parts["norm1"], parts["mixer"], parts.get("norm2"), parts.get("ffn")
        if (self.ffn is None) != (self.norm2 is None):
            raise ValueError("a gated pre-norm block has a feed-forward and its norm, or neither")
        self.hidden_size, self.conv_taps, self.residual_gates = int(hidden_size), int(conv_taps or 0), bool(residual_gates)
        if self.conv_taps > 16:
            raise ValueError(f"conv_taps {conv_taps}: the convolution kernel takes up to 16 taps")
        self.names = dict(self.TENSORS, **(names or {}))
        self._prefixes = prefixes
        self.taps = self.gate1 = self.gate2 = None

    def children(self):
        return [(self._prefixes[s], getattr(self, s)) for s in ("norm1", "mixer", "norm2", "ffn") if getattr(self, s) is not None]

    def param_specs(self):
        W, n = self.hidden_size, self.names
        specs = {}
        if self.conv_taps:
            specs[n["conv"]] = ParamSpec((W, self.conv_taps))
        if self.residual_gates:
            specs.update({n["gate1"]: ParamSpec((W, W)), n["gate1_bias"]: ParamSpec((W,), init="zeros")})
            if self.ffn is not None:
                specs.update({n["gate2"]: ParamSpec((W, W)), n["gate2_bias"]: ParamSpec((W,), init="zeros")})
        return specs

    def load(self, fetch):
        n = self.names
        if self.conv_taps:
            self.taps = fetch(n["conv"]).float().contiguous()
        if self.residual_gates:
            self.gate1 = Linear(fetch(n["gate1"]), fetch(n["gate1_bias"]).float().contiguous())
            if self.ffn is not None:
                self.gate2 = Linear(fetch(n["gate2"]), fetch(n["gate2_bias"]).float().contiguous())

    def state_shapes(self) -> dict:
        return {"conv": ((self.hidden_size, self.conv_taps - 1), torch.float32)} if self.conv_taps else {}

    @staticmethod
    def _into(part, out, x, ctx, *cache):
        """The sublayer's output rows in `out`: a part that says `takes_fresh` stores them with its last product,
        any other adds them into a zeroed buffer."""
        from .. import ops
        if getattr(part, "takes_fresh", False):
            part.forward(x, ctx, *cache, out, fresh=True)
        else:
            ops.fill_u32(out, 0)
            part.forward(x, ctx, *cache, out)

    def _join(self, h, out, gate, x, ctx=None, then=None):
        """The sublayer's rows through their gate into the stream.  `then`: the norm that reads the stream next; if it
        offers `after_gated_add`, the add and that norm are one launch, and its rows are returned."""
        from .. import ops
        debug.region("residual gate")
        if gate is None:
            ops.residual_add(h, out)
            return None
        logits = gate(x, epilogue=ops.EPI_STORE_F32)
        fused = getattr(then, "after_gated_add", None)
        normed = fused(h, out, logits, ctx) if fused is not None else None
        if normed is None:
            ops.gated_add(h, out, logits)
        return normed

    chains_norms = True     # forward takes `normed` and `then` and returns what the next block may take as `normed`

    @property
    def first_norm(self):
        return self.norm1

    def forward(self, h, ctx, cache, normed=None, then=None):
        """`normed`: norm1(h), if the block before has made it with the add that finished its rows.  `then`: (the
        norm that the next block applies first, ...): this block's last gated add makes that norm's rows too, where
        the norm offers it, and they are returned (else None)."""
        from .. import ops
        from .recurrent import sequence_starts
        after = then[0] if then is not None else None
        x = normed
        if x is None:
            debug.region("norm")
            x = self.norm1.forward(h, ctx)
        read = x
        if self.conv_taps:
            debug.region("input conv")
            read = ops.short_conv(x, self.taps, cache.state["block.conv"], ctx.token_seq, sequence_starts(ctx), ctx.slot_ids,
                                  ctx.n_seqs, activation=None, add_input=True, out_dtype=x.dtype)
        out = torch.empty_like(h)
        self._into(self.mixer, out, read, ctx, cache)
        x = self._join(h, out, self.gate1, x, ctx, self.norm2 if self.ffn is not None else after)
        if self.ffn is None:
            return x
        if x is None:
            debug.region("norm")
            x = self.norm2.forward(h, ctx)
        self._into(self.ffn, out, x, ctx)
        return self._join(h, out, self.gate2, x, ctx, after)
