"""Causal grouped-query attention over the paged cache.

Per token (ferrox-models/src/decoder.rs:3224-3560): q, k, v = W x + b, the bias
added before the rotation; q and k rotated by the position encoding; k and v
written into the pages; the query attends to its sequence's pages (its own
position included, through the cache just written); the heads' outputs go
through o_proj (no bias) into the residual stream.  Optionally every head of q
and of k goes through a norm of its own between the bias and the rotation
(`qk_norm`; the reference applies such norms where a model's tensors exist,
decoder.rs:2099-2104, 3256-3267; this architecture has none).
"""
from __future__ import annotations

import math

import torch

from .. import debug, limits, ops
from .base import MIXERS, NORMS, POSITION_ENCODINGS, Mixer, ParamSpec, PartSpec, Rotary
from .linear import Linear, matmul, same_dtype

NO_ROTATION = Rotary(0, 1.0)
FUSE_HEAD_NORMS = True      # (a switch for tests: the norms of q's and k's heads and the cache write as one launch)
EVEN_BLOCKS_PER_CU = 250 / 256     # items of 128 queries pay from about one evenly loaded block per CU on (measured on 256 CUs)


def attention_items(ctx, tile_q: int = 64):
    """Work items of a step, shared by the attention layers of one item size: sequences with one
    new token go to the split decode kernel, the others are cut into blocks of
    tile_q consecutive queries."""
    if ctx.recorded:      # token t is the one token of sequence t; nothing is made from host lists
        return {"n_decode": ctx.n_seqs, "n_tiles": 0, "max_kv": ctx.kv_bound, "dec_seq": ctx.token_seq,
                "dec_tok": ctx.token_seq}
    dec_seq, dec_tok, t_seq, t_tok, t_n = [], [], [], [], []
    max_kv = 1
    for s in range(ctx.n_seqs):
        b, e = ctx.q_starts[s], ctx.q_starts[s + 1]
        if e - b == 1:
            dec_seq.append(s)
            dec_tok.append(b)
            max_kv = max(max_kv, ctx.kv_lens[s])
        else:
            for t0 in range(b, e, tile_q):
                t_seq.append(s)
                t_tok.append(t0)
                t_n.append(min(tile_q, e - t0))
    flat = dec_seq + dec_tok + t_seq + t_tok + t_n
    # through pinned memory, so that the host does not wait here for the kernels launched before
    dev = torch.tensor(flat, dtype=torch.int32).pin_memory().to(ctx.device, non_blocking=True) if flat else None
    nd, nt = len(dec_seq), len(t_seq)
    items = {"n_decode": nd, "n_tiles": nt, "max_kv": max_kv}
    if nd:
        items["dec_seq"], items["dec_tok"] = dev[:nd], dev[nd:2 * nd]
    if nt:
        o = 2 * nd
        items["tile_seq"], items["tile_tok"], items["tile_n"] = dev[o:o + nt], dev[o + nt:o + 2 * nt], dev[o + 2 * nt:]
    return items


@MIXERS.register("paged_attention")
class PagedAttention(Mixer):
    kernel_libraries = ("elementwise", "gemm", "attention")
    graph_safe = True      # its launches depend on device data and on sizes that are fixed per graph
    takes_post_norm = True     # forward(..., post_norm=(weight, eps)) norms the output rows before they join the stream
    TENSORS = {"q": "q_proj.weight", "k": "k_proj.weight", "v": "v_proj.weight", "o": "o_proj.weight",
               "q_bias": "q_proj.bias", "k_bias": "k_proj.bias", "v_bias": "v_proj.bias",
               "q_norm": "q_norm.", "k_norm": "k_norm.", "sink": "sinks", "gate": "gate_proj.weight"}

    def __init__(self, hidden_size: int, n_heads: int, n_kv_heads: int, head_dim: int, bias: bool,
                 position: PartSpec, window: int | None = None, scale: float | None = None,
                 qk_norm: PartSpec | None = None, v_dim: int | None = None, chunk: int | None = None,
                 names: dict | None = None, keep_first: int = 0, sink: bool = False, out_gate: bool = False,
                 own_kv: bool = True, retain: tuple | None = None, softcap: float | None = None,
                 distance_slopes=None, values_from_keys: bool = False, qk_norm_span: str = "head",
                 q_temperature: tuple | None = None, unit_values: float | None = None):
        """`qk_norm`: kind and arguments of a norm over head_dim; two of them are built, with tensors under
        `q_norm.` and `k_norm.`, and applied to every head of q and of k before the rotation.
        `v_dim`: size of a value head where it differs from head_dim (the size of a query and key head).
        `chunk`: a query at position p sees the keys t <= p of its own chunk only, floor(t / chunk) == floor(p / chunk),
        chunks counted from position 0 of the sequence.
        `names`: what the checkpoint calls this part's tensors, where that differs from `TENSORS` (the prefixes of
        the two norms among them).
        `keep_first` (with a window): the first so many keys of a sequence stay visible to every later query.
        `sink`: a learned logit per head ([n_heads]) joins the softmax's denominator; it has no key and no value.
        `out_gate`: the heads' outputs are multiplied by sigmoid(W_g x), x the mixer's input, before the output
        projection (W_g: [n_heads * v_dim, hidden]); "head": one gate per head, W_g: [n_heads, hidden].
        `q_temperature` = (coef, every): the query at position p is multiplied by 1 + coef ln(floor((p + 1) / every) + 1),
        which is how positions enter the scores of such a mixer (it rotates nothing).
        `unit_values` (an eps): every value head is divided by its root mean square over v_dim (eps inside the root,
        no weight) and cached so.
        `own_kv` False: the mixer has no key and value projections and writes no cache; its schedule entry reads
        the cache of an entry that has them (with these head counts and sizes).
        `retain` = (window or None, keep_first): how the pages of this mixer's cache group age, where that is not
        its own mask: the longest window and the most kept keys among the mixers that read the same cache.
        `softcap`: a scaled score s becomes softcap * tanh(s / softcap) before the softmax.
        `distance_slopes` (n_heads numbers): the score of key t for the query at position p then loses
        slope_h * (p - t); this is how positions enter the scores of a mixer that rotates nothing.
        `values_from_keys`: the mixer has no value projection; a key as projected (before any norm) is its value.
        `qk_norm_span` "projection": the norms of `qk_norm` run over all heads of q at once and over all heads of k at
        once (weights of n_heads * head_dim and n_kv_heads * head_dim elements) instead of over every head."""
        if n_heads % n_kv_heads:
            raise ValueError(f"n_heads {n_heads} is not a multiple of n_kv_heads {n_kv_heads}")
        # (the matrix-unit kernels take multiples of HEAD_DIM_STEP; other sizes run on the kernels for any shape)
        if not 1 <= head_dim <= limits.HEAD_DIM_MAX:
            raise ValueError(f"head_dim {head_dim}: the attention kernels take head sizes up to {limits.HEAD_DIM_MAX}")
        self.hidden_size, self.n_heads, self.n_kv_heads, self.head_dim = hidden_size, n_heads, n_kv_heads, head_dim
        self.bias = bool(bias)
        self.window = int(window) if window else None
        self.chunk = int(chunk) if chunk else None
        if self.window and self.chunk:
            raise ValueError("an attention layer has a sliding window or a chunked mask, not both")
        self.keep_first = int(keep_first or 0) if self.window else 0
        if self.keep_first < 0:
            raise ValueError(f"keep_first {keep_first} is negative")
        self.has_sink, self.out_gate, self.own_kv = bool(sink), bool(out_gate), bool(own_kv)
        self.gate_per_head = out_gate == "head"
        self.q_temperature = (float(q_temperature[0]), int(q_temperature[1])) if q_temperature else None
        if self.q_temperature and self.q_temperature[1] < 1:
            raise ValueError(f"a query temperature that steps every {q_temperature[1]} positions")
        self.unit_values = float(unit_values) if unit_values is not None else None
        # queries warmed by position or values of unit size: both are float32 arithmetic on the products' float32 rows,
        # done by the launch that writes the cache
        self.prepares = self.q_temperature is not None or self.unit_values is not None
        if self.prepares and (bias or qk_norm is not None or values_from_keys or not own_kv):
            raise ValueError("a query temperature and unit values go with projections of q, k and v without biases and head norms")
        if self.chunk and (retain is not None or keep_first):
            raise ValueError("kept first keys and a retention of their own go with a window, not with a chunked mask")
        # (None, 0): every key is kept; (W, F): the last W and the first F
        self.retain = (self.window, self.keep_first) if retain is None else (int(retain[0]) if retain[0] else None, int(retain[1] or 0))
        if self.retain[0] is not None and (self.window is None or self.window > self.retain[0] or self.keep_first > self.retain[1]):
            raise ValueError(f"a cache that keeps the last {self.retain[0]} and the first {self.retain[1]} keys does not hold "
                             f"what a window of {self.window} with {self.keep_first} kept keys sees")
        self.v_dim = int(v_dim) if v_dim else head_dim
        self.softcap = float(softcap) if softcap else 0.0
        if not 0.0 <= self.softcap < math.inf:
            raise ValueError(f"a cap of {softcap} on the scores")
        self.distance_slopes = tuple(float(x) for x in distance_slopes) if distance_slopes is not None else None
        if self.distance_slopes is not None and len(self.distance_slopes) != n_heads:
            raise ValueError(f"{len(self.distance_slopes)} distance slopes for {n_heads} heads")
        self.values_from_keys = bool(values_from_keys)
        if self.values_from_keys and (self.v_dim != head_dim or bias):
            raise ValueError("keys that are their own values have the values' size and no biases")
        if qk_norm_span not in ("head", "projection"):
            raise ValueError(f"qk_norm_span '{qk_norm_span}' is not 'head' or 'projection'")
        self.span_norms = qk_norm_span == "projection"
        if self.span_norms and qk_norm is None:
            raise ValueError("norms over the whole projection need `qk_norm`")
        if self.values_from_keys and not self.span_norms:
            raise ValueError("keys that are their own values come with norms over the whole projection here")
        if not 1 <= self.v_dim <= limits.HEAD_DIM_MAX:
            raise ValueError(f"v_dim {self.v_dim}: the attention kernels take up to {limits.HEAD_DIM_MAX}")
        self.names = dict(self.TENSORS, **(names or {}))
        self.scale = float(scale) if scale is not None else 1.0 / math.sqrt(head_dim)   # attention.rs:433
        if not 0.0 < self.scale < math.inf:
            raise ValueError(f"the scale of the attention scores must be positive and finite, got {self.scale}")
        self.position = POSITION_ENCODINGS.build(position)
        if not self.own_kv and (bias or (self.position.rotary() or Rotary(1, 1.0)).rotary_dim):
            raise ValueError("a mixer that reads another mixer's keys and values has neither biases nor a rotation here")
        self._position_prefix = position.prefix or ""       # where the encoding's own tensors (if any) are named
        self.qw, self.kvw, self.vw, self.ow = n_heads * head_dim, n_kv_heads * head_dim, n_kv_heads * self.v_dim, n_heads * self.v_dim
        if not self.own_kv:
            self.kvw = self.vw = 0       # (no rows of k and v in the mixer's matrix)
        if self.values_from_keys:
            self.vw = 0                  # (no rows of v: the key rows are the values)
        self.qkv = self.o_proj = self.sinks = self.slopes = None
        self.q_norm = self.k_norm = None
        if qk_norm is not None and self.span_norms:
            self.q_norm = NORMS.build(PartSpec(qk_norm.kind, dict(qk_norm.args, size=self.qw)))
            self.k_norm = NORMS.build(PartSpec(qk_norm.kind, dict(qk_norm.args, size=self.kvw))) if self.kvw else None
            if self.q_norm.rms_params() is None or (self.position.rotary() or Rotary(1, 1.0)).rotary_dim:
                raise ValueError("norms over the whole projection are RMS norms with a weight, under a mixer that rotates nothing")
        elif qk_norm is not None:
            self.q_norm, self.k_norm = (NORMS.build(PartSpec(qk_norm.kind, dict(qk_norm.args))) for _ in range(2))
        if self.prepares and (self.position.rotary() is None or self.position.rotary().rotary_dim):
            raise ValueError("a query temperature and unit values go with a mixer that rotates nothing")
        if (self.position.rotary() or Rotary(0, 1.0)).magnitude != 1.0:
            raise ValueError("this mixer's rotation kernels turn and do not stretch: a rotation's magnitude must be 1")
        if bias and out_gate:
            raise ValueError("an attention layer with an output gate has no biases here")

    def children(self):
        norms = [(self.names[n], p) for n, p in (("q_norm", self.q_norm), ("k_norm", self.k_norm)) if p is not None]
        return [(self._position_prefix, self.position)] + norms

    def param_specs(self):
        H, n = self.hidden_size, self.names
        specs = {n["q"]: ParamSpec((self.qw, H)), n["o"]: ParamSpec((H, self.ow))}
        if self.own_kv:
            specs[n["k"]] = ParamSpec((self.kvw, H))
            if not self.values_from_keys:
                specs[n["v"]] = ParamSpec((self.vw, H))
        if self.bias:
            specs.update({n["q_bias"]: ParamSpec((self.qw,)), n["k_bias"]: ParamSpec((self.kvw,)),
                          n["v_bias"]: ParamSpec((self.vw,))})
        if self.has_sink:
            specs[n["sink"]] = ParamSpec((self.n_heads,))
        if self.out_gate:
            specs[n["gate"]] = ParamSpec((self.n_heads if self.gate_per_head else self.ow, H))
        return specs

    def load(self, fetch):
        # one matrix: the rows of q, then (a mixer with projections of its own) of k and v, then of the output gate
        n = self.names
        rows = [fetch(n["q"])] + ([fetch(n["k"])] if self.own_kv else []) \
            + ([fetch(n["v"])] if self.own_kv and not self.values_from_keys else []) \
            + ([fetch(n["gate"])] if self.out_gate else [])
        w = torch.cat(same_dtype(rows), dim=0)
        b = None
        if self.bias:
            b = torch.cat(same_dtype([fetch(n["q_bias"]), fetch(n["k_bias"]), fetch(n["v_bias"])]), dim=0)
        self.qkv = Linear(w, b)
        self.o_proj = Linear(fetch(n["o"]))
        if self.has_sink:
            self.sinks = fetch(n["sink"]).float().contiguous()
        if self.distance_slopes is not None:
            self.slopes = torch.tensor(self.distance_slopes, dtype=torch.float64).to(torch.float32).to(w.device)

    def normed_spans_and_cache(self, x, ctx, table, cache):
        """As `normed_heads_and_cache` for norms over the whole projection: q [T, qw] normed over all its columns, the
        keys normed over all theirs into the key page and, where they are their own values, as projected into the
        value page, in one launch; returns q and the rest of the product (v, the output gate's rows)."""
        wq, eps = self.q_norm.rms_params()
        w = self.qkv.weight
        cut = self.qw + self.kvw
        qk = matmul(x, w[:cut], epilogue=ops.EPI_STORE_F32)
        rest = matmul(x, w[cut:]) if w.shape[0] > cut else None
        q = torch.empty((ctx.n_tokens, self.qw), dtype=ctx.act_dtype, device=qk.device)
        writes = self.own_kv and cache.writes
        if writes and not self.values_from_keys:
            raise ValueError("norms over the whole projection with a value projection of their own have no kernel yet")
        debug.region("rope + cache write")
        wk = self.k_norm.rms_params()[0] if self.k_norm is not None else None
        ops.span_norm_kv_write(qk, q, wq, wk, eps, ctx.positions, ctx.token_seq, table,
                               cache.pages["k"] if writes else None, cache.pages["v"] if writes else None,
                               self.n_heads, self.n_kv_heads, self.head_dim, cache.block_size)
        return q, rest

    def page_shapes(self, block_size: int) -> dict:
        return {"k": (self.n_kv_heads, block_size, self.head_dim),
                "v": (self.n_kv_heads, self.v_dim, block_size)}

    def cache_group(self):
        if self.chunk:      # pages age with the chunks: those of a chunk that has ended are given back
            return ("chunk", self.chunk), ("chunk", self.chunk)
        window, keep = self.retain
        if window and keep:      # the last `window` keys and the first `keep`
            return ("window", window, "keep", keep), ("keep", window, keep)
        return (("window", window), window) if window else (("full",), None)

    def forward_from_residual(self, norm, ctx, cache, residual) -> bool:
        """Few tokens: the norm is applied inside the q/k/v product (up to 16 rows it saves a launch; with
        more, every block's reading and norming of all rows costs more than the norm kernel)."""
        rms = norm.rms_params()
        # (heads that are normed again take their q and k from a float32 product; the norm inside two products, one
        # of them stored in float32, was measured and is behind the norm kernel: every block norms all rows)
        if (ctx.act_dtype != torch.bfloat16 or rms is None or residual.shape[0] > 16 or self.q_norm is not None
                or self.prepares or not self.own_kv or not ops.can_fuse_norm(residual, self.qkv.weight, residual.shape[0])):
            return False
        debug.region("qkv")
        qkv = ops.gemm(residual, self.qkv.weight, bias=self.qkv.bias, norm=rms)
        self.forward(None, ctx, cache, residual, qkv=qkv)
        return True

    def takes_scale_later(self, act_dtype) -> bool:
        """Whether forward takes an ops.ScaleLater as x (the block before then leaves its rows that way)."""
        w = self.qkv.weight
        return (self.q_norm is None and not self.prepares and self.own_kv and act_dtype == torch.bfloat16 and w.dtype == torch.bfloat16
                and w.shape[1] % 8 == 0 and w.data_ptr() % 16 == 0)

    def tile_queries(self, ctx, dtype, block_size: int) -> int:
        """Queries per work item of this step's prompt portions: 64, or 128 where the kernel takes that many (a block
        of eight waves then shares every tile of keys it brings in between twice as many queries).  The kernel gives
        a launch of no more blocks than the GPU has CUs (256) two groups of waves per block, which halves a block's chain of
        tiles; so: items of 64 while they number no more than the CUs; else items of 128 if those do (a 2,048-token
        portion deep in a prompt: 603 against 784 us at 16 heads); else items of 128 if they still number about
        one evenly loaded block per CU (blocks of a portion that starts a prompt differ in work up to the portion's
        length in keys and count by their mean share of the longest; +8-26 % from 448 such blocks on); else 64."""
        if ctx.recorded or self.v_dim != self.head_dim:      # (the kernels for unequal head sizes take items of 64)
            return 64
        widest = ops.attention_tile_queries(dtype, self.head_dim, block_size)
        if widest == 64:
            return 64
        cus = ops.compute_units(ctx.device)
        small = large = 0
        even_blocks = 0.0
        for s in range(ctx.n_seqs):
            n = ctx.q_starts[s + 1] - ctx.q_starts[s]
            if n > 1:
                before = ctx.kv_lens[s] - n
                small += -(-n // 64) * self.n_heads
                large += -(-n // widest) * self.n_heads
                even_blocks += -(-n // widest) * self.n_heads * (before + n / 2) / (before + n)
        if small <= cus:
            return 64
        return widest if large <= cus or even_blocks >= EVEN_BLOCKS_PER_CU * cus else 64

    def normed_heads(self, x, ctx):
        """q [T, qw], k [T, kvw] with every head normed, and the rest of the product, [T, vw (+ ow)]: v and the
        output gate's rows.  The q and k products are made in float32 (the norms read float32 rows), each head a
        row of a [T * (nh + nkv), head_dim] matrix that the norm kernels gather their rows from.  A mixer without
        projections of its own has no k and no v."""
        T, nh, hd = ctx.n_tokens, self.n_heads, self.head_dim
        nkv = self.n_kv_heads if self.own_kv else 0
        w, b = self.qkv.weight, self.qkv.bias
        cut = self.qw + self.kvw
        qk = matmul(x, w[:cut], bias=None if b is None else b[:cut], epilogue=ops.EPI_STORE_F32)
        v = matmul(x, w[cut:], bias=None if b is None else b[cut:]) if w.shape[0] > cut else None

        def head_rows():
            first = torch.arange(T, dtype=torch.int32, device=qk.device)[:, None] * (nh + nkv)
            heads = torch.arange(nh + nkv, dtype=torch.int32, device=qk.device)[None, :]
            rows = first + heads
            return rows[:, :nh].reshape(-1).contiguous(), rows[:, nh:].reshape(-1).contiguous()

        q_rows, k_rows = ctx.memo(f"head rows {nh} {nkv}", head_rows)
        heads = qk.view(T * (nh + nkv), hd)
        q = self.q_norm.forward(heads, ctx, rows=q_rows).view(T, self.qw)
        k = self.k_norm.forward(heads, ctx, rows=k_rows).view(T, self.kvw) if nkv else None
        return q, k, v

    def fuses_head_norms(self) -> bool:
        """Whether the heads' norms and the cache write are one launch: both norms of the RMS form (with or without
        a weight) under one eps, nothing rotated, no biases."""
        if not FUSE_HEAD_NORMS or self.q_norm is None or self.bias or self.head_dim > 256:
            return False
        rot = self.position.rotary()
        units = (self.q_norm.unit_params(), self.k_norm.unit_params())
        return rot is not None and rot.rotary_dim == 0 and None not in units and units[0][1] == units[1][1]

    def normed_heads_and_cache(self, x, ctx, table, cache):
        """As `normed_heads` for norms of the RMS form and no rotation, with the cache written by the same launch:
        returns q [T, qw] and the rest of the product (v, the output gate's rows)."""
        units = (self.q_norm.unit_params(), self.k_norm.unit_params())
        w = self.qkv.weight
        cut = self.qw + self.kvw
        qk = matmul(x, w[:cut], epilogue=ops.EPI_STORE_F32)
        rest = matmul(x, w[cut:]) if w.shape[0] > cut else None
        q = torch.empty((ctx.n_tokens, self.qw), dtype=ctx.act_dtype, device=qk.device)
        writes = self.own_kv and cache.writes
        debug.region("rope + cache write")
        ops.head_norm_kv_write(qk, q, rest[:, :self.vw] if writes else None, units[0][0], units[1][0], units[0][1],
                               ctx.positions, ctx.token_seq, table, cache.pages["k"] if writes else None,
                               cache.pages["v"] if writes else None, self.n_heads, self.n_kv_heads, self.head_dim,
                               cache.block_size, self.v_dim)
        return q, rest

    takes_fresh = True

    def forward(self, x, ctx, cache, residual, qkv=None, post_norm=None, out_scale: float | None = None, fresh: bool = False) -> None:
        """`out_scale`: a constant that the mixer's output is multiplied by on its way into the stream (a mixer that
        runs beside another one, the two weighted).  `fresh`: `residual` holds nothing yet; the output is stored into it."""
        table = ctx.block_tables[cache.group]
        k_pages, v_pages = cache.pages["k"], cache.pages["v"]
        rot = self.position.rotary()
        debug.region("qkv")
        fused = (qkv is None and self.q_norm is None and rot is not None and rot.frequencies is None and not self.prepares
                 and self.v_dim == self.head_dim and self.own_kv and not self.out_gate
                 and ops.can_qkv_rope(x, self.qkv.weight, ctx.n_tokens, self.head_dim, rot.rotary_dim, rot.interleaved))
        if fused:
            # few tokens: rotation and cache write happen in the product's epilogue
            qkv = ops.qkv_rope(x, self.qkv.weight, self.qkv.bias, ctx.positions, ctx.token_seq, table,
                               k_pages if cache.writes else None, v_pages if cache.writes else None,
                               self.n_heads, self.n_kv_heads, self.head_dim, cache.block_size, rot.rotary_dim, rot.theta,
                               rot.freq_factors)
            q = qkv[:, :self.qw]
        else:
            gate = None
            wrote = False
            if self.prepares:
                # one float32 product, then one launch: q times its position's temperature, the gate's columns behind
                # it, k into its page, v (of unit size) into its page
                n_gate = (self.n_heads if self.gate_per_head else self.ow) if self.out_gate else 0
                rows = matmul(x, self.qkv.weight, epilogue=ops.EPI_STORE_F32)
                qkv = torch.empty((ctx.n_tokens, self.qw + n_gate), dtype=ctx.act_dtype, device=rows.device)
                debug.region("rope + cache write")
                ops.temp_unit_kv_write(rows, qkv, ctx.positions, ctx.token_seq, table, k_pages if cache.writes else None,
                                       v_pages if cache.writes else None, self.n_heads, self.n_kv_heads, self.head_dim,
                                       self.v_dim, cache.block_size, n_gate=n_gate, temperature=self.q_temperature,
                                       unit_values=self.unit_values is not None, eps=self.unit_values or 0.0)
                q, k, v, wrote = qkv[:, :self.qw], None, None, True
                if n_gate:
                    gate = qkv[:, self.qw:]
            elif self.q_norm is not None:           # every head of q and k through its norm, between bias and rotation
                if self.span_norms:
                    q, rest = self.normed_spans_and_cache(x, ctx, table, cache)
                    k, wrote = None, True
                elif self.fuses_head_norms():
                    # RMS norms and no rotation: one launch norms the heads and writes q, k's and v's pages
                    q, rest = self.normed_heads_and_cache(x, ctx, table, cache)
                    k, wrote = None, True
                else:
                    q, k, rest = self.normed_heads(x, ctx)
                qkv = q
                v = rest[:, :self.vw] if rest is not None else None
                if self.out_gate:
                    gate = rest[:, self.vw:]
            else:
                if qkv is None:
                    if isinstance(x, ops.ScaleLater):     # rows of a norm whose scale the product applies
                        qkv = ops.gemm(x.x, self.qkv.weight, bias=self.qkv.bias, row_ss=(x.ss, x.eps))
                    else:
                        qkv = self.qkv(x)
                cut = self.qw + self.kvw
                q, k, v = qkv[:, :self.qw], qkv[:, self.qw:cut], qkv[:, cut:cut + self.vw]
                if self.out_gate:
                    gate = qkv[:, cut + self.vw:]
            debug.region("rope + cache write")
            if self.own_kv and not wrote:       # (a mixer without keys of its own has no rotation either: nothing to do for its q)
                if rot is None:
                    self.position.apply(q, k, ctx)
                    rot = NO_ROTATION
                ops.rope_kv_write(q, k, v, ctx.positions, ctx.token_seq, table,
                                  k_pages if cache.writes else None, v_pages if cache.writes else None,
                                  self.n_heads, self.n_kv_heads, self.head_dim, cache.block_size, rot.rotary_dim, rot.theta,
                                  rot.interleaved, rot.freq_factors, frequencies=rot.frequencies, v_dim=self.v_dim)
        debug.region("attention")
        out = torch.empty((ctx.n_tokens, self.ow), dtype=qkv.dtype, device=qkv.device)
        tile_q = ctx.memo(f"attention tile {self.n_heads} {self.head_dim} {self.v_dim} {cache.block_size} {q.dtype}",
                          lambda: self.tile_queries(ctx, q.dtype, cache.block_size))
        items = ctx.memo(f"attention_items {tile_q}", lambda: attention_items(ctx, tile_q))
        common = (self.n_heads, self.n_kv_heads, self.head_dim, cache.block_size, self.window, self.scale)
        # (the gate multiplies the heads' outputs as the attention kernels write them)
        mask = dict(mask_chunk=self.chunk or 0, v_dim=self.v_dim, keep_first=self.keep_first, sinks=self.sinks,
                    gate=None if fused else gate, softcap=self.softcap, slopes=self.slopes,
                    gate_per_head=self.gate_per_head and gate is not None)
        if items["n_tiles"]:
            ops.attention_tiles(q, out, k_pages, v_pages, table, ctx.positions,
                                items["tile_seq"], items["tile_tok"], items["tile_n"], *common, tile_q=tile_q, **mask)
        if items["n_decode"]:
            ops.attention_decode(q, out, k_pages, v_pages, table, ctx.positions,
                                 items["dec_seq"], items["dec_tok"], *common, max_kv_len=items["max_kv"], **mask)
        debug.region("o_proj")
        if post_norm is None and fresh and (out_scale is None or out_scale == 1.0):
            self.o_proj(out, epilogue=ops.EPI_STORE_F32, out=residual)
        elif post_norm is None:
            if fresh:
                ops.fill_u32(residual, 0)
            scale = ops.constant_rows(out.device, out_scale, ctx.n_tokens) if out_scale is not None and out_scale != 1.0 else None
            self.o_proj(out, epilogue=ops.EPI_RESID, out=residual, row_scale=scale)
        else:       # the output rows are normed before they join the stream: float32 rows, then one kernel norms and adds
            ops.rmsnorm_add(residual, self.o_proj(out, epilogue=ops.EPI_STORE_F32), post_norm[0], post_norm[1])
