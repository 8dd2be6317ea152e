"""Latent attention: queries, keys and values go through low-rank latents, and only the keys' and values' latent is
kept in the cache.

Per token, with h the mixer's input row, H heads, D unrotated and P rotated query/key dimensions a head, value heads
of V, latents of Rq (queries) and R (keys and values):
    c_q = N(W_dq h),  q = W_uq c_q                                  q: per head [D unrotated | P rotated]
    (c', kr') = W_dkv h,  c = N(c') [R],  kr = rot(kr') [P]          kr: one rotated key part for all heads
    k_h = (W_uk,h c | kr),  v_h = W_uv,h c
    score_h(t) = (q_h[:D] . W_uk,h c_t + rot(q_h[D:]) . kr_t) * scale
    y = W_o concat_h( sum_t p_h(t) W_uv,h c_t )                      p: softmax over the window, optionally with a sink
The cache holds (c | kr) per position and nothing per head.  The kernels never make k_h and v_h: since
q_h[:D] . W_uk,h c = (W_uk,h^T W_uq,h[:D] c_q) . c, the queries' up-projection is multiplied with the transposes of the
heads' key up-projections once, when the weights are loaded (in float32, then kept in the weights' type), and one
product takes c_q to H query heads of [R absorbed | P to be rotated]; the attention kernels then see H query heads of
R + P dimensions over ONE key head (c | kr) whose values are c; the heads' outputs, sums of latents, go through
W_uv,h afterwards (one grouped launch in which a head is a group of rows).  A mixer with `own_kv` False has no W_dkv: its schedule entry reads
the cache of a layer that has one, with W_uk, W_uv, queries, mask and sink of its own.
"""
from __future__ import annotations

import math

import torch

from .. import debug, limits, ops
from .attention import attention_items
from .base import MIXERS, NORMS, POSITION_ENCODINGS, Mixer, ParamSpec, PartSpec
from .linear import Linear, matmul

_head_groups: dict = {}


def head_groups(device, n_tokens: int, n_heads: int):
    """(rows, offsets) for a product in which head h of every token is a group of its own: the matrix of T tokens x
    H heads is seen as T*H rows (row t*H + h), `rows` lists them head by head and `offsets` [H + 1] says where each
    head's rows begin.  They depend on the two sizes alone and are kept for the life of the process (recorded steps
    hold their addresses)."""
    key = (torch.device(device), int(n_tokens), int(n_heads))
    if key not in _head_groups:
        t = torch.arange(n_tokens, dtype=torch.int32)[None, :] * n_heads + torch.arange(n_heads, dtype=torch.int32)[:, None]
        off = torch.arange(n_heads + 1, dtype=torch.int32) * n_tokens
        _head_groups[key] = (t.reshape(-1).contiguous().to(device), off.to(device))
        if len(_head_groups) > 4096:       # (prompt portions of many lengths: the oldest tables go; recorded sizes are few)
            _head_groups.pop(next(iter(_head_groups)))
    return _head_groups[key]


@MIXERS.register("latent_attention")
class LatentAttention(Mixer):
    kernel_libraries = ("elementwise", "gemm", "attention")
    graph_safe = True
    TENSORS = {"dq": "dq", "dq_norm": "dq.", "uq": "uq", "dkv": "dkv", "dkv_norm": "dkv.", "uk": "uk", "uv": "uv",
               "sink": "sink", "o": "o"}

    def __init__(self, hidden_size: int, n_heads: int, head_dim: int, rot_dim: int, v_dim: int, q_rank: int, kv_rank: int,
                 latent_norm: PartSpec, position: PartSpec, scale: float, window: int | None = None, sink: bool = False,
                 own_kv: bool = True, retain_window: int | None = None, names: dict | None = None):
        """`head_dim`: unrotated query/key dimensions a head; `rot_dim`: rotated ones (the shared key part's size).
        `latent_norm`: kind and arguments of the norm over a latent (`size` is set here: q_rank, kv_rank); it must be
        an RMS norm with a weight.  `position`: the rotation of the rot_dim part (a `Rotary`, adjacent pairs).
        `scale`: of the scores, as given.  `window`: a query at p sees the keys t with 0 <= p - t < window.
        `own_kv` False: no W_dkv; the schedule entry reads another entry's cache.  `retain_window`: how the pages of
        the cache group age where that is not this mixer's own window (the widest among the mixers that read the
        cache; 0 or None with `window` None: nothing is given back)."""
        self.hidden_size, self.n_heads = int(hidden_size), int(n_heads)
        self.head_dim, self.rot_dim, self.v_dim = int(head_dim), int(rot_dim), int(v_dim)
        self.q_rank, self.kv_rank = int(q_rank), int(kv_rank)
        if min(self.n_heads, self.head_dim, self.v_dim, self.q_rank, self.kv_rank) < 1 or self.rot_dim < 0:
            raise ValueError("latent attention: heads, sizes and ranks are positive")
        self.key_width = self.kv_rank + self.rot_dim          # what the attention kernels see as the one key head
        # (up to HEAD_DIM_MAX on the matrix units; wider, on the kernels for any shape)
        if self.key_width > limits.HEAD_DIM_MAX_ANY:
            raise ValueError(f"latent attention: kv_rank {kv_rank} + rot_dim {rot_dim} is more than the attention kernels' "
                             f"{limits.HEAD_DIM_MAX_ANY}")
        self.scale = float(scale)
        if not 0.0 < self.scale < math.inf:
            raise ValueError(f"the scale of the attention scores must be positive and finite, got {self.scale}")
        self.window = int(window) if window else None
        self.retain_window = self.window if retain_window is None else (int(retain_window) or None)
        if self.retain_window is not None and (self.window is None or self.window > self.retain_window):
            raise ValueError(f"a cache that keeps the last {self.retain_window} keys does not hold what a window of {self.window} sees")
        self.has_sink, self.own_kv = bool(sink), bool(own_kv)
        self.names = dict(self.TENSORS, **(names or {}))
        self.position = POSITION_ENCODINGS.build(position)
        rot = self.position.rotary()
        if rot is None or (rot.rotary_dim and not rot.interleaved) or rot.rotary_dim > self.rot_dim or rot.freq_factors is not None:
            raise ValueError("latent attention rotates adjacent pairs of its rotated part with a rotation the kernels apply")
        self.rot = rot
        self.q_norm = NORMS.build(PartSpec(latent_norm.kind, dict(latent_norm.args, size=self.q_rank)))
        self.kv_norm = NORMS.build(PartSpec(latent_norm.kind, dict(latent_norm.args, size=self.kv_rank))) if self.own_kv else None
        if self.q_norm.rms_params() is None:
            raise ValueError("latent attention norms its latents with an RMS norm that has a weight")
        self.q_width = self.n_heads * (self.head_dim + self.rot_dim)
        self.down = self.up_q = self.uv = self.o_proj = self.sinks = self.inv_freq = None

    def children(self):
        n = self.names
        return [(n["dq_norm"], self.q_norm)] + ([(n["dkv_norm"], self.kv_norm)] if self.own_kv else [])

    def param_specs(self):
        W, n, H = self.hidden_size, self.names, self.n_heads
        specs = {n["dq"]: ParamSpec((self.q_rank, W)), n["uq"]: ParamSpec((self.q_width, self.q_rank)),
                 n["uk"]: ParamSpec((H * self.head_dim, self.kv_rank)), n["uv"]: ParamSpec((H * self.v_dim, self.kv_rank)),
                 n["o"]: ParamSpec((W, H * self.v_dim))}
        if self.own_kv:
            specs[n["dkv"]] = ParamSpec((self.key_width, W))
        if self.has_sink:
            specs[n["sink"]] = ParamSpec((H,))
        return specs

    def load(self, fetch):
        n, H = self.names, self.n_heads
        # one matrix makes both down-projections: the rows of W_dq, then (a mixer with keys of its own) of W_dkv
        self.down = torch.cat([fetch(n["dq"])] + ([fetch(n["dkv"])] if self.own_kv else []), dim=0).contiguous()
        # per head, rows [R: W_uk,h^T W_uq,h[:D] | P: W_uq,h[D:]]: c_q goes straight to what the attention kernels read
        D, P, R = self.head_dim, self.rot_dim, self.kv_rank
        uq = fetch(n["uq"]).view(H, D + P, self.q_rank)
        uk_t = fetch(n["uk"]).view(H, D, R).transpose(1, 2)
        absorbed = torch.bmm(uk_t.float(), uq[:, :D].float()).to(uq.dtype)                  # [H, R, q_rank]
        self.up_q = Linear(torch.cat([absorbed, uq[:, D:]], dim=1).reshape(H * (R + P), self.q_rank).contiguous())
        self.uv = fetch(n["uv"]).view(H, self.v_dim, self.kv_rank).contiguous()
        self.o_proj = Linear(fetch(n["o"]))
        if self.has_sink:
            self.sinks = fetch(n["sink"]).float().contiguous()
        self.inv_freq = ops.rotary_frequencies(self.down.device, self.rot.rotary_dim, self.rot.theta, self.rot.frequencies)

    # what the attention kernels see: one key head of kv_rank + rot_dim, values of kv_rank
    def page_shapes(self, block_size: int) -> dict:
        return {"k": (1, block_size, self.key_width), "v": (1, self.kv_rank, block_size)}

    def cache_group(self):
        w = self.retain_window
        return (("window", w), w) if w else (("full",), None)

    def forward(self, x, ctx, cache, residual, out_scale: float | None = None) -> None:
        T, H, D, P, R, V = ctx.n_tokens, self.n_heads, self.head_dim, self.rot_dim, self.kv_rank, self.v_dim
        table = ctx.block_tables[cache.group]
        k_pages, v_pages = cache.pages["k"], cache.pages["v"]
        debug.region("latent down")
        down = matmul(x, self.down, epilogue=ops.EPI_STORE_F32)          # float32: the norms read it
        wq, eps = self.q_norm.rms_params()
        if self.own_kv and cache.writes:
            # one launch: the keys' latent normed, the shared key part rotated, both written; the queries' latent normed
            debug.region("rope + cache write")
            wkv, eps_kv = self.kv_norm.rms_params()
            fused = wq.dtype == wkv.dtype and k_pages.dtype == ctx.act_dtype
            c_q = ops.latent_kv_write(down[:, self.q_rank:], wkv, eps_kv, ctx.positions, ctx.token_seq, table, k_pages, v_pages,
                                      R, P, self.rot.rotary_dim, cache.block_size, self.inv_freq, self.rot.magnitude,
                                      q_latent=(down, wq, eps) if fused else None)
            if not fused:
                c_q = ops.rmsnorm(down, wq, eps, ctx.act_dtype, width=self.q_rank)
        else:
            c_q = ops.rmsnorm(down, wq, eps, ctx.act_dtype, width=self.q_rank)
        debug.region("latent up")
        q_lat = self.up_q(c_q)                                            # [T, H * (R + P)]: absorbed parts, parts to rotate
        q = q_lat
        if self.rot.rotary_dim:                                           # (in place: a pair is read and written by one thread)
            ops.latent_q_rot(q_lat, q_lat, ctx.positions, H, R, P, self.rot.rotary_dim, R, self.inv_freq, self.rot.magnitude)
        debug.region("attention")
        out = torch.empty((T, H * R), dtype=q.dtype, device=q.device)
        items = ctx.memo("attention_items 64", lambda: attention_items(ctx, 64))
        common = (H, 1, R + P, cache.block_size, self.window, self.scale)
        extras = dict(v_dim=R, sinks=self.sinks)
        if items["n_tiles"]:
            ops.attention_tiles(q_lat, out, k_pages, v_pages, table, ctx.positions, items["tile_seq"], items["tile_tok"],
                                items["tile_n"], *common, tile_q=64, **extras)
        if items["n_decode"]:
            ops.attention_decode(q_lat, out, k_pages, v_pages, table, ctx.positions, items["dec_seq"], items["dec_tok"],
                                 *common, max_kv_len=items["max_kv"], **extras)
        debug.region("latent values")
        heads = torch.empty((T, H * V), dtype=q.dtype, device=q.device)
        rows, offsets = head_groups(q.device, T, H)
        # head h of token t: row t*H + h of [T*H, R] and of [T*H, V]
        ops.gemm(out.view(T * H, R), self.uv, a_rows=rows, c_rows=rows, expert_offsets=offsets, n_rows=T * H,
                 out=heads.view(T * H, V))
        debug.region("o_proj")
        scale = ops.constant_rows(heads.device, out_scale, T) if out_scale is not None and out_scale != 1.0 else None
        self.o_proj(heads, epilogue=ops.EPI_RESID, out=residual, row_scale=scale)
