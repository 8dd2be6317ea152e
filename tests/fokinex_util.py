"""Helpers of the Fokinex tests: small configurations, weights made in the test, and the comparison of the
engine's logits with the plain model (`plain_fokinex`)."""
from __future__ import annotations

import torch

import plain_fokinex as plain
from rafilix_util import random_tokens, row_errors, run_schedule, write_model  # noqa: F401  (schedules and files are alike)


def latent_layer(heads=4, dim=16, rot_dim=8, vdim=24, q_rank=20, kv_rank=32, window=24, scale=0.3, rot_dims=None,
                 base=10000.0, scaling=None, kv_from=None, mlp=None):
    """`rot_dims` None: all of rot_dim is rotated; 0: no rotation at all."""
    mixer = {"heads": heads, "dim": dim, "rot_dim": rot_dim, "vdim": vdim, "q_rank": q_rank, "kv_rank": kv_rank, "scale": scale}
    dims = rot_dim if rot_dims is None else rot_dims
    if dims:
        mixer["rot"] = {"base": base, "dims": dims}
        if scaling:
            mixer["rot"]["scaling"] = dict(zip(("factor", "original", "fast", "slow"), scaling))
    if window:
        mixer["mask"] = {"size": window}
    if kv_from is not None:
        mixer["kv_from"] = kv_from
    return {"type": "latent_attention", "mixer": mixer, "mlp": mlp}


def parallel_layer(heads=4, kv_heads=2, dim=16, window=12, scale=0.4, softcap=15.0, r_heads=4, r_kv_heads=2, r_dim=16,
                   r_vdim=24, conv=3, left_scale=0.8, right_scale=1.4, mlp=None):
    left = {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": dim, "scale": scale}
    if softcap:
        left["softcap"] = softcap
    if window:
        left["mask"] = {"size": window}
    right = {"heads": r_heads, "kv_heads": r_kv_heads, "dim": r_dim, "vdim": r_vdim, "conv": conv}
    return {"type": "parallel", "mixer": {"left": left, "right": right, "left_scale": left_scale, "right_scale": right_scale},
            "mlp": mlp}


def dense(ff=48):
    return {"kind": "dense", "ff": ff}


def config(layers, width=64, vocab=160, eps=1e-6, emb_scale=2.5):
    out = {"architecture": "Fokinex", "vocab": vocab, "width": width, "norm": {"eps": eps}, "layers": layers}
    if emb_scale is not None:
        out["embedding"] = {"scale": emb_scale}
    return out


STRETCH = (3.0, 40, 4.0, 0.5)        # (factor, original, fast, slow): with base 100 and 8 rotated dimensions all three bands occur

# Layers unlike each other: latent attention with stretched and plain frequencies, with fewer rotated dimensions than the
# rotated part has, with none, without a mask, readers of another layer's latents whose window is wider and narrower
# than the owner's; side-by-side layers with and without a cap, with equal and unequal head counts on either side, taps
# from 2 to 5; layers without a feed-forward.
CFG_MAIN = config([
    latent_layer(heads=4, dim=16, rot_dim=8, vdim=24, q_rank=20, kv_rank=32, window=20, scale=0.35, base=100.0, scaling=STRETCH, mlp=dense(48)),
    parallel_layer(heads=4, kv_heads=2, dim=16, window=13, scale=0.4, softcap=4.0, r_heads=4, r_kv_heads=2, r_dim=16, r_vdim=24, conv=4,
                   left_scale=0.8, right_scale=1.4, mlp=dense(40)),
    latent_layer(heads=2, dim=24, rot_dim=8, vdim=16, q_rank=12, kv_rank=32, window=37, scale=0.3, base=100.0, scaling=STRETCH, kv_from=0, mlp=None),
    latent_layer(heads=3, dim=8, rot_dim=12, vdim=8, q_rank=24, kv_rank=20, window=0, scale=0.4, rot_dims=4, base=50.0, mlp=dense(24)),
    latent_layer(heads=6, dim=16, rot_dim=12, vdim=16, q_rank=16, kv_rank=20, window=9, scale=0.5, rot_dims=4, base=50.0, kv_from=3, mlp=dense(16)),
    parallel_layer(heads=2, kv_heads=2, dim=24, window=0, scale=0.3, softcap=None, r_heads=3, r_kv_heads=3, r_dim=8, r_vdim=8, conv=2,
                   left_scale=1.0, right_scale=0.6, mlp=None),
    latent_layer(heads=2, dim=16, rot_dim=0, vdim=16, q_rank=16, kv_rank=16, window=11, scale=0.5, kv_from=None, mlp=dense(24)),
], width=64, vocab=160)
# bfloat16 on the matrix units: sizes in multiples of 16, widths in multiples of 64
CFG_MFMA = config([
    latent_layer(heads=4, dim=32, rot_dim=16, vdim=32, q_rank=64, kv_rank=64, window=70, scale=0.2, base=1000.0, scaling=(2.0, 64, 8.0, 1.0), mlp=dense(128)),
    parallel_layer(heads=4, kv_heads=2, dim=64, window=100, scale=0.2, softcap=10.0, r_heads=4, r_kv_heads=2, r_dim=32, r_vdim=64, conv=4,
                   left_scale=1.1, right_scale=0.7, mlp=dense(128)),
    latent_layer(heads=2, dim=64, rot_dim=16, vdim=64, q_rank=32, kv_rank=64, window=150, scale=0.15, base=1000.0, scaling=(2.0, 64, 8.0, 1.0), kv_from=0, mlp=dense(64)),
    parallel_layer(heads=2, kv_heads=1, dim=128, window=33, scale=0.15, softcap=None, r_heads=2, r_kv_heads=1, r_dim=64, r_vdim=64, conv=3,
                   left_scale=0.9, right_scale=1.0, mlp=None),
], width=128, vocab=256)


def tensor_shapes(cfg: dict) -> dict:
    """Names and shapes of a model's tensors, from its configuration."""
    W = cfg["width"]
    out = {"embed": (cfg["vocab"], W), "final.norm": (W,), "head": (cfg["vocab"], W)}
    for i, layer in enumerate(cfg["layers"]):
        p, m = f"l{i}.", layer["mixer"]
        out[p + "norm1"] = (W,)
        if layer["type"] == "latent_attention":
            H, D, P, V, Rq, R = m["heads"], m["dim"], m["rot_dim"], m["vdim"], m["q_rank"], m["kv_rank"]
            out.update({p + "mix.dq": (Rq, W), p + "mix.dq.norm": (Rq,), p + "mix.uq": (H * (D + P), Rq),
                        p + "mix.uk": (H * D, R), p + "mix.uv": (H * V, R), p + "mix.sink": (H,), p + "mix.o": (W, H * V)})
            if m.get("kv_from") is None:
                out.update({p + "mix.dkv": (R + P, W), p + "mix.dkv.norm": (R,)})
        else:
            a, b = m["left"], m["right"]
            q = p + "mix.left."
            out.update({q + "q": (a["heads"] * a["dim"], W), q + "k": (a["kv_heads"] * a["dim"], W),
                        q + "q.norm": (a["heads"] * a["dim"],), q + "k.norm": (a["kv_heads"] * a["dim"],),
                        q + "g": (a["heads"] * a["vdim"], W), q + "o": (W, a["heads"] * a["vdim"])})
            q = p + "mix.right."
            H, G, D, V, t = b["heads"], b["kv_heads"], b["dim"], b["vdim"], b["conv"]
            out.update({q + "q": (G * D, W), q + "q.conv": (G * D, t), q + "k": (G * D, W), q + "k.conv": (G * D, t),
                        q + "v": (H * V, W), q + "v.conv": (H * V, t), q + "b": (H, W), q + "A_log": (H,), q + "norm": (V,),
                        q + "a": (H, W), q + "dt_bias": (H,), q + "g": (H * V, W), q + "o": (W, H * V)})
        if layer.get("mlp"):
            ff = layer["mlp"]["ff"]
            out.update({p + "mlp.gate": (ff, W), p + "mlp.up": (ff, W), p + "mlp.down": (W, ff)})
    return out


def make_weights(cfg: dict, seed: int) -> dict:
    """Random weights, bfloat16 values, of a size that keeps every sublayer's output of order one: a missing key,
    a sink that is left out, a lost state or a wrong window then moves the logits."""
    gen = torch.Generator().manual_seed(seed)
    out = {}
    for name, shape in tensor_shapes(cfg).items():
        last = name.split(".")[-1]
        if last in ("norm", "norm1"):
            t = 1.0 + 0.2 * torch.randn(shape, generator=gen)
        elif last == "sink":
            t = 1.0 + torch.randn(shape, generator=gen)
        elif last == "A_log":
            t = -2.0 + 0.5 * torch.randn(shape, generator=gen)       # decays of 0.8 to 0.97: tens of tokens are remembered
        elif last == "dt_bias":
            t = 0.5 * torch.randn(shape, generator=gen)
        elif last == "conv":
            t = torch.randn(shape, generator=gen) / shape[-1] ** 0.5
        elif name == "embed":
            t = torch.randn(shape, generator=gen) / cfg.get("embedding", {}).get("scale", 1.0)
        else:
            t = 1.3 * torch.randn(shape, generator=gen) / shape[-1] ** 0.5
        out[name] = t.to(torch.bfloat16)
    return out


# (bfloat16: a layer of this design adds two sublayers' outputs, made from one normed row, to the stream at once, and
# its latents are few numbers that every head reads; the roundings of seven such layers reach 0.05 to 0.08 of a row's
# spread at single positions, the same position whatever the cut or the batch, and which position it is changes with
# the order of the roundings (random configurations of real layer sizes stay below 0.08 too).  float32 is the sharp
# test.  EDGE_LIMIT: for models with peaked softmaxes, whose rounding errors are larger, and for one engine run
# against another.)
LIMIT = {"float32": 3e-5, "bfloat16": 1e-1}
EDGE_LIMIT = {"float32": 6e-5, "bfloat16": 1.2e-1}


def check_against_plain(cfg, weights, requests, got, dtype, what="", limit=None):
    """Every position of every request against the plain model."""
    limit = limit or LIMIT[dtype]
    worst = 0.0
    for r, tokens in requests.items():
        want = plain.forward(cfg, weights, tokens)
        err = row_errors(got[r], want)
        i = int(err.argmax())
        assert float(err[i]) <= limit, (f"{what} request {r}: position {i} of {len(tokens)} is off by {float(err[i]):.3g} "
                                        f"(limit {limit:g}); first position over it: {int((err > limit).nonzero()[0])}")
        worst = max(worst, float(err[i]))
    return worst


def changed(cfg: dict, layer: int, **mixer_changes) -> dict:
    """The configuration with keys of one layer's mixer replaced (a dotted key reaches into 'left' or 'right')."""
    import copy
    out = copy.deepcopy(cfg)
    for key, value in mixer_changes.items():
        at = out["layers"][layer]["mixer"]
        parts = key.split("__")
        for part in parts[:-1]:
            at = at[part]
        if value is None:
            at.pop(parts[-1], None)
        else:
            at[parts[-1]] = value
    return out
