"""Helpers of the Panarax tests: small configurations, weights made in the test, and the comparison of the
engine's logits with the plain model (`plain_panarax`)."""
from __future__ import annotations

import torch

import plain_panarax as plain
from rafilix_util import random_tokens, row_errors, run_schedule, write_model  # noqa: F401  (schedules and files are alike)


def rglru_layer(width=48, blocks=3, conv=3, mlp=None):
    return {"type": "rglru", "mixer": {"width": width, "blocks": blocks, "conv": conv}, "mlp": mlp}


def lightning_layer(heads=3, dim=8, vdim=12, decay=None, mlp=None):
    decay = decay or [0.55 + 0.44 * h / max(1, heads - 1) for h in range(heads)]
    return {"type": "lightning", "mixer": {"heads": heads, "dim": dim, "vdim": vdim, "decay": list(decay)}, "mlp": mlp}


def parallel_layer(heads=4, kv_heads=2, dim=8, vdim=12, scale=0.5, coef=0.4, every=7, r_heads=3, r_dim=8, r_vdim=12,
                   gate_cap=10.0, mlp=None):
    left = {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim, "scale": scale}
    if every:
        left["q_temp"] = {"coef": coef, "every": every}
    right = {"heads": r_heads, "dim": r_dim, "vdim": r_vdim, "gate_cap": gate_cap}
    return {"type": "parallel", "mixer": {"left": left, "right": right}, "mlp": mlp}


def dense(ff=40):
    return {"kind": "dense", "ff": ff}


def moe(experts=6, top=2, ff=16, limit=1.5):
    return {"kind": "moe", "expert": {"ff": ff, "limit": limit}, "router": {"experts": experts, "top": top}}


def config(layers, width=48, vocab=150, eps=1e-5, taps=3, max_positions=512):
    out = {"architecture": "Panarax", "vocab": vocab, "width": width, "max_positions": max_positions, "norm": {"eps": eps},
           "layers": layers}
    if taps:
        out["canon"] = {"taps": taps}
    return out


# Layers unlike each other, in an order of their own: every mixer twice with other sizes, experts chosen one, two and
# three at a time, a layer without a feed-forward, heads that share key heads and heads that do not, a head whose
# state never decays, temperature steps of 5 and 16 positions.
CFG_MAIN = config([
    parallel_layer(heads=4, kv_heads=2, dim=8, vdim=12, scale=0.5, coef=0.4, every=5, r_heads=3, r_dim=8, r_vdim=12, gate_cap=10.0,
                   mlp=moe(6, 2, 16, 1.5)),
    rglru_layer(width=40, blocks=5, conv=2, mlp=dense(40)),
    lightning_layer(heads=3, dim=8, vdim=12, decay=[0.6, 0.93, 1.0], mlp=moe(5, 3, 24, 0.8)),
    parallel_layer(heads=3, kv_heads=3, dim=12, vdim=8, scale=0.35, coef=0.9, every=16, r_heads=2, r_dim=12, r_vdim=20, gate_cap=6.0,
                   mlp=None),
    rglru_layer(width=64, blocks=2, conv=4, mlp=moe(4, 1, 32, 3.0)),
    lightning_layer(heads=2, dim=16, vdim=8, decay=[0.97, 0.8], mlp=dense(24)),
], width=48, vocab=150, taps=3)
# bfloat16 on the matrix units: sizes in multiples of 16, widths in multiples of 64
CFG_MFMA = config([
    lightning_layer(heads=4, dim=32, vdim=64, decay=[0.7, 0.9, 0.98, 0.999], mlp=moe(8, 2, 64, 2.5)),
    parallel_layer(heads=4, kv_heads=2, dim=64, vdim=64, scale=0.2, coef=0.3, every=100, r_heads=2, r_dim=32, r_vdim=64, gate_cap=12.0,
                   mlp=dense(128)),
    rglru_layer(width=192, blocks=3, conv=4, mlp=moe(8, 1, 64, 2.0)),
    parallel_layer(heads=2, kv_heads=1, dim=128, vdim=128, scale=0.1, coef=0.2, every=64, r_heads=2, r_dim=64, r_vdim=32, gate_cap=8.0,
                   mlp=dense(64)),
], width=128, vocab=256, taps=4, max_positions=1024)


def tensor_shapes(cfg: dict) -> dict:
    """Names and shapes of a model's tensors, from its configuration."""
    W = cfg["width"]
    out = {"embed": (cfg["vocab"], W), "pos": (cfg["max_positions"], W), "final.norm": (W,), "final.norm.b": (W,)}
    for i, layer in enumerate(cfg["layers"]):
        p, m = f"l{i}.", layer["mixer"]
        out.update({p + "norm1": (W,), p + "norm1.b": (W,), p + "rg1": (W, W), p + "rg1.b": (W,)})
        if cfg.get("canon"):
            out[p + "canon1"] = (W, cfg["canon"]["taps"])
        q = p + "mix."
        if layer["type"] == "rglru":
            C, B = m["width"], m["blocks"]
            out.update({q + "y": (C, W), q + "y.b": (C,), q + "x": (C, W), q + "x.b": (C,), q + "conv": (C, m["conv"]),
                        q + "conv.b": (C,), q + "ra": (B, C // B, C // B), q + "ra.b": (B, C // B), q + "ri": (B, C // B, C // B),
                        q + "ri.b": (B, C // B), q + "lam": (C,), q + "o": (W, C)})
        elif layer["type"] == "lightning":
            H, D, V = m["heads"], m["dim"], m["vdim"]
            out.update({q + "q": (H * D, W), q + "k": (H * D, W), q + "v": (H * V, W), q + "g": (H * V, W), q + "norm": (H * V,),
                        q + "o": (W, H * V)})
        else:
            a, b = m["left"], m["right"]
            out.update({q + "left.q": (a["heads"] * a["dim"], W), q + "left.k": (a["kv_heads"] * a["dim"], W),
                        q + "left.v": (a["kv_heads"] * a["vdim"], W), q + "left.g": (a["heads"], W),
                        q + "left.o": (W, a["heads"] * a["vdim"]), q + "left.out": (W,), q + "right.out": (W,)})
            H, D, V = b["heads"], b["dim"], b["vdim"]
            out.update({q + "right.q": (H * D, W), q + "right.k": (H * D, W), q + "right.v": (H * V, W), q + "right.g": (H * V, W),
                        q + "right.i": (H, W), q + "right.i.b": (H,), q + "right.f": (H, W), q + "right.f.b": (H,),
                        q + "right.norm": (H * V,), q + "right.o": (W, H * V)})
        f = layer.get("mlp")
        if f:
            out.update({p + "norm2": (W,), p + "norm2.b": (W,), p + "rg2": (W, W), p + "rg2.b": (W,)})
            if f["kind"] == "dense":
                out.update({p + "mlp.gate": (f["ff"], W), p + "mlp.up": (f["ff"], W), p + "mlp.down": (W, f["ff"])})
            else:
                out[p + "mlp.router"] = (f["router"]["experts"], W)
                for e in range(f["router"]["experts"]):
                    out.update({p + f"mlp.e{e}.gate": (f["expert"]["ff"], W), p + f"mlp.e{e}.up": (f["expert"]["ff"], W),
                                p + f"mlp.e{e}.down": (W, f["expert"]["ff"])})
    return out


def make_weights(cfg: dict, seed: int) -> dict:
    """Random weights, bfloat16 values, of a size that keeps every sublayer's output of order one: a lost state, a
    wrong expert, a missing key or a gate that is left out then moves the logits."""
    gen = torch.Generator().manual_seed(seed)
    out = {}
    for name, shape in tensor_shapes(cfg).items():
        last = name.split(".")[-1]
        if name.endswith(".b"):
            t = 0.3 * torch.randn(shape, generator=gen)
            if name.endswith(".f.b"):
                t = t + 2.5                               # a memory that forgets slowly
        elif last in ("norm", "norm1", "norm2", "out"):
            t = 1.0 + 0.2 * torch.randn(shape, generator=gen)
        elif last in ("conv", "canon1"):
            t = torch.randn(shape, generator=gen) / shape[-1] ** 0.5
        elif last == "lam":
            t = -2.5 + 0.8 * torch.randn(shape, generator=gen)      # a of 0.6 to 0.99
        elif name == "embed":
            t = torch.randn(shape, generator=gen)
        elif name == "pos":
            t = 0.5 * torch.randn(shape, generator=gen)
        elif last == "router":
            t = 2.0 * torch.randn(shape, generator=gen) / shape[-1] ** 0.5
        else:
            t = 1.3 * torch.randn(shape, generator=gen) / shape[-1] ** 0.5
        out[name] = t.to(torch.bfloat16)
    return out


def as_float64(weights: dict) -> dict:
    return {k: v.to(torch.float64) for k, v in weights.items()}


LIMIT = {"float32": 3e-5, "bfloat16": 6e-2}
EDGE_LIMIT = {"float32": 6e-5, "bfloat16": 1e-1}
MARGIN = 0.02      # a bfloat16 engine may exchange experts whose scores are this close


def moe_layers(cfg: dict) -> list:
    return [i for i, layer in enumerate(cfg["layers"]) if (layer.get("mlp") or {}).get("kind") == "moe"]


def check_against_plain(cfg, weights, requests, got, dtype, chosen=None, what="", limit=None):
    """Every position of every request against the plain model.  Under bfloat16 the plain model follows the engine's
    expert choices, each of which must be a top choice of the plain router up to MARGIN."""
    limit = limit or LIMIT[dtype]
    w64 = as_float64(weights)
    worst = 0.0
    for r, tokens in requests.items():
        routing = None
        if chosen and chosen.get(r) is not None:
            routing = {layer: torch.tensor(ids) for layer, ids in zip(moe_layers(cfg), chosen[r])}
        want = plain.forward(cfg, w64, tokens, routing=routing)
        if routing is not None:
            check_choices(cfg, w64, tokens, routing, f"{what} {r}")
        err = row_errors(got[r], want)
        i = int(err.argmax())
        assert float(err[i]) <= limit, (f"{what} request {r}: position {i} of {len(tokens)} is off by {float(err[i]):.3g} "
                                        f"(limit {limit:g}); first position over it: {int((err > limit).nonzero()[0])}")
        worst = max(worst, float(err[i]))
    return worst


def check_choices(cfg, w64, tokens, routing, what):
    """The engine's experts, followed by the plain model, must each score within MARGIN of the plain router's k-th best."""
    streams = []
    plain.forward(cfg, w64, tokens, layers_out=streams, routing=routing)
    tokens_t = torch.as_tensor(tokens)
    x = w64["embed"][tokens_t] + w64["pos"][:len(tokens)]
    for i, entry in enumerate(cfg["layers"]):
        if i in routing:
            lp, eps = f"l{i}.", cfg["norm"]["eps"]
            h = plain.layer_norm(x, w64[lp + "norm1"], w64[lp + "norm1.b"], eps)
            read = h + plain.causal_conv(h, w64[lp + "canon1"]) if cfg.get("canon") else h
            mid = x + plain.mixer(entry["type"], read, w64, lp + "mix.", entry["mixer"], eps) * plain.sigmoid(h @ w64[lp + "rg1"].T + w64[lp + "rg1.b"])
            h2 = plain.layer_norm(mid, w64[lp + "norm2"], w64[lp + "norm2.b"], eps)
            scores = plain.router_scores(h2, w64, lp + "mlp.")
            top = entry["mlp"]["router"]["top"]
            kth = torch.sort(scores, dim=-1, descending=True).values[:, top - 1]
            took = torch.gather(scores, 1, routing[i].to(torch.int64))
            assert float((kth[:, None] - took).max()) <= MARGIN, f"{what}: layer {i} chose an expert {float((kth[:, None] - took).max()):.3g} below the plain router's"
        x = streams[i]


def changed(cfg: dict, layer: int, **mixer_changes) -> dict:
    """The configuration with keys of one layer's mixer replaced ('left__scale' reaches into 'left')."""
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
