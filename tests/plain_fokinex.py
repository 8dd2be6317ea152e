"""Fokinex, written out plainly: one function per mechanism, float64, whole sequences, no cache.

The oracle of the Fokinex tests.  It shares nothing with the package: weights come in as a dict
name -> tensor ([out, in] matrices), the configuration as the dict that config.json holds.

A layer has one norm whose output both sublayers read:  x += mixer(N(x)) + ff(N(x)),
N(x) = x / sqrt(mean(x^2) + eps) * w.  The embedding is multiplied by a constant.  A mixer is
either `latent_attention` (queries and keys/values through low-rank latents, one rotated key
part shared by the heads, a sliding window, a sink in the softmax's denominator; a layer may
read another layer's latents) or `parallel`: a windowed grouped-query attention whose values
are its un-normed keys, with capped scores and a distance penalty, beside a gated delta rule
with one decay per head, the two summed with constant weights.  The feed-forward is silu-gated.
"""
from __future__ import annotations

import math

import numpy as np
import torch

F64 = torch.float64


def rms_norm(x, w, eps):
    return x / torch.sqrt((x * x).mean(-1, keepdim=True) + eps) * w


def silu(z):
    return z * torch.sigmoid(z)


def window_visible(n: int, size: int | None, first_pos: int = 0):
    """[n, n] bool: query i (row) sees key j (column): 0 <= i - j < size."""
    i = torch.arange(n)[:, None]
    j = torch.arange(n)[None, :]
    see = j <= i
    if size:
        see &= (i - j) < size
    return see


# --------------------------------------------------------------------------
# rotation with scaled frequencies
# --------------------------------------------------------------------------
def scaled_rotation(dims: int, base: float, scaling: dict | None):
    """(frequencies f_i for i < dims/2, magnitude).  Without scaling f_i = base^(-2i/dims) and the magnitude is 1.
    With scaling {factor, original, fast, slow}: d(t) = dims ln(original / (2 pi t)) / (2 ln base) is the pair
    index whose wave turns t times over `original` positions; pairs below lo = floor(d(fast)) keep f_i, pairs
    above hi = ceil(d(slow)) get f_i / factor, in between the two are blended linearly in the pair index; the
    rotated vector's cos and sin are both multiplied by 0.1 ln(factor) + 1."""
    freqs = [float(base) ** (-2.0 * i / dims) for i in range(dims // 2)]
    if not scaling:
        return freqs, 1.0
    factor, orig = float(scaling["factor"]), float(scaling["original"])

    def pair_index(turns):
        return dims * math.log(orig / (2.0 * math.pi * turns)) / (2.0 * math.log(base))

    lo = max(math.floor(pair_index(float(scaling["fast"]))), 0)
    hi = min(math.ceil(pair_index(float(scaling["slow"]))), dims - 1)
    out = []
    for i, f in enumerate(freqs):
        ramp = min(max((i - lo) / max(hi - lo, 0.001), 0.0), 1.0)
        out.append(f / factor * ramp + f * (1.0 - ramp))
    return out, 0.1 * math.log(factor) + 1.0


def rotate_pairs(vec, positions, freqs, magnitude=1.0, angles="float32"):
    """vec [n, ..., d]: pairs (2i, 2i+1) of the first 2 len(freqs) entries of the last dimension of row t turn by
    positions[t] * f_i (and grow by `magnitude`); the rest passes.  angles="float32": frequency and product
    rounded to float32, as a 32-bit implementation has them; "exact": float64."""
    out = vec.clone()
    for t, p in enumerate(positions):
        for i, f in enumerate(freqs):
            a = float(np.float32(p) * np.float32(f)) if angles == "float32" else p * f
            c, s = math.cos(a) * magnitude, math.sin(a) * magnitude
            u, v = vec[t, ..., 2 * i], vec[t, ..., 2 * i + 1]
            out[t, ..., 2 * i] = u * c - v * s
            out[t, ..., 2 * i + 1] = v * c + u * s
    return out


# --------------------------------------------------------------------------
# latent attention
# --------------------------------------------------------------------------
def _rotation_of(m):
    rot = m.get("rot")
    if not rot or not rot.get("dims"):
        return [], 1.0
    return scaled_rotation(rot["dims"], rot["base"], rot.get("scaling"))


def latents(h, w, m, eps, angles="float32"):
    """What a latent-attention layer with a down-projection of its own keeps per position: the normed latent
    c [n, kv_rank] and the rotated key part [n, rot_dim] that all heads share."""
    n = h.shape[0]
    R = m["kv_rank"]
    down = h @ w["dkv"].T
    c = rms_norm(down[:, :R], w["dkv.norm"], eps)
    freqs, mag = _rotation_of(m)
    k_rot = rotate_pairs(down[:, R:], list(range(n)), freqs, mag, angles)
    return c, k_rot


def softmax_with_sink(s, sink):
    """Rows of s (masked entries -inf) to weights whose denominator has one more term exp(sink)."""
    top = torch.maximum(s.max(-1, keepdim=True).values, sink)
    e = torch.exp(s - top)
    return e / (e.sum(-1, keepdim=True) + torch.exp(sink - top))


def latent_attention(h, w, m, eps, kept, angles="float32"):
    """The mixer's output [n, width] from its input rows and the (c, k_rot) it reads (its own or another layer's)."""
    n = h.shape[0]
    H, D, Rd, V = m["heads"], m["dim"], m["rot_dim"], m["vdim"]
    c, k_rot = kept
    c_q = rms_norm(h @ w["dq"].T, w["dq.norm"], eps)
    q = (c_q @ w["uq"].T).view(n, H, D + Rd)
    freqs, mag = _rotation_of(m)
    q_plain, q_rot = q[..., :D], rotate_pairs(q[..., D:], list(range(n)), freqs, mag, angles)
    k_plain = (c @ w["uk"].T).view(n, H, D)
    v = (c @ w["uv"].T).view(n, H, V)
    see = window_visible(n, (m.get("mask") or {}).get("size"))
    out = torch.zeros(n, H, V, dtype=h.dtype)
    for a in range(H):
        s = (q_plain[:, a] @ k_plain[:, a].T + q_rot[:, a] @ k_rot.T) * m["scale"]
        s = s.masked_fill(~see, -math.inf)
        out[:, a] = softmax_with_sink(s, w["sink"][a]) @ v[:, a]
    return out.reshape(n, H * V) @ w["o"].T


# --------------------------------------------------------------------------
# the two halves of the parallel mixer
# --------------------------------------------------------------------------
def distance_slopes(H: int):
    return [2.0 ** (-8.0 * (a + 1) / H) for a in range(H)]


def capped_attention(h, w, m, eps):
    """Grouped-query attention: q and k normed over their whole projection, values = keys before the norm, scores
    capped by tanh, a penalty slope_h * (i - j) taken off after the cap, a sliding window, an output gate."""
    n = h.shape[0]
    H, G, D, V = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    q_all, k_all = h @ w["q"].T, h @ w["k"].T
    v = k_all.view(n, G, V)                                   # the keys as projected are the values
    q = rms_norm(q_all, w["q.norm"], eps).view(n, H, D)
    k = rms_norm(k_all, w["k.norm"], eps).view(n, G, D)
    see = window_visible(n, (m.get("mask") or {}).get("size"))
    cap = m.get("softcap")
    dist = (torch.arange(n)[:, None] - torch.arange(n)[None, :]).to(h.dtype)
    out = torch.zeros(n, H, V, dtype=h.dtype)
    for a, slope in enumerate(distance_slopes(H)):
        s = (q[:, a] @ k[:, a // (H // G)].T) * m["scale"]
        if cap:
            s = cap * torch.tanh(s / cap)
        s = (s - slope * dist).masked_fill(~see, -math.inf)
        out[:, a] = torch.softmax(s, dim=-1) @ v[:, a // (H // G)]
    gate = torch.sigmoid(h @ w["g"].T)
    return (out.reshape(n, H * V) * gate) @ w["o"].T


def short_conv_silu(x, taps):
    """x [n, C], taps [C, k]: y[t, c] = silu(sum_j taps[c, k-1-j] x[t-j, c]), zeros before the start."""
    n, _ = x.shape
    k = taps.shape[1]
    y = torch.zeros_like(x)
    for t in range(n):
        for j in range(k):
            if t - j >= 0:
                y[t] += taps[:, k - 1 - j] * x[t - j]
    return silu(y)


def unit(x):
    return x / torch.sqrt((x * x).sum(-1, keepdim=True) + 1e-6)


def gated_delta(h, w, m, eps):
    """Gated delta rule with one decay per head.  Per head, S [dim, vdim] from zero:
        S <- g_t S;  u = beta_t (v_t - S^T k_t);  S <- S + k_t u^T;  o_t = S^T q_t."""
    n = h.shape[0]
    H, G, D, V = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    q = unit(short_conv_silu(h @ w["q"].T, w["q.conv"]).view(n, G, D)) * D ** -0.5
    k = unit(short_conv_silu(h @ w["k"].T, w["k.conv"]).view(n, G, D))
    v = short_conv_silu(h @ w["v"].T, w["v.conv"]).view(n, H, V)
    beta = torch.sigmoid(h @ w["b"].T)                                                        # [n, H]
    g = torch.exp(-torch.exp(w["A_log"]) * torch.nn.functional.softplus(h @ w["a"].T + w["dt_bias"]))   # [n, H]
    out = torch.zeros(n, H, V, dtype=h.dtype)
    for a in range(H):
        kv = a // (H // G)
        S = torch.zeros(D, V, dtype=h.dtype)
        for t in range(n):
            S = g[t, a] * S
            u = beta[t, a] * (v[t, a] - S.T @ k[t, kv])
            S = S + torch.outer(k[t, kv], u)
            out[t, a] = S.T @ q[t, kv]
    out = out / torch.sqrt((out * out).mean(-1, keepdim=True) + eps) * w["norm"]
    out = out * silu(h @ w["g"].T).view(n, H, V)
    return out.reshape(n, H * V) @ w["o"].T


def parallel_mixer(h, w, m, eps):
    left = capped_attention(h, sub(w, "left."), m["left"], eps)
    right = gated_delta(h, sub(w, "right."), m["right"], eps)
    return m["left_scale"] * left + m["right_scale"] * right


# --------------------------------------------------------------------------
# feed-forward and the model
# --------------------------------------------------------------------------
def gated_mlp(h, w):
    return (silu(h @ w["gate"].T) * (h @ w["up"].T)) @ w["down"].T


def sub(weights: dict, prefix: str) -> dict:
    return {k[len(prefix):]: v for k, v in weights.items() if k.startswith(prefix)}


def forward(cfg: dict, weights: dict, tokens: list, dtype=F64, angles: str = "float32", layers_out=None):
    """Logits [n, vocab] of one sequence from position 0.  `layers_out`: a list that receives the residual stream
    after every layer.  (A test that wants a mechanism left out changes the configuration or the weights.)"""
    W = {k: (v.to(dtype) if v.is_floating_point() else v) for k, v in weights.items()}
    eps = cfg["norm"]["eps"]
    x = W["embed"][torch.tensor(tokens)] * (cfg.get("embedding") or {}).get("scale", 1.0)
    kept = {}
    for i, layer in enumerate(cfg["layers"]):
        p = f"l{i}."
        h = rms_norm(x, W[p + "norm1"], eps)
        w, m = sub(W, p + "mix."), layer["mixer"]
        if layer["type"] == "latent_attention":
            if m.get("kv_from") is None:
                kept[i] = latents(h, w, m, eps, angles)
            y = latent_attention(h, w, m, eps, kept[i if m.get("kv_from") is None else m["kv_from"]], angles)
        elif layer["type"] == "parallel":
            y = parallel_mixer(h, w, m, eps)
        else:
            raise ValueError(f"layer {i}: unknown type {layer['type']}")
        if layer.get("mlp"):
            y = y + gated_mlp(h, sub(W, p + "mlp."))
        x = x + y
        if layers_out is not None:
            layers_out.append(x.clone())
    return rms_norm(x, W["final.norm"], eps) @ W["head"].T
