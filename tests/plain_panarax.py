"""Plain, slow Panarax: every formula of the design, one function per mechanism, float64 on the CPU, whole
sequences at once, no cache.  It shares no code with the package: tests hold the engine against it.

A model is (cfg, w): cfg the config.json dict, w a dict name -> float64 tensor.  `forward(cfg, w, tokens)` returns
logits [T, vocab]; `layers_out` receives the stream after every layer."""
from __future__ import annotations

import math

import torch

F64 = torch.float64


def sigmoid(x):
    return 1.0 / (1.0 + torch.exp(-x))


def silu(x):
    return x * sigmoid(x)


def softplus(x):
    return torch.where(x > 30.0, x, torch.log1p(torch.exp(torch.clamp(x, max=30.0))))


def logsigmoid(x):
    return -softplus(-x)


def gelu_tanh(z):
    return 0.5 * z * (1.0 + torch.tanh(math.sqrt(2.0 / math.pi) * (z + 0.044715 * z ** 3)))


def layer_norm(x, weight, bias, eps):
    mean = x.mean(-1, keepdim=True)
    var = ((x - mean) ** 2).mean(-1, keepdim=True)
    return (x - mean) / torch.sqrt(var + eps) * weight + bias


def unit_rms(x, eps):
    return x / torch.sqrt((x * x).mean(-1, keepdim=True) + eps)


def causal_conv(x, taps, bias=None):
    """y_t = sum_j taps[:, j] x_(t - n + 1 + j): the last column of taps meets the current token; zeros before
    the start.  x [T, C], taps [C, n]."""
    T, C = x.shape
    n = taps.shape[1]
    padded = torch.cat([torch.zeros(n - 1, C, dtype=x.dtype), x], dim=0)
    y = torch.zeros_like(x)
    for j in range(n):
        y = y + taps[:, j] * padded[j:j + T]
    return y if bias is None else y + bias


# ---- mixers ------------------------------------------------------------------------------------------------
def rglru(h, w, p, m):
    """The recurrent block around a real-gated linear recurrent unit.  m: blocks, conv, width."""
    C, B = m["width"], m["blocks"]
    y = gelu_tanh(h @ w[p + "y"].T + w[p + "y.b"])
    u = causal_conv(h @ w[p + "x"].T + w[p + "x.b"], w[p + "conv"], w[p + "conv.b"])
    T = h.shape[0]
    ub = u.view(T, B, C // B)
    r = sigmoid(torch.einsum("tbi,boi->tbo", ub, w[p + "ra"]) + w[p + "ra.b"]).reshape(T, C)
    i = sigmoid(torch.einsum("tbi,boi->tbo", ub, w[p + "ri"]) + w[p + "ri.b"]).reshape(T, C)
    log_a = -8.0 * r * softplus(w[p + "lam"])
    a = torch.exp(log_a)
    x_in = torch.sqrt(1.0 - a * a) * i * u
    S = torch.zeros(C, dtype=h.dtype)
    out = []
    for t in range(T):
        S = a[t] * S + x_in[t]
        out.append(S)
    return (torch.stack(out) * y) @ w[p + "o"].T


def lightning(h, w, p, m, eps):
    """Linear attention with one constant decay per head."""
    H, D, V = m["heads"], m["dim"], m["vdim"]
    T = h.shape[0]
    q = silu(h @ w[p + "q"].T).view(T, H, D)
    k = silu(h @ w[p + "k"].T).view(T, H, D)
    v = silu(h @ w[p + "v"].T).view(T, H, V)
    decay = torch.tensor(m["decay"], dtype=h.dtype)
    S = torch.zeros(H, D, V, dtype=h.dtype)
    out = []
    for t in range(T):
        S = decay[:, None, None] * S + k[t][:, :, None] * v[t][:, None, :]
        out.append(torch.einsum("hdv,hd->hv", S, q[t]))
    o = torch.stack(out).reshape(T, H * V)
    o = unit_rms(o, eps) * w[p + "norm"]
    return (o * sigmoid(h @ w[p + "g"].T)) @ w[p + "o"].T


def query_temperature(positions, coef, every):
    return 1.0 + coef * torch.log(torch.floor((positions + 1) / every) + 1.0)


def softmax_attention(h, w, p, m, eps):
    """Grouped-query attention: a temperature on the queries by position, unit values, an output gate a head."""
    H, G, D, V = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    T = h.shape[0]
    pos = torch.arange(T, dtype=h.dtype)
    q = (h @ w[p + "q"].T).view(T, H, D)
    if m.get("q_temp"):
        q = q * query_temperature(pos, m["q_temp"]["coef"], m["q_temp"]["every"])[:, None, None]
    k = (h @ w[p + "k"].T).view(T, G, D)
    v = unit_rms((h @ w[p + "v"].T).view(T, G, V), eps)
    gate = sigmoid(h @ w[p + "g"].T)                                   # [T, H]
    visible = pos[None, :] <= pos[:, None]
    outs = []
    for head in range(H):
        g = head // (H // G)
        s = (q[:, head] @ k[:, g].T) * m["scale"]
        s = torch.where(visible, s, torch.full_like(s, -math.inf))
        outs.append((torch.softmax(s, dim=-1) @ v[:, g]) * gate[:, head:head + 1])
    return torch.cat(outs, dim=-1) @ w[p + "o"].T


def matrix_memory(h, w, p, m, eps):
    """A matrix memory with exponential gates kept in range by a running maximum."""
    H, D, V, cap = m["heads"], m["dim"], m["vdim"], m["gate_cap"]
    T = h.shape[0]
    q = (h @ w[p + "q"].T).view(T, H, D) * D ** -0.5
    k = (h @ w[p + "k"].T).view(T, H, D)
    v = (h @ w[p + "v"].T).view(T, H, V)
    i_gate = cap * torch.tanh((h @ w[p + "i"].T + w[p + "i.b"]) / cap)                    # [T, H], a logarithm
    f_gate = logsigmoid(cap * torch.tanh((h @ w[p + "f"].T + w[p + "f.b"]) / cap))
    S = torch.zeros(H, D, V, dtype=h.dtype)
    n = torch.zeros(H, D, dtype=h.dtype)
    mx = torch.zeros(H, dtype=h.dtype)
    out = []
    for t in range(T):
        m_new = torch.maximum(f_gate[t] + mx, i_gate[t])
        keep, take = torch.exp(f_gate[t] + mx - m_new), torch.exp(i_gate[t] - m_new)
        S = keep[:, None, None] * S + take[:, None, None] * k[t][:, :, None] * v[t][:, None, :]
        n = keep[:, None] * n + take[:, None] * k[t]
        mx = m_new
        num = torch.einsum("hdv,hd->hv", S, q[t])
        den = torch.maximum((n * q[t]).sum(-1).abs(), torch.exp(-mx)) + 1e-6
        out.append(num / den[:, None])
    o = unit_rms(torch.stack(out), eps).reshape(T, H * V) * w[p + "norm"]
    return (o * sigmoid(h @ w[p + "g"].T)) @ w[p + "o"].T


def side_by_side(h, w, p, m, eps):
    left = softmax_attention(h, w, p + "left.", m["left"], eps)
    right = matrix_memory(h, w, p + "right.", m["right"], eps)
    return 0.5 * (unit_rms(left, eps) * w[p + "left.out"] + unit_rms(right, eps) * w[p + "right.out"])


# ---- feed-forwards -----------------------------------------------------------------------------------------
def dense_ff(h, w, p):
    return (silu(h @ w[p + "gate"].T) * (h @ w[p + "up"].T)) @ w[p + "down"].T


def expert(x, w, p, limit):
    g = torch.clamp(x @ w[p + "gate"].T, max=limit)
    u = torch.clamp(x @ w[p + "up"].T, -limit, limit)
    return (g * sigmoid(1.702 * g) * (u + 1.0)) @ w[p + "down"].T


def router_scores(h, w, p):
    return sigmoid(h @ w[p + "router"].T)


def choose(scores, top):
    """The `top` largest scores of each row, ties to the lower index: (ids, weights)."""
    order = torch.sort(scores, dim=-1, descending=True, stable=True).indices[:, :top]
    return order, torch.gather(scores, 1, order)


def mixture(h, w, p, mlp, routing=None):
    """The weight of a chosen expert multiplies what the expert reads.  `routing`: ids [T, top] to use instead of
    the plain choice (the weights are the plain scores of those ids)."""
    scores = router_scores(h, w, p)
    ids, weights = choose(scores, mlp["router"]["top"])
    if routing is not None:
        ids = routing.to(torch.int64)
        weights = torch.gather(scores, 1, ids)
    out = torch.zeros_like(h)
    for t in range(h.shape[0]):
        for j in range(ids.shape[1]):
            e = int(ids[t, j])
            out[t] = out[t] + expert(weights[t, j] * h[t:t + 1], w, f"{p}e{e}.", mlp["expert"]["limit"])[0]
    return out


# ---- the model ---------------------------------------------------------------------------------------------
def mixer(kind, h, w, p, m, eps):
    if kind == "rglru":
        return rglru(h, w, p, m)
    if kind == "lightning":
        return lightning(h, w, p, m, eps)
    if kind == "parallel":
        return side_by_side(h, w, p, m, eps)
    raise ValueError(kind)


def layer(x, w, i, entry, cfg, routing=None):
    eps, lp = cfg["norm"]["eps"], f"l{i}."
    h = layer_norm(x, w[lp + "norm1"], w[lp + "norm1.b"], eps)
    read = h + causal_conv(h, w[lp + "canon1"]) if cfg.get("canon") else h
    y = mixer(entry["type"], read, w, lp + "mix.", entry["mixer"], eps)
    x = x + y * sigmoid(h @ w[lp + "rg1"].T + w[lp + "rg1.b"])
    if entry.get("mlp") is None:
        return x
    h = layer_norm(x, w[lp + "norm2"], w[lp + "norm2.b"], eps)
    if entry["mlp"]["kind"] == "dense":
        y = dense_ff(h, w, lp + "mlp.")
    else:
        y = mixture(h, w, lp + "mlp.", entry["mlp"], routing)
    return x + y * sigmoid(h @ w[lp + "rg2"].T + w[lp + "rg2.b"])


def forward(cfg, w, tokens, layers_out=None, routing=None):
    """Logits [T, vocab] of one sequence from position 0.  `routing`: layer -> expert ids [T, top]."""
    tokens = torch.as_tensor(tokens, dtype=torch.int64)
    T = tokens.numel()
    x = w["embed"][tokens] + w["pos"][:T]
    for i, entry in enumerate(cfg["layers"]):
        x = layer(x, w, i, entry, cfg, None if routing is None else routing.get(i))
        if layers_out is not None:
            layers_out.append(x.clone())
    x = layer_norm(x, w["final.norm"], w["final.norm.b"], cfg["norm"]["eps"])
    return x @ w["embed"].T
