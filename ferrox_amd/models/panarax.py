"""Panarax as a list of parts.

Every layer is a gated pre-norm block: x += G1 * mixer(C(N1(x))), x += G2 * ff(N2(x)), N a layer norm with weight
and bias, C the input convolution (what the mixer reads is h + conv(h), a short causal convolution per channel), G a
learned gate sigmoid(W h + b) on what the sublayer returns.  The mixer is a recurrent block around a real-gated linear
recurrent unit, linear attention with a constant decay per head, or two mixers side by side whose outputs are each
normed over the model width and averaged: grouped-query softmax attention (queries warmed by position, values of unit
size, one output gate a head, no rotation) and a matrix memory with exponential gates.  The feed-forward is
silu-gated, or a mixture whose experts clamp gate and up and whose weights (sigmoid scores, not renormalised) multiply
what the experts read.  A learned vector per position joins the embedding; the head is the embedding table.  Tensor
names are the checkpoint's: `l<i>.norm1`, `l<i>.norm1.b`, `l<i>.canon1`, `l<i>.rg1`, `l<i>.mix.left.q`,
`l<i>.mlp.e<j>.gate`, `embed`, `pos`, `final.norm`.
"""
from __future__ import annotations

from ..config.panarax import DenseConfig, PanaraxConfig
from ..parts.base import LayerSpec, ModelSpec, PartSpec, ScheduleEntry

GATED_NAMES = {"gate": "gate", "up": "up", "down": "down"}
MOE_NAMES = {"router": "router", "gate": "e{}.gate", "up": "e{}.up", "down": "e{}.down"}
BLOCK_NAMES = {"conv": "canon1", "gate1": "rg1", "gate1_bias": "rg1.b", "gate2": "rg2", "gate2_bias": "rg2.b"}
EXPERT_SLOPE = 1.702          # an expert's gate is g * sigmoid(1.702 g)
SIDE_WEIGHT = 0.5             # the two mixers of a parallel layer are averaged


def _norm(width: int, eps: float, name: str) -> PartSpec:
    return PartSpec("layernorm", {"size": width, "eps": eps, "name": name, "bias_name": name + ".b"})


def _mixer(kind: str, m, W: int, eps: float) -> PartSpec:
    if kind == "rglru":
        return PartSpec("rglru", {"hidden_size": W, "width": m.width, "n_blocks": m.blocks, "conv_taps": m.conv}, prefix="mix.")
    if kind == "lightning":
        return PartSpec("decay_attention", {"hidden_size": W, "n_heads": m.heads, "key_dim": m.dim, "v_dim": m.vdim,
                                            "decay": m.decay, "norm_eps": eps, "activation": "silu"}, prefix="mix.")
    left, right = m.left, m.right
    return PartSpec("side_by_side", {
        "members": {
            "left": PartSpec("paged_attention", {
                "hidden_size": W, "n_heads": left.heads, "n_kv_heads": left.kv_heads, "head_dim": left.dim,
                "v_dim": left.vdim, "bias": False, "scale": left.scale, "position": PartSpec("none", {"head_dim": left.dim}),
                "q_temperature": left.q_temp, "unit_values": eps, "out_gate": "head",
                "names": {"q": "q", "k": "k", "v": "v", "o": "o", "gate": "g"},
            }, prefix="left."),
            "right": PartSpec("matrix_memory", {
                "hidden_size": W, "n_heads": right.heads, "key_dim": right.dim, "v_dim": right.vdim,
                "gate_cap": right.gate_cap, "norm_eps": eps,
            }, prefix="right."),
        },
        "scales": {"left": SIDE_WEIGHT, "right": SIDE_WEIGHT},
        "member_norms": {"left": PartSpec("rmsnorm", {"size": W, "eps": eps, "name": "left.out"}),
                         "right": PartSpec("rmsnorm", {"size": W, "eps": eps, "name": "right.out"})},
    }, prefix="mix.")


def _feed_forward(mlp, W: int) -> PartSpec:
    if isinstance(mlp, DenseConfig):
        return PartSpec("gated_mlp", {"hidden_size": W, "intermediate_size": mlp.ff, "activation": "silu",
                                      "names": GATED_NAMES}, prefix="mlp.")
    return PartSpec("sparse_moe", {
        "hidden_size": W, "n_experts": mlp.experts, "top_k": mlp.top, "expert_intermediate_size": mlp.ff,
        "norm_topk_prob": False, "gating": "sigmoid", "activation": "swiglu_clamped",
        "activation_params": (mlp.limit, EXPERT_SLOPE), "weight_input": True, "names": MOE_NAMES,
    }, prefix="mlp.")


def build_spec(cfg: PanaraxConfig, tensor_names=None) -> ModelSpec:
    W, eps = cfg.width, cfg.eps
    layers = []
    for i, layer in enumerate(cfg.layers):
        parts = {"norm1": _norm(W, eps, "norm1"), "mixer": _mixer(layer.type, layer.mixer, W, eps)}
        if layer.mlp is not None:
            parts["norm2"] = _norm(W, eps, "norm2")
            parts["ffn"] = _feed_forward(layer.mlp, W)
        layers.append(LayerSpec("gated_prenorm", f"l{i}.", parts,
                                args={"hidden_size": W, "conv_taps": cfg.canon_taps, "residual_gates": True, "names": BLOCK_NAMES}))
    return ModelSpec(
        hidden_size=W, vocab_size=cfg.vocab,
        embedding=PartSpec("token_embedding", {"vocab_size": cfg.vocab, "hidden_size": W, "name": "embed",
                                               "position_table": "pos", "max_positions": cfg.max_positions}),
        layers=layers,
        schedule=[ScheduleEntry(i) for i in range(len(cfg.layers))],
        final_norm=_norm(W, eps, "final.norm"),
        head=PartSpec("linear_head", {"vocab_size": cfg.vocab, "hidden_size": W, "tied_to": "embed"}),
        max_positions=cfg.max_positions,
        eos_token_id=cfg.eos_token_id,
    )
