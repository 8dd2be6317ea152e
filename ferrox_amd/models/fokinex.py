"""Fokinex as a list of parts.

Every layer is a parallel block, x += mixer(norm1(x)) + ff(norm1(x)): one norm, both sublayers read it.  The mixer
is latent attention (low-rank latents for queries and for keys/values, one rotated key part shared by the heads,
frequencies stretched by pair index, a sliding window, a sink logit per head; a layer may read an earlier layer's
latents), or two mixers side by side whose outputs are summed with constant weights: windowed grouped-query attention
whose keys are its values (norms over the whole q and k projections, capped scores, a penalty per head for distance,
an output gate) and a gated delta rule with one decay per head.  The feed-forward is silu-gated.  The embedding is
multiplied by a constant; the head has a matrix of its own.  Tensor names are the checkpoint's: `l<i>.norm1`,
`l<i>.mix.dq`, `l<i>.mix.left.q`, `l<i>.mlp.up`, `embed`, `final.norm`, `head`.
"""
from __future__ import annotations

from ..config.fokinex import FokinexConfig
from ..parts.base import LayerSpec, ModelSpec, PartSpec, ScheduleEntry

GATED_NAMES = {"gate": "gate", "up": "up", "down": "down"}
SLOPE_EXPONENT = 8.0        # head h of H loses 2^(-8 (h + 1) / H) of its score per position of distance


def distance_slopes(n_heads: int) -> tuple:
    return tuple(2.0 ** (-SLOPE_EXPONENT * (h + 1) / n_heads) for h in range(n_heads))


def _norm(width: int, eps: float, name: str) -> PartSpec:
    return PartSpec("rmsnorm", {"size": width, "eps": eps, "name": name})


def latent_retention(cfg: FokinexConfig) -> dict:
    """layer -> the window its cache must hold (None: every key): a layer with latents of its own serves its own
    mask and those of the layers that read its cache, which may be wider."""
    need = {}
    for i, layer in enumerate(cfg.layers):
        if layer.type != "latent_attention":
            continue
        m = layer.mixer
        owner = i if m.kv_from is None else m.kv_from
        window = need.get(owner, 0)
        need[owner] = None if (m.window is None or window is None) else max(window, m.window)
    return {i: need[i if layer.mixer.kv_from is None else layer.mixer.kv_from]
            for i, layer in enumerate(cfg.layers) if layer.type == "latent_attention"}


def build_spec(cfg: FokinexConfig, tensor_names=None) -> ModelSpec:
    W, eps = cfg.width, cfg.eps
    retain = latent_retention(cfg)
    layers = []
    for i, layer in enumerate(cfg.layers):
        m = layer.mixer
        if layer.type == "latent_attention":
            position = PartSpec("none", {"head_dim": m.rot_dim})
            if m.rot is not None:
                position = PartSpec("rope_ramped", {"head_dim": m.rot_dim, "theta": m.rot.base, "rotary_dim": m.rot.dims,
                                                    "interleaved": True, "scaling": m.rot.scaling})
            mixer = PartSpec("latent_attention", {
                "hidden_size": W, "n_heads": m.heads, "head_dim": m.dim, "rot_dim": m.rot_dim, "v_dim": m.vdim,
                "q_rank": m.q_rank, "kv_rank": m.kv_rank, "scale": m.scale, "window": m.window, "sink": True,
                "latent_norm": PartSpec("rmsnorm", {"eps": eps, "name": "norm"}), "position": position,
                "own_kv": m.kv_from is None, "retain_window": retain[i] or 0,
            }, prefix="mix.")
        else:
            left, right = m.left, m.right
            mixer = PartSpec("side_by_side", {
                "members": {
                    "left": PartSpec("paged_attention", {
                        "hidden_size": W, "n_heads": left.heads, "n_kv_heads": left.kv_heads, "head_dim": left.dim,
                        "v_dim": left.vdim, "bias": False, "scale": left.scale, "window": left.window,
                        "position": PartSpec("none", {"head_dim": left.dim}),
                        "qk_norm": PartSpec("rmsnorm", {"size": left.dim, "eps": eps, "name": "norm"}),
                        "qk_norm_span": "projection", "values_from_keys": True, "softcap": left.softcap,
                        "distance_slopes": distance_slopes(left.heads), "out_gate": True,
                        "names": {"q": "q", "k": "k", "o": "o", "gate": "g", "q_norm": "q.", "k_norm": "k."},
                    }, prefix="left."),
                    "right": PartSpec("head_delta", {
                        "hidden_size": W, "n_heads": right.heads, "n_kv_heads": right.kv_heads, "key_dim": right.dim,
                        "v_dim": right.vdim, "conv_taps": right.conv, "norm_eps": eps, "gate_activation": "silu",
                    }, prefix="right."),
                },
                "scales": {"left": m.left_scale, "right": m.right_scale},
            }, prefix="mix.")
        parts = {"norm1": _norm(W, eps, "norm1"), "mixer": mixer}
        if layer.mlp is not None:
            parts["ffn"] = PartSpec("gated_mlp", {"hidden_size": W, "intermediate_size": layer.mlp.ff, "activation": "silu",
                                                  "names": GATED_NAMES}, prefix="mlp.")
        layers.append(LayerSpec("parallel", f"l{i}.", parts))
    return ModelSpec(
        hidden_size=W, vocab_size=cfg.vocab,
        embedding=PartSpec("token_embedding", {"vocab_size": cfg.vocab, "hidden_size": W, "name": "embed",
                                               "scale": cfg.embedding_scale}),
        layers=layers,
        schedule=[ScheduleEntry(i, cache=getattr(layer.mixer, "kv_from", None)) for i, layer in enumerate(cfg.layers)],
        final_norm=PartSpec("rmsnorm", {"size": W, "eps": eps, "name": "final.norm"}),
        head=PartSpec("linear_head", {"vocab_size": cfg.vocab, "hidden_size": W, "name": "head"}),
        max_positions=cfg.max_positions,
        eos_token_id=cfg.eos_token_id,
    )
