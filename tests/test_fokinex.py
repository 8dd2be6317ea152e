"""Fokinex without a GPU: the plain model's own properties, the configuration reader, the description's tensor
names, what the caches of its layers must hold, the frequencies of the stretched rotation."""
import copy
import math

import pytest
import torch

import fokinex_util as u
import plain_fokinex as plain
from ferrox_amd.config.base import ConfigError
from ferrox_amd.config.fokinex import FokinexConfig
from ferrox_amd.engine.model import Model
from ferrox_amd.models.fokinex import build_spec, distance_slopes, latent_retention
from ferrox_amd.models.registry import resolve
from ferrox_amd.parts.rope import ramped_frequencies

F64 = torch.float64


def as64(w):
    return {k: v.to(F64) for k, v in w.items()}


# ---------------------------------------------------------------------------
# the plain model
# ---------------------------------------------------------------------------
def test_window_visibility():
    see = plain.window_visible(8, 3)
    assert see[7].tolist() == [False] * 5 + [True] * 3
    assert see[1].tolist() == [True, True] + [False] * 6
    assert plain.window_visible(5, None).tolist() == torch.tril(torch.ones(5, 5)).bool().tolist()


def test_stretched_rotation_has_three_bands_and_a_magnitude():
    dims, base = 16, 100.0
    plain_f, one = plain.scaled_rotation(dims, base, None)
    assert one == 1.0 and plain_f[3] == pytest.approx(base ** (-6 / 16))
    f, mag = plain.scaled_rotation(dims, base, dict(zip(("factor", "original", "fast", "slow"), (4.0, 40, 4.0, 0.5))))
    assert mag == pytest.approx(0.1 * math.log(4.0) + 1.0)
    ratios = [a / b for a, b in zip(f, plain_f)]
    assert ratios[0] == 1.0 and ratios[-1] == pytest.approx(0.25)             # fast waves kept, slow ones stretched
    assert any(0.25 < r < 1.0 for r in ratios) and ratios == sorted(ratios, reverse=True)
    # the package's table is the same numbers
    assert ramped_frequencies(dims, base, 4.0, 40, 4.0, 0.5) == pytest.approx(f, rel=1e-15)


def test_rotation_depends_on_distance_alone():
    freqs, mag = plain.scaled_rotation(8, 50.0, None)
    q, k = torch.randn(1, 8, dtype=F64), torch.randn(1, 8, dtype=F64)
    a = (plain.rotate_pairs(q, [11], freqs, mag, "exact") * plain.rotate_pairs(k, [4], freqs, mag, "exact")).sum()
    b = (plain.rotate_pairs(q, [107], freqs, mag, "exact") * plain.rotate_pairs(k, [100], freqs, mag, "exact")).sum()
    assert float(a) == pytest.approx(float(b), abs=1e-12)
    # a magnitude m multiplies the rotated part's share of a score by m^2
    c = (plain.rotate_pairs(q, [11], freqs, 1.3, "exact") * plain.rotate_pairs(k, [4], freqs, 1.3, "exact")).sum()
    assert float(c) == pytest.approx(1.69 * float(a), rel=1e-12)


def test_the_sink_takes_weight_and_brings_no_value():
    s = torch.tensor([[0.3, -math.inf, -math.inf]], dtype=F64)
    p = plain.softmax_with_sink(s, torch.tensor(1.1, dtype=F64))
    assert float(p[0, 0]) == pytest.approx(1.0 / (1.0 + math.exp(1.1 - 0.3))) and float(p[0, 1]) == 0.0
    assert float(plain.softmax_with_sink(s, torch.tensor(-800.0, dtype=F64))[0, 0]) == pytest.approx(1.0)
    assert float(plain.softmax_with_sink(s, torch.tensor(800.0, dtype=F64))[0, 0]) == 0.0


def test_latent_attention_equals_attention_over_projected_keys_and_latent_values():
    """The form the engine computes (queries through the transposed key projection, one shared key head, values
    projected after the sum) against the plain form with keys and values per head."""
    cfg = u.config([u.latent_layer(heads=3, dim=8, rot_dim=4, vdim=6, q_rank=10, kv_rank=12, window=5, scale=0.4)], width=32)
    w = as64(plain.sub(u.make_weights(cfg, 2), "l0.mix."))
    m = cfg["layers"][0]["mixer"]
    h = torch.randn(9, 32, dtype=F64)
    kept = plain.latents(h, w, m, 1e-6)
    want = plain.latent_attention(h, w, m, 1e-6, kept)
    c, kr = kept
    n, H, D, P, V, R = 9, 3, 8, 4, 6, 12
    q = (plain.rms_norm(h @ w["dq"].T, w["dq.norm"], 1e-6) @ w["uq"].T).view(n, H, D + P)
    freqs, mag = plain.scaled_rotation(4, 10000.0, None)
    heads = torch.zeros(n, H, V, dtype=F64)
    see = plain.window_visible(n, 5)
    for a in range(H):
        q_lat = torch.cat([q[:, a, :D] @ w["uk"][a * D:(a + 1) * D], plain.rotate_pairs(q[:, a, D:], list(range(n)), freqs, mag)], dim=1)
        s = (q_lat @ torch.cat([c, kr], dim=1).T * m["scale"]).masked_fill(~see, -math.inf)
        heads[:, a] = (plain.softmax_with_sink(s, w["sink"][a]) @ c) @ w["uv"][a * V:(a + 1) * V].T
    assert torch.allclose(heads.reshape(n, H * V) @ w["o"].T, want, atol=1e-12)


def test_a_reader_of_another_layers_latents_sees_them():
    cfg = u.config([u.latent_layer(heads=2, dim=8, rot_dim=4, vdim=8, q_rank=8, kv_rank=12, window=6),
                    u.latent_layer(heads=3, dim=4, rot_dim=4, vdim=8, q_rank=8, kv_rank=12, window=9, kv_from=0)], width=32)
    w = u.make_weights(cfg, 3)
    tokens = u.random_tokens(cfg["vocab"], 14, 1)
    base = plain.forward(cfg, w, tokens)
    other = dict(w, **{"l0.mix.dkv": (w["l0.mix.dkv"].float() * 1.5).to(torch.bfloat16)})
    layers_a, layers_b = [], []
    plain.forward(cfg, w, tokens, layers_out=layers_a)
    plain.forward(cfg, other, tokens, layers_out=layers_b)
    assert not torch.allclose(layers_a[1] - layers_a[0], layers_b[1] - layers_b[0])      # layer 1 has no W_dkv, yet it moved
    assert base.shape == (14, cfg["vocab"])


def test_capped_scores_and_the_distance_penalty():
    cfg = u.config([u.parallel_layer(heads=2, kv_heads=1, dim=8, window=0, scale=3.0, softcap=2.0, right_scale=0.0)], width=16)
    w = as64(plain.sub(u.make_weights(cfg, 4), "l0.mix.left."))
    m = cfg["layers"][0]["mixer"]["left"]
    h = torch.randn(6, 16, dtype=F64)
    got = plain.capped_attention(h, w, m, 1e-6)
    # by hand for the last query: scores capped at +-2, then less slope * distance, values are the raw keys
    q = plain.rms_norm(h @ w["q"].T, w["q.norm"], 1e-6).view(6, 2, 8)
    k_raw = h @ w["k"].T
    k = plain.rms_norm(k_raw, w["k.norm"], 1e-6)
    out = []
    for a, slope in enumerate(distance_slopes(2)):
        s = 2.0 * torch.tanh((k @ q[5, a]) * 3.0 / 2.0) - slope * (5 - torch.arange(6, dtype=F64))
        assert float(s.max()) <= 2.0
        out.append(torch.softmax(s, 0) @ k_raw)
    want = (torch.cat(out) * torch.sigmoid(w["g"] @ h[5])) @ w["o"].T
    assert torch.allclose(got[5], want, atol=1e-12)
    assert distance_slopes(4) == pytest.approx([2.0 ** -2, 2.0 ** -4, 2.0 ** -6, 2.0 ** -8])
    assert plain.distance_slopes(4) == pytest.approx(distance_slopes(4))


def test_the_convolution_is_causal_and_the_delta_rule_reads_back_what_it_wrote():
    x = torch.randn(7, 5, dtype=F64)
    taps = torch.randn(5, 3, dtype=F64)
    y = plain.short_conv_silu(x, taps)
    x2 = x.clone()
    x2[4:] += 1.0
    assert torch.equal(plain.short_conv_silu(x2, taps)[:4], y[:4])
    pre = taps[:, 2] * x[0]                        # the first token sees zeros before it: the last tap alone
    assert torch.allclose(y[0], pre * torch.sigmoid(pre))
    # one head, no decay, beta 1: after writing (k, v), reading with q = k gives v back
    S = torch.zeros(4, 3, dtype=F64)
    k = plain.unit(torch.randn(4, dtype=F64))
    v = torch.randn(3, dtype=F64)
    S = S + torch.outer(k, 1.0 * (v - S.T @ k))
    assert torch.allclose(S.T @ k, v, atol=1e-5)


def test_the_plain_model_shows_every_mechanism():
    """Leaving a mechanism out, or a window one position off, moves the plain model's logits far beyond the limits of
    the GPU tests: those tests can tell."""
    cfg = u.config([u.latent_layer(heads=2, dim=16, rot_dim=8, vdim=16, q_rank=16, kv_rank=24, window=7, scale=0.9, base=100.0, scaling=u.STRETCH, mlp=u.dense(32)),
                    u.parallel_layer(heads=2, kv_heads=1, dim=16, window=6, scale=0.9, softcap=1.5, r_heads=2, r_kv_heads=1, r_dim=8, r_vdim=16, conv=3),
                    u.latent_layer(heads=2, dim=16, rot_dim=8, vdim=16, q_rank=16, kv_rank=24, window=12, scale=0.9, base=100.0, scaling=u.STRETCH, kv_from=0)], width=32)
    w = u.make_weights(cfg, 5)
    tokens = u.random_tokens(cfg["vocab"], 40, 2)
    right = plain.forward(cfg, w, tokens)

    def moved(other_cfg=None, other_w=None):
        return float(u.row_errors(plain.forward(other_cfg or cfg, other_w or w, tokens), right).max())

    assert moved(u.changed(cfg, 0, mask={"size": 6})) > 0.02 and moved(u.changed(cfg, 0, mask={"size": 8})) > 0.02
    assert moved(u.changed(cfg, 2, mask={"size": 11})) > 0.01 and moved(u.changed(cfg, 2, mask={"size": 13})) > 0.01
    assert moved(u.changed(cfg, 1, left__mask={"size": 5})) > 0.01 and moved(u.changed(cfg, 1, left__mask={"size": 7})) > 0.01
    assert moved(u.changed(cfg, 1, left__softcap=None)) > 0.01
    assert moved(u.changed(cfg, 1, left_scale=1.0)) > 0.005 and moved(u.changed(cfg, 1, right_scale=1.0)) > 0.005
    assert moved(u.changed(cfg, 0, rot={"base": 100.0, "dims": 8})) > 0.01                  # no stretching, magnitude 1
    assert moved(dict(cfg, embedding={"scale": 1.0})) > 0.05
    low = dict(w, **{"l0.mix.sink": w["l0.mix.sink"] - 30.0})
    assert moved(other_w=low) > 0.02
    no_state = dict(w, **{"l1.mix.right.A_log": w["l1.mix.right.A_log"] + 8.0})              # a decay that forgets at once
    assert moved(other_w=no_state) > 0.01


# ---------------------------------------------------------------------------
# configuration and description
# ---------------------------------------------------------------------------
def test_configuration_reads_every_size_from_the_file():
    cfg = FokinexConfig.from_dict(copy.deepcopy(u.CFG_MAIN))
    assert (cfg.vocab, cfg.width, cfg.eps, cfg.embedding_scale, len(cfg.layers)) == (160, 64, 1e-6, 2.5, 7)
    a = cfg.layers[0].mixer
    assert (a.heads, a.dim, a.rot_dim, a.vdim, a.q_rank, a.kv_rank, a.window, a.kv_from) == (4, 16, 8, 24, 20, 32, 20, None)
    assert a.rot.dims == 8 and a.rot.base == 100.0 and a.rot.scaling == (3.0, 40.0, 4.0, 0.5)
    assert cfg.layers[2].mixer.kv_from == 0 and cfg.layers[2].mlp is None
    assert cfg.layers[3].mixer.window is None and cfg.layers[3].mixer.rot.dims == 4 and cfg.layers[3].mixer.rot.scaling is None
    assert cfg.layers[6].mixer.rot is None
    p = cfg.layers[1].mixer
    assert (p.left.heads, p.left.kv_heads, p.left.dim, p.left.softcap, p.left.window) == (4, 2, 16, 4.0, 13)
    assert (p.right.heads, p.right.kv_heads, p.right.dim, p.right.vdim, p.right.conv) == (4, 2, 16, 24, 4)
    assert (p.left_scale, p.right_scale) == (0.8, 1.4)
    assert cfg.layers[5].mixer.left.softcap is None and cfg.layers[5].mixer.left.window is None
    assert FokinexConfig.from_dict(cfg.to_dict()) == cfg
    assert resolve(u.CFG_MAIN).config_class is FokinexConfig
    assert FokinexConfig.from_dict(u.config([u.latent_layer()], emb_scale=None)).embedding_scale == 1.0


@pytest.mark.parametrize("change,complaint", [
    (lambda c: c["layers"][0].update(type="attention"), "type 'attention'"),
    (lambda c: c["layers"][2]["mixer"].update(kv_from=2), "earlier layer"),
    (lambda c: c["layers"][2]["mixer"].update(kv_from=1), "no latents of its own"),
    (lambda c: c["layers"][4]["mixer"].update(kv_from=2), "no latents of its own"),
    (lambda c: c["layers"][2]["mixer"].update(kv_rank=16), "another latent size"),
    (lambda c: c["layers"][0]["mixer"]["rot"].update(dims=10), "at most rot_dim"),
    (lambda c: c["layers"][0]["mixer"].update(kv_rank=510), "attention kernels"),
    (lambda c: c["layers"][1]["mixer"]["left"].update(vdim=8), "keys are the values"),
    (lambda c: c["layers"][1]["mixer"]["left"].update(kv_heads=3), "not a multiple"),
    (lambda c: c["layers"][1]["mixer"]["right"].update(conv=40), "taps"),
    (lambda c: c["layers"][0]["mlp"].update(kind="moe"), "kind 'moe'"),
    (lambda c: c.pop("norm"), "'norm'"),
    (lambda c: c.update(layers=[]), "at least one layer"),
])
def test_configuration_refusals(change, complaint):
    raw = copy.deepcopy(u.CFG_MAIN)
    change(raw)
    with pytest.raises(ConfigError) as e:
        FokinexConfig.from_dict(raw)
    assert complaint in str(e.value)


def test_tensor_names_and_shapes_of_the_description():
    for cfg in (u.CFG_MAIN, u.CFG_MFMA):
        model = Model(build_spec(FokinexConfig.from_dict(cfg)))
        assert {k: tuple(v.shape) for k, v in model.named_params().items()} == u.tensor_shapes(cfg)


def test_a_cache_holds_what_its_widest_reader_sees():
    cfg = FokinexConfig.from_dict(u.CFG_MAIN)
    assert latent_retention(cfg) == {0: 37, 2: 37, 3: None, 4: None, 6: 11}
    model = Model(build_spec(cfg))
    groups = model.cache_groups()
    assert groups == {("window", 37): 37, ("window", 13): 13, ("full",): None, ("window", 11): 11}
    assert [e.cache for e in model.schedule] == [None, None, 0, None, 3, None, None]
    # a reader's mixer sees its owner's pages; the layer of two mixers keeps the attention's pages and the rule's state
    side = model.blocks[1].mixer
    assert set(side.page_shapes(16)) == {"left.k", "left.v"} and set(side.state_shapes()) == {"right.conv", "right.S"}
    assert side.page_shapes(16)["left.k"] == (2, 16, 16) and side.state_shapes()["right.S"][0] == (4, 24, 16)
    latent = model.blocks[0].mixer
    assert latent.page_shapes(16) == {"k": (1, 16, 40), "v": (1, 32, 16)}      # (c | rotated part) and c, one head
    assert model.blocks[2].mixer.page_shapes(16) == latent.page_shapes(16)


def test_named_shape_of_the_design_reads():
    from ferrox_amd.config import presets
    raw = presets.load("fokinex-2k")
    assert resolve(raw).name == "Fokinex"
    cfg = FokinexConfig.from_dict(raw)
    assert len(cfg.layers) == 8 and {layer.type for layer in cfg.layers} == {"latent_attention", "parallel"}
    assert [layer.mixer.kv_from for layer in cfg.layers if layer.type == "latent_attention"] == [None, None, 1, None, None, 5]
    assert Model(build_spec(cfg)).cache_groups() == {("window", 8192): 8192}
