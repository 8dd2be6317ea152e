"""Panarax on the CPU: the plain model's own properties (it is the judge of the GPU tests), the configuration reader
and its refusals, and the tensor names and shapes of the model description against a list written from the design."""
import copy
import math

import pytest
import torch

import panarax_util as u
import plain_panarax as plain

F64 = torch.float64


def rand(*shape, seed=0):
    return torch.randn(*shape, dtype=F64, generator=torch.Generator().manual_seed(seed))


# ---------------------------------------------------------------------------
# the plain model
# ---------------------------------------------------------------------------
def test_layer_norm_has_zero_mean_and_unit_variance_before_weight_and_bias():
    x = rand(5, 33) * 3 + 2
    y = plain.layer_norm(x, torch.ones(33, dtype=F64), torch.zeros(33, dtype=F64), 0.0)
    assert float(y.mean(-1).abs().max()) < 1e-12 and float(((y * y).mean(-1) - 1).abs().max()) < 1e-12
    w, b = rand(33, seed=1), rand(33, seed=2)
    assert torch.allclose(plain.layer_norm(x, w, b, 0.0), y * w + b)


def test_convolution_is_causal_and_its_last_column_meets_the_current_token():
    x, taps = rand(9, 4), rand(4, 3, seed=1)
    y = plain.causal_conv(x, taps)
    assert torch.allclose(y[0], taps[:, 2] * x[0])
    assert torch.allclose(y[5], taps[:, 2] * x[5] + taps[:, 1] * x[4] + taps[:, 0] * x[3])
    x2 = x.clone()
    x2[6:] += 1.0
    assert torch.equal(plain.causal_conv(x2, taps)[:6], y[:6])


def test_query_temperature_steps_with_the_position():
    pos = torch.arange(40, dtype=F64)
    t = plain.query_temperature(pos, 0.5, 8)
    assert torch.all(t[:7] == 1.0) and float(t[7]) == pytest.approx(1 + 0.5 * math.log(2)) and float(t[14]) == float(t[7])
    assert float(t[15]) == pytest.approx(1 + 0.5 * math.log(3))


def test_linear_attention_reads_back_what_it_wrote_with_the_decay():
    """One head, identity projections: the token whose key equals the query comes back, times decay^distance."""
    W = 4
    w = {"q": torch.eye(W, dtype=F64), "k": torch.eye(W, dtype=F64), "v": torch.eye(W, dtype=F64), "g": torch.zeros(W, W, dtype=F64),
         "norm": torch.ones(W, dtype=F64), "o": torch.eye(W, dtype=F64)}
    m = {"heads": 1, "dim": W, "vdim": W, "decay": [0.5]}
    h = torch.zeros(6, W, dtype=F64)
    h[1, 0] = 30.0          # silu(30) = 30: key, query and value along channel 0
    h[4, 0] = 30.0
    out = plain.lightning(h, w, "", m, 0.0)
    # at token 4 the state holds 0.5^3 * k1 v1 + k4 v4; the read-out is normed, so only its direction shows
    assert float(out[4, 0]) > 0 and float(out[4, 1:].abs().max()) < 1e-9
    S = torch.zeros(W, W, dtype=F64)
    k = plain.silu(h)
    for t in range(5):
        S = 0.5 * S + torch.outer(k[t], k[t])
    assert float(S[0, 0]) == pytest.approx(float(k[1, 0]) ** 2 * 0.125 + float(k[4, 0]) ** 2, rel=1e-6)


def test_matrix_memory_starts_its_maximum_at_zero():
    """With the maximum starting at minus infinity the first token's write would be scaled to one whatever its input gate."""
    cfg = u.config([u.parallel_layer()], taps=0)
    w = u.as_float64(u.make_weights(cfg, 1))
    m = cfg["layers"][0]["mixer"]["right"]
    h = rand(1, cfg["width"])
    w = dict(w)
    w["l0.mix.right.i.b"] = torch.full_like(w["l0.mix.right.i.b"], -5.0)       # i far below 0: m stays 0, the write is exp(i)
    out = plain.matrix_memory(h, w, "l0.mix.right.", m, 1e-6)
    w["l0.mix.right.i.b"] = torch.full_like(w["l0.mix.right.i.b"], -6.0)
    out2 = plain.matrix_memory(h, w, "l0.mix.right.", m, 1e-6)
    assert not torch.allclose(out, out2, rtol=1e-3), "a maximum that started at minus infinity would hide the input gate"


def test_lru_gate_of_one_forgets_nothing_and_takes_nothing():
    a = torch.exp(-8.0 * torch.tensor(0.0, dtype=F64) * plain.softplus(torch.tensor(1.0, dtype=F64)))
    assert float(a) == 1.0 and float(torch.sqrt(1 - a * a)) == 0.0


def test_experts_clamp_and_weights_act_on_the_input():
    W, F = 6, 5
    w = {"e0.gate": rand(F, W, seed=1) * 3, "e0.up": rand(F, W, seed=2) * 3, "e0.down": rand(W, F, seed=3)}
    x = rand(1, W, seed=4)
    y = plain.expert(x, w, "e0.", 0.7)
    g = torch.clamp(x @ w["e0.gate"].T, max=0.7)
    up = torch.clamp(x @ w["e0.up"].T, -0.7, 0.7)
    assert torch.allclose(y, (g * plain.sigmoid(1.702 * g) * (up + 1)) @ w["e0.down"].T)
    assert not torch.allclose(plain.expert(0.5 * x, w, "e0.", 0.7), 0.5 * y), "an expert is not linear: where the weight acts matters"


def test_the_largest_scores_are_chosen_and_kept_as_weights():
    scores = torch.tensor([[0.1, 0.9, 0.5, 0.9], [0.3, 0.2, 0.8, 0.1]], dtype=F64)
    ids, weights = plain.choose(scores, 2)
    assert ids.tolist() == [[1, 3], [2, 0]] and weights.tolist() == [[0.9, 0.9], [0.8, 0.3]]


def test_the_plain_model_is_causal_and_depends_on_every_mechanism():
    cfg = u.CFG_MAIN
    w = u.as_float64(u.make_weights(cfg, 3))
    tokens = u.random_tokens(cfg["vocab"], 30, 1)
    base = plain.forward(cfg, w, tokens)
    assert torch.allclose(plain.forward(cfg, w, tokens[:17]), base[:17], atol=1e-9)
    spread = float(base.std())
    for name in ("pos", "l0.canon1", "l0.rg1.b", "l0.mix.left.g", "l0.mix.right.i.b", "l0.mix.left.out", "l1.mix.lam", "l1.mix.ra.b",
                 "l2.mix.norm", "l2.mlp.router", "l3.mix.right.norm", "l4.mix.conv.b", "final.norm.b"):
        w2 = dict(w)
        w2[name] = w[name] * 1.5 + torch.linspace(0.0, 0.5, w[name].numel(), dtype=F64).view_as(w[name])     # (no uniform shift: the norms take a row's mean off)
        assert float((plain.forward(cfg, w2, tokens) - base).abs().max()) > 1e-3 * spread, name


# ---------------------------------------------------------------------------
# configuration and description
# ---------------------------------------------------------------------------
def test_configuration_reads_every_size_and_constant():
    from ferrox_amd.config.panarax import PanaraxConfig
    cfg = PanaraxConfig.from_dict(copy.deepcopy(u.CFG_MAIN))
    assert (cfg.vocab, cfg.width, cfg.eps, cfg.canon_taps, cfg.max_positions) == (150, 48, 1e-5, 3, 512)
    assert [layer.type for layer in cfg.layers] == ["parallel", "rglru", "lightning", "parallel", "rglru", "lightning"]
    left = cfg.layers[0].mixer.left
    assert (left.heads, left.kv_heads, left.dim, left.vdim, left.scale, left.q_temp) == (4, 2, 8, 12, 0.5, (0.4, 5))
    assert cfg.layers[2].mixer.decay == (0.6, 0.93, 1.0) and cfg.layers[3].mlp is None
    assert (cfg.layers[4].mlp.experts, cfg.layers[4].mlp.top, cfg.layers[4].mlp.ff, cfg.layers[4].mlp.limit) == (4, 1, 32, 3.0)
    assert cfg.to_dict()["layers"] == u.CFG_MAIN["layers"]


@pytest.mark.parametrize("change, message", [
    (lambda c: c["layers"][0].update(type="conv"), "type 'conv'"),
    (lambda c: c["layers"][1]["mixer"].update(blocks=7), "equal blocks"),
    (lambda c: c["layers"][2]["mixer"].update(decay=[0.5, 0.5]), "decay"),
    (lambda c: c["layers"][2]["mixer"].update(decay=[0.5, 1.5, 0.2]), "decay"),
    (lambda c: c["layers"][0]["mixer"]["left"].update(kv_heads=3), "multiple of kv_heads"),
    (lambda c: c["layers"][0]["mlp"]["router"].update(top=9), "top 9"),
    (lambda c: c["layers"][1]["mlp"].update(kind="shared"), "kind 'shared'"),
    (lambda c: c.pop("max_positions"), "max_positions"),
    (lambda c: c["layers"][3]["mixer"]["right"].update(dim=300), "256 key channels"),
    (lambda c: c["canon"].update(taps=40), "16 taps"),
])
def test_configuration_refuses(change, message):
    from ferrox_amd.config.base import ConfigError
    from ferrox_amd.config.panarax import PanaraxConfig
    raw = copy.deepcopy(u.CFG_MAIN)
    change(raw)
    with pytest.raises(ConfigError, match=message):
        PanaraxConfig.from_dict(raw)


@pytest.mark.parametrize("cfg", [u.CFG_MAIN, u.CFG_MFMA, u.config([u.rglru_layer(mlp=u.dense())], taps=0)])
def test_description_names_the_designs_tensors(cfg):
    from ferrox_amd.engine.model import Model
    from ferrox_amd.models.registry import resolve
    arch = resolve(cfg)
    assert arch.name == "Panarax"
    model = Model(arch.build_spec(arch.config_class.from_dict(copy.deepcopy(cfg)), None))
    got = {name: tuple(spec.shape) for name, spec in model.named_params().items()}
    assert got == u.tensor_shapes(cfg)
    assert all(b.mixer.graph_safe for b in model.blocks), "decode steps of this design are recorded"
    assert model.cache_groups() == ({("full",): None} if any(layer["type"] == "parallel" for layer in cfg["layers"]) else {})


def test_the_named_shape_is_a_configuration_of_the_design():
    from ferrox_amd.config import presets
    from ferrox_amd.config.panarax import PanaraxConfig
    cfg = PanaraxConfig.from_dict(presets.load("panarax-2k"))
    assert {layer.type for layer in cfg.layers} == {"rglru", "lightning", "parallel"} and cfg.width == 2048
