"""Panarax on the GPU against the plain model (`plain_panarax`): every mechanism alone, the new kernels alone, whole
prompts, decoding through cache and state, portions down to two tokens, unequal batches, pages and slots used again,
keys far away and at page borders, temperature steps in prompts and in decoding, states written far back, long
decoding, other sizes, and generation through the engine's entry points."""
import contextlib
import math

import pytest
import torch

import panarax_util as u
import plain_panarax as plain

pytestmark = pytest.mark.gpu

_models = {}
F64 = torch.float64


def model_for(tmp_path_factory, name, cfg, seed, dtype, change=None):
    """(weights as the plain model reads them, loaded engine model); made once per (name, dtype)."""
    from ferrox_amd.engine.loading import load_model
    key = (name, dtype)
    if key not in _models:
        weights = u.make_weights(cfg, seed)
        if change:
            change(weights)
        folder = u.write_model(str(tmp_path_factory.mktemp(f"panarax_{name}")), cfg, weights)
        _models[key] = (weights, load_model(folder, dtype, "cuda:0"))
    return _models[key]


def runner_of(model, block_size=16, num_pages=24, max_seqs=4, **kw):
    from ferrox_amd.engine.runner import ModelRunner
    return ModelRunner(model, block_size=block_size, num_pages=num_pages, max_seqs=max_seqs, **kw)


def tracing(dtype):
    from ferrox_amd import debug
    return debug.trace_routing() if dtype == "bfloat16" else contextlib.nullcontext()


def run_and_check(cfg, weights, model, requests, schedule, dtype, what, limit=None, **runner_kw):
    runner = runner_of(model, **runner_kw)
    with tracing(dtype) as trace:
        got, chosen = u.run_schedule(runner, requests, schedule, trace=trace)
    for key in runner.manager.groups:
        assert runner.manager.n_free_pages(key) == runner_kw.get("num_pages", 24), "pages were lost"
    return u.check_against_plain(cfg, weights, requests, got, dtype, chosen, what, limit)


# ---------------------------------------------------------------------------
# each mechanism alone: models of one layer
# ---------------------------------------------------------------------------
SINGLE = {
    "lru": u.config([u.rglru_layer(width=48, blocks=3, conv=3)]),
    "lru_one_block_one_tap": u.config([u.rglru_layer(width=40, blocks=1, conv=1)], taps=1),
    "lru_many_blocks": u.config([u.rglru_layer(width=60, blocks=12, conv=5)], taps=5),
    "lightning": u.config([u.lightning_layer(heads=3, dim=8, vdim=12)]),
    "lightning_no_decay_one_head": u.config([u.lightning_layer(heads=1, dim=16, vdim=8, decay=[1.0])], taps=2),
    "side_by_side": u.config([u.parallel_layer()]),
    "side_by_side_no_temperature": u.config([u.parallel_layer(heads=2, kv_heads=2, dim=16, vdim=16, every=0, r_heads=1, r_dim=16, r_vdim=8)]),
    "side_by_side_one_key_head": u.config([u.parallel_layer(heads=6, kv_heads=1, dim=8, vdim=20, every=3, coef=1.5, r_heads=4, r_dim=4, r_vdim=4,
                                                            gate_cap=3.0)]),
    "no_input_convolution": u.config([u.lightning_layer(mlp=u.dense(24))], taps=0),
    "dense": u.config([u.lightning_layer(mlp=u.dense(56))]),
    "experts_one": u.config([u.lightning_layer(mlp=u.moe(5, 1, 16, 1.0))]),
    "experts_three": u.config([u.rglru_layer(mlp=u.moe(7, 3, 24, 0.6))]),
    "experts_all": u.config([u.rglru_layer(mlp=u.moe(3, 3, 8, 50.0))]),
}


@pytest.mark.parametrize("name", sorted(SINGLE))
def test_each_mechanism_alone(tmp_path_factory, name):
    cfg = SINGLE[name]
    for dtype in ("float32", "bfloat16"):
        weights, model = model_for(tmp_path_factory, name, cfg, 11, dtype)
        reqs = {"a": u.random_tokens(cfg["vocab"], 45, 1), "b": u.random_tokens(cfg["vocab"], 19, 2)}
        run_and_check(cfg, weights, model, reqs, [[("a", 45)], [("b", 19)]], dtype, name + " whole")
        cut = [[("a", 17), ("b", 2)], [("a", 1), ("b", 16)], [("a", 20), ("b", 1)]] + [[("a", 1)]] * 7
        run_and_check(cfg, weights, model, reqs, cut, dtype, name + " cut")


def test_the_plain_model_moves_when_a_mechanism_is_left_out(tmp_path_factory):
    """What the comparisons above can see: the plain model without one mechanism is far beyond the limit."""
    cfg = u.CFG_MAIN
    weights = u.make_weights(cfg, 3)
    w = u.as_float64(weights)
    tokens = u.random_tokens(cfg["vocab"], 60, 5)
    base = plain.forward(cfg, w, tokens)

    def moved(other_cfg=None, **replace):
        w2 = dict(w, **replace)
        return float(u.row_errors(plain.forward(other_cfg or cfg, w2, tokens), base).max())

    zero = lambda name: {name: torch.zeros_like(w[name])}
    assert moved(**zero("pos")) > 100 * u.LIMIT["bfloat16"] / 10
    assert moved(**zero("l0.canon1")) > u.EDGE_LIMIT["bfloat16"]
    assert moved(**{"l0.rg1": torch.zeros_like(w["l0.rg1"]), "l0.rg1.b": torch.full_like(w["l0.rg1.b"], 30.0)}) > u.EDGE_LIMIT["bfloat16"]
    assert moved(u.changed(cfg, 0, left__q_temp=None)) > u.EDGE_LIMIT["bfloat16"]
    assert moved(u.changed(cfg, 2, decay=[1.0, 1.0, 1.0])) > u.EDGE_LIMIT["bfloat16"]
    assert moved(u.changed(cfg, 3, right__gate_cap=0.5)) > u.EDGE_LIMIT["bfloat16"]
    no_limit = {**cfg, "layers": [dict(layer) for layer in cfg["layers"]]}
    no_limit["layers"][2] = {**cfg["layers"][2], "mlp": u.moe(5, 3, 24, 1e9)}
    assert moved(no_limit) > u.EDGE_LIMIT["bfloat16"]


# ---------------------------------------------------------------------------
# the new kernels alone, against torch in float64
# ---------------------------------------------------------------------------
def starts_of(lengths):
    s = [0]
    for n in lengths:
        s.append(s[-1] + n)
    return torch.tensor(s, dtype=torch.int32, device="cuda")


@pytest.mark.parametrize("H, G, D, V, normalizer", [(3, 3, 8, 12, False), (4, 2, 20, 7, True), (2, 2, 128, 64, True), (2, 1, 130, 40, False),
                                                     (1, 1, 64, 33, True), (2, 2, 6, 5, True)])
def test_gated_outer_product_recurrence(H, G, D, V, normalizer):
    """Portions of three sequences in one launch, from states that an earlier launch left, against a loop."""
    from ferrox_amd import ops
    gen = torch.Generator().manual_seed(H * 100 + D)
    lengths, slots = [37, 1, 9], [2, 0, 3]
    T = sum(lengths)
    q, k = (torch.randn(T, G * D, generator=gen) for _ in range(2))
    v = torch.randn(T, H * V, generator=gen)
    keep, take = torch.rand(T, H, generator=gen) * 0.5 + 0.5, torch.rand(T, H, generator=gen) + 0.2
    VS = V + (1 if normalizer else 0)
    state0 = torch.randn(5, H, VS, D, generator=gen)
    state = state0.clone().cuda()
    out = ops.gated_outer(q.cuda(), k.cuda(), v.cuda(), keep.cuda(), take.cuda(), state, starts_of(lengths),
                          torch.tensor(slots, dtype=torch.int32, device="cuda"), 3, H, G, D, V, q_scale=0.7, normalizer=normalizer)
    o, nq = out if normalizer else (out, None)
    t0 = 0
    for n, slot in zip(lengths, slots):
        S = state0[slot].to(F64).clone()                               # [H, VS, D]
        for t in range(t0, t0 + n):
            for h in range(H):
                g = h // (H // G)
                kk, qq = k[t, g * D:(g + 1) * D].to(F64), q[t, g * D:(g + 1) * D].to(F64)
                vv = v[t, h * V:(h + 1) * V].to(F64)
                if normalizer:
                    vv = torch.cat([vv, torch.ones(1, dtype=F64)])
                S[h] = float(keep[t, h]) * S[h] + float(take[t, h]) * vv[:, None] * kk[None, :]
                read = 0.7 * (S[h] @ qq)
                assert torch.allclose(o[t, h * V:(h + 1) * V].cpu().to(F64), read[:V], rtol=2e-5, atol=2e-5), (t, h)
                if normalizer:
                    assert float(nq[t, h]) == pytest.approx(float(read[V]), rel=2e-5, abs=2e-5)
        assert torch.allclose(state[slot].cpu().to(F64), S, rtol=2e-5, atol=2e-5)
        t0 += n
    assert torch.equal(state[1].cpu(), state0[1]) and torch.equal(state[4].cpu(), state0[4]), "a slot of no sequence was written"
    # the same factor at every token, no writing factor: what linear attention with a constant decay asks for
    if not normalizer:
        decay = torch.rand(H, generator=gen) * 0.5 + 0.5
        s1, s2 = state0.clone().cuda(), state0.clone().cuda()
        a = ops.gated_outer(q.cuda(), k.cuda(), v.cuda(), decay.cuda(), None, s1, starts_of(lengths),
                            torch.tensor(slots, dtype=torch.int32, device="cuda"), 3, H, G, D, V)
        b = ops.gated_outer(q.cuda(), k.cuda(), v.cuda(), decay[None, :].expand(T, H).contiguous().cuda(), torch.ones(T, H).cuda(), s2,
                            starts_of(lengths), torch.tensor(slots, dtype=torch.int32, device="cuda"), 3, H, G, D, V)
        assert torch.equal(a, b) and torch.equal(s1, s2)


def test_exponential_gates_under_a_running_maximum():
    """Sequences longer than a wave's 64 tokens, a continued one, and gates far outside the cap."""
    from ferrox_amd import ops
    gen = torch.Generator().manual_seed(5)
    H, cap = 3, 4.0
    lengths, slots = [150, 1, 64, 65], [1, 3, 0, 2]
    T = sum(lengths)
    xi, xf = torch.randn(T, H, generator=gen) * 6, torch.randn(T, H, generator=gen) * 6 + 2
    m0 = torch.tensor([[0.0] * H, [0.3, -1.0, 2.0], [0.0] * H, [1.0, 0.5, -0.2]])
    state = m0.clone().cuda()
    keep, take, m = ops.exp_gate_scan(xi.cuda(), xf.cuda(), cap, state, starts_of(lengths),
                                      torch.tensor(slots, dtype=torch.int32, device="cuda"), 4, H)
    t0 = 0
    for n, slot in zip(lengths, slots):
        mx = m0[slot].to(F64)
        for t in range(t0, t0 + n):
            i = cap * torch.tanh(xi[t].to(F64) / cap)
            f = plain.logsigmoid(cap * torch.tanh(xf[t].to(F64) / cap))
            new = torch.maximum(f + mx, i)
            assert torch.allclose(m[t].cpu().to(F64), new, rtol=1e-5, atol=1e-5), t
            assert torch.allclose(keep[t].cpu().to(F64), torch.exp(f + mx - new), rtol=2e-5, atol=1e-6), t
            assert torch.allclose(take[t].cpu().to(F64), torch.exp(i - new), rtol=2e-5, atol=1e-6), t
            mx = new
        assert torch.allclose(state[slot].cpu().to(F64), mx, rtol=1e-5, atol=1e-5)
        t0 += n


@pytest.mark.parametrize("C, parts, lengths", [(48, 3, [5, 1, 300]), (70, 7, [1, 1, 1]), (256, 2, [17, 700, 40])])
def test_gated_linear_recurrent_unit(C, parts, lengths):
    from ferrox_amd import ops
    gen = torch.Generator().manual_seed(C)
    slots = [2, 0, 1]
    T, cb = sum(lengths), C // parts
    u_in, branch = torch.randn(T, C, generator=gen), torch.randn(T, C, generator=gen)
    logits, bias = torch.randn(T, parts, 2, cb, generator=gen), torch.randn(parts, 2, cb, generator=gen)
    lam = torch.randn(C, generator=gen) - 2.5
    state0 = torch.randn(4, C, generator=gen)
    state = state0.clone().cuda()
    y = ops.rglru(u_in.cuda(), logits.cuda(), bias.cuda(), parts, lam.cuda(), branch.cuda(), state, starts_of(lengths),
                  torch.tensor(slots, dtype=torch.int32, device="cuda"), 3, max(lengths), torch.float32)
    full = (logits + bias).to(F64)
    r = plain.sigmoid(full[:, :, 0, :].reshape(T, C))
    i = plain.sigmoid(full[:, :, 1, :].reshape(T, C))
    a = torch.exp(-8.0 * r * plain.softplus(lam.to(F64)))
    x = torch.sqrt(1 - a * a) * i * u_in.to(F64)
    t0 = 0
    for n, slot in zip(lengths, slots):
        S = state0[slot].to(F64)
        for t in range(t0, t0 + n):
            S = a[t] * S + x[t]
            assert torch.allclose(y[t].cpu().to(F64), S * plain.gelu_tanh(branch[t].to(F64)), rtol=3e-5, atol=3e-5), t
        assert torch.allclose(state[slot].cpu().to(F64), S, rtol=3e-5, atol=3e-5)
        t0 += n


@pytest.mark.parametrize("H, V, per_head, den", [(3, 20, True, True), (1, 1500, False, False), (2, 640, True, True), (4, 64, False, False)])
def test_read_out_norm_with_weights_per_head_and_denominators(H, V, per_head, den):
    """Short rows (a wave each) and long ones (a block each), a weight per head and channel, the memory's denominators."""
    from ferrox_amd import ops
    gen = torch.Generator().manual_seed(V)
    T = 5
    o, gate = torch.randn(T, H * V, generator=gen), torch.randn(T, H * V, generator=gen)
    w = torch.randn(H * V if per_head else V, generator=gen)
    nq, m = torch.randn(T, H, generator=gen) * 2, torch.randn(T, H, generator=gen)
    y = ops.gated_head_norm(o.cuda(), gate.cuda(), w.cuda(), 1e-5, H, V, torch.float32,
                            denominators=(nq.cuda(), m.cuda()) if den else None)
    x = o.to(F64).view(T, H, V)
    if den:
        x = x / (torch.maximum(nq.to(F64).abs(), torch.exp(-m.to(F64))) + 1e-6)[:, :, None]
    want = plain.unit_rms(x, 1e-5) * (w.to(F64).view(H, V) if per_head else w.to(F64)) * plain.sigmoid(gate.to(F64).view(T, H, V))
    assert torch.allclose(y.cpu().to(F64), want.reshape(T, H * V), rtol=2e-5, atol=2e-5)


def test_block_diagonal_product_for_few_rows():
    """The small launch of a decode step gives what the grouped product gives for many rows."""
    from ferrox_amd import ops
    from ferrox_amd.parts.latent import head_groups
    gen = torch.Generator().manual_seed(4)
    for T, parts, K, N in ((1, 3, 16, 32), (7, 5, 80, 160), (32, 2, 300, 70)):
        x = torch.randn(T, parts * K + 3, generator=gen).cuda()[:, :parts * K]
        w = torch.randn(parts, N, K, generator=gen).cuda()
        got = ops.small_rows_parts(x, w.transpose(1, 2).contiguous())
        want = torch.einsum("tjk,jnk->tjn", x.cpu().to(F64).view(T, parts, K), w.cpu().to(F64))
        assert torch.allclose(got.cpu().to(F64), want, rtol=1e-5, atol=1e-4)
        rows, offsets = head_groups("cuda:0", T, parts)
        tiled = torch.empty(T * parts, N, device="cuda")
        ops.gemm(x.contiguous().view(T * parts, K), w, a_rows=rows, c_rows=rows, expert_offsets=offsets, n_rows=T * parts,
                 epilogue=ops.EPI_STORE_F32, out=tiled)
        assert torch.equal(got.view(T * parts, N), tiled), "few rows and many rows round differently"


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_layer_norm_gated_add_and_position_table(dtype):
    from ferrox_amd import ops
    gen = torch.Generator().manual_seed(1)
    h = (torch.randn(7, 70, generator=gen) * 3 + 1).cuda()
    w, b = torch.randn(70, generator=gen).cuda(), torch.randn(70, generator=gen).cuda()
    rows = torch.tensor([5, 0, 5], dtype=torch.int32, device="cuda")
    want = plain.layer_norm(h.cpu().to(F64), w.cpu().to(F64), b.cpu().to(F64), 1e-5)
    tol = dict(rtol=1e-5, atol=1e-5) if dtype == torch.float32 else dict(rtol=1e-2, atol=1e-2)
    assert torch.allclose(ops.layernorm(h, w, b, 1e-5, dtype).cpu().to(F64), want, **tol)
    assert torch.allclose(ops.layernorm(h, w, b, 1e-5, dtype, rows=rows).cpu().to(F64), want[[5, 0, 5]], **tol)
    wide = (torch.randn(3, 4500, generator=gen) * 2 - 1).cuda()        # (rows beyond what a block keeps in registers)
    ww, wb = torch.randn(4500, generator=gen).cuda(), torch.randn(4500, generator=gen).cuda()
    assert torch.allclose(ops.layernorm(wide, ww, wb, 1e-6, dtype).cpu().to(F64),
                          plain.layer_norm(wide.cpu().to(F64), ww.cpu().to(F64), wb.cpu().to(F64), 1e-6), **tol)
    y, g = torch.randn(7, 70, generator=gen).cuda(), torch.randn(7, 70, generator=gen).cuda() * 3
    out = h.clone()
    ops.gated_add(out, y, g)
    assert torch.allclose(out.cpu().to(F64), h.cpu().to(F64) + y.cpu().to(F64) * plain.sigmoid(g.cpu().to(F64)), rtol=1e-6, atol=1e-6)
    # the add and the norm behind it as one launch: the bits of the two launches
    both = h.clone()
    normed = ops.gated_add_layernorm(both, y, g, w, b, 1e-5, dtype)
    assert torch.equal(both, out) and torch.equal(normed, ops.layernorm(out, w, b, 1e-5, dtype))
    table, pos = torch.randn(20, 70, generator=gen).to(dtype).cuda(), torch.randn(9, 70, generator=gen).to(dtype).cuda()
    ids = torch.tensor([3, 19, 0, 3], dtype=torch.int32, device="cuda")
    places = torch.tensor([0, 8, 2, 2], dtype=torch.int32, device="cuda")
    got = ops.embed(table, ids, position_table=pos, positions=places)
    assert torch.equal(got, table[ids.long()].float() + pos[places.long()].float())


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_short_convolution_with_bias_and_its_input_added(dtype):
    """The generalised convolution: no activation, a bias, the input added, rows of either type, taps of 1 to 5."""
    from ferrox_amd import ops
    gen = torch.Generator().manual_seed(2)
    lengths, slots = [6, 1, 11], [1, 2, 0]
    T, C = sum(lengths), 37
    for taps in (1, 2, 3, 4, 5):
        x = torch.randn(T, C, generator=gen).to(dtype)
        w, bias = torch.randn(C, taps, generator=gen), torch.randn(C, generator=gen)
        state0 = torch.randn(3, C, taps - 1, generator=gen)
        state = state0.clone().cuda()
        y = ops.short_conv(x.cuda(), w.cuda(), state, torch.tensor([0] * 6 + [1] + [2] * 11, dtype=torch.int32, device="cuda"),
                           starts_of(lengths), torch.tensor(slots, dtype=torch.int32, device="cuda"), 3, activation=None,
                           bias=bias.cuda(), add_input=True, out_dtype=dtype)
        t0 = 0
        for n, slot in zip(lengths, slots):
            hist = torch.cat([state0[slot].t().to(F64), x[t0:t0 + n].to(F64)])          # [taps - 1 + n, C]
            for i in range(n):
                want = (w.to(F64).t() * hist[i:i + taps]).sum(0) + bias.to(F64) + x[t0 + i].to(F64)
                tol = dict(rtol=1e-5, atol=1e-5) if dtype == torch.float32 else dict(rtol=2e-2, atol=2e-2)
                assert torch.allclose(y[t0 + i].cpu().to(F64), want, **tol), (taps, t0 + i)
            if taps > 1:
                assert torch.allclose(state[slot].cpu().to(F64), hist[n:].t(), atol=1e-6), taps
            t0 += n


@pytest.mark.parametrize("dtype, nh, nkv, hd, vd, bs", [(torch.float32, 4, 2, 8, 12, 16), (torch.bfloat16, 4, 1, 64, 64, 64),
                                                        (torch.bfloat16, 2, 2, 24, 40, 16), (torch.float32, 3, 3, 130, 200, 8)])
def test_temperature_unit_values_and_cache_write(dtype, nh, nkv, hd, vd, bs):
    from ferrox_amd import ops
    gen = torch.Generator().manual_seed(nh + hd)
    positions = list(range(29, 29 + 21)) + [0, 7]                         # a portion across page borders, two single tokens
    seqs = [0] * 21 + [1, 2]
    T = len(positions)
    cols = (nh + nkv) * hd + nkv * vd + nh
    qkv = torch.randn(T, cols, generator=gen).cuda()
    table = torch.tensor([[3, 5, 1, 6], [2, 0, 0, 0], [4, 0, 0, 0]], dtype=torch.int32, device="cuda")
    if bs == 8:
        table = torch.tensor([[3, 5, 1, 6, 7, 8, 9], [2] + [0] * 6, [4] + [0] * 6], dtype=torch.int32, device="cuda")
    k_pages = torch.zeros(10, nkv, bs, hd, dtype=dtype, device="cuda")
    v_pages = torch.zeros(10, nkv, vd, bs, dtype=dtype, device="cuda")
    q_out = torch.zeros(T, nh * hd + nh, dtype=dtype, device="cuda")
    ops.temp_unit_kv_write(qkv, q_out, torch.tensor(positions, dtype=torch.int32, device="cuda"),
                           torch.tensor(seqs, dtype=torch.int32, device="cuda"), table, k_pages, v_pages, nh, nkv, hd, vd, bs,
                           n_gate=nh, temperature=(0.6, 5), unit_values=True, eps=1e-5)
    x = qkv.cpu().to(F64)
    temp = plain.query_temperature(torch.tensor(positions, dtype=F64), 0.6, 5)
    tol = dict(rtol=1e-5, atol=1e-5) if dtype == torch.float32 else dict(rtol=1e-2, atol=1e-2)
    assert torch.allclose(q_out[:, :nh * hd].cpu().to(F64), x[:, :nh * hd] * temp[:, None], **tol)
    assert torch.allclose(q_out[:, nh * hd:].cpu().to(F64), x[:, cols - nh:], **tol)
    for t, (p, s) in enumerate(zip(positions, seqs)):
        page = int(table[s, p // bs])
        k = x[t, nh * hd:(nh + nkv) * hd].view(nkv, hd)
        v = plain.unit_rms(x[t, (nh + nkv) * hd:cols - nh].view(nkv, vd), 1e-5)
        assert torch.allclose(k_pages[page, :, p % bs, :].cpu().to(F64), k, **tol), t
        assert torch.allclose(v_pages[page, :, :, p % bs].cpu().to(F64), v, **tol), t


# ---------------------------------------------------------------------------
# whole models: prompts, decoding, portions, batches
# ---------------------------------------------------------------------------
def main_requests():
    V = u.CFG_MAIN["vocab"]
    return {"r97": u.random_tokens(V, 97, 1), "r23": u.random_tokens(V, 23, 2), "r1": u.random_tokens(V, 1, 3),
            "r50": u.random_tokens(V, 50, 4), "r2": u.random_tokens(V, 2, 5)}


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_whole_prompts_and_decoding(tmp_path_factory, dtype):
    weights, model = model_for(tmp_path_factory, "main", u.CFG_MAIN, 3, dtype)
    reqs = main_requests()
    run_and_check(u.CFG_MAIN, weights, model, reqs, [[(r, len(t))] for r, t in reqs.items()], dtype, "whole")
    # most of a prompt in one step, the last 40 tokens (or all but one) one by one: states and convolutions are carried
    # on, the temperature steps every 5 and 16 positions under decoded tokens, keys cross the page borders at 16, 32, ...
    sched = []
    for r, t in reqs.items():
        first = max(1, len(t) - 40)
        sched += [[(r, first)]] + [[(r, 1)]] * (len(t) - first)
    run_and_check(u.CFG_MAIN, weights, model, reqs, sched, dtype, "decode")
    # token by token from the first token on: states that start at zero, convolutions that look before the start
    one = {"r50": reqs["r50"]}
    run_and_check(u.CFG_MAIN, weights, model, one, [[("r50", 1)]] * 50, dtype, "token by token")


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_portions_of_changing_size(tmp_path_factory, dtype):
    weights, model = model_for(tmp_path_factory, "main", u.CFG_MAIN, 3, dtype)
    reqs = main_requests()
    sizes = [2, 5, 2, 16, 1, 7, 24, 3, 2, 17, 1, 1, 9]
    sched = []
    for r, t in reqs.items():
        left, i = len(t), 0
        while left:
            n = min(sizes[i % len(sizes)], left)
            sched.append([(r, n)])
            left -= n
            i += 1
    run_and_check(u.CFG_MAIN, weights, model, reqs, sched, dtype, "portions")


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_unequal_batches_with_pages_and_slots_used_again(tmp_path_factory, dtype):
    """Up to three live requests under three slots and a pool of 14 pages of 16 (the requests' sum needs 18):
    portions beside single tokens, requests that pause, slots (and the states in them) and pages taken again."""
    weights, model = model_for(tmp_path_factory, "main", u.CFG_MAIN, 3, dtype)
    reqs = main_requests()
    reqs["s40"] = u.random_tokens(u.CFG_MAIN["vocab"], 40, 7)
    sched = [
        [("r97", 30), ("r23", 2), ("r1", 1)],
        [("r97", 3), ("r23", 1), ("r2", 2)],                    # r1's slot goes to r2
        [("r97", 1), ("r23", 18)],
        [("r23", 1), ("r50", 21)],                              # r97 pauses
        [("r97", 40), ("r23", 1), ("r50", 1)],                  # r23 ends
        [("r97", 1), ("r50", 27), ("s40", 2)],
        [("r97", 22), ("r50", 1), ("s40", 37)],                 # r97 and r50 end
        [("s40", 1)],
    ]
    run_and_check(u.CFG_MAIN, weights, model, reqs, sched, dtype, "mixed", num_pages=14, max_seqs=3)
    alone = runner_of(model, num_pages=14, max_seqs=3)
    mixed = runner_of(model, num_pages=14, max_seqs=3)
    got_alone, _ = u.run_schedule(alone, reqs, [[(r, len(t))] for r, t in reqs.items()])
    got_mixed, _ = u.run_schedule(mixed, reqs, sched)
    for r in reqs:
        assert float(u.row_errors(got_mixed[r], got_alone[r]).max()) <= u.EDGE_LIMIT[dtype], r


def test_one_slot_for_requests_in_a_row(tmp_path_factory):
    """One slot and ten pages: every request takes the slot, the states and the pages that the one before left."""
    weights, model = model_for(tmp_path_factory, "main", u.CFG_MAIN, 3, "float32")
    V = u.CFG_MAIN["vocab"]
    reqs = {"z": u.random_tokens(V, 150, 2), "y": u.random_tokens(V, 60, 3), "x": u.random_tokens(V, 5, 4)}
    sched = [[("z", 8)]] * 17 + [[("z", 1)]] * 14 + [[("y", 7)]] * 8 + [[("y", 2)]] * 2 + [[("x", 2)], [("x", 1)], [("x", 2)]]
    run_and_check(u.CFG_MAIN, weights, model, reqs, sched, "float32", "one slot", num_pages=10, max_seqs=1)


# ---------------------------------------------------------------------------
# where a fault hides behind random weights
# ---------------------------------------------------------------------------
@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_a_far_key_among_hundreds_and_keys_at_page_borders(tmp_path_factory, dtype):
    """Queries and keys of the attention scaled up: the softmax is peaked, so single keys carry the output, and a key
    that is lost (a page's first or last slot, a key hundreds back, the query's own) moves the logits.  The temperature
    steps every 50 positions, in the prompt and under decoded tokens."""
    cfg = u.config([u.parallel_layer(heads=4, kv_heads=2, dim=16, vdim=16, scale=0.25, coef=0.8, every=50, r_heads=2, r_dim=8, r_vdim=8,
                                     mlp=u.dense(32))], width=64, max_positions=600)

    # (bfloat16 rounds the scores themselves, a 250th of their size: scores of some tens would differ by tenths)
    factor = 6 if dtype == "float32" else 2.5

    def peaked(w):
        w["l0.mix.left.q"] = (w["l0.mix.left.q"].float() * factor).to(torch.bfloat16)
        w["l0.mix.left.k"] = (w["l0.mix.left.k"].float() * factor).to(torch.bfloat16)

    weights, model = model_for(tmp_path_factory, "peaked", cfg, 21, dtype, change=peaked)
    reqs = {"long": u.random_tokens(cfg["vocab"], 420, 6)}
    limit = u.EDGE_LIMIT[dtype]
    run_and_check(cfg, weights, model, reqs, [[("long", 420)]], dtype, "peaked whole", limit=limit, num_pages=30)
    sched = [[("long", 330)]] + [[("long", 1)]] * 60 + [[("long", 2)]] * 15
    run_and_check(cfg, weights, model, reqs, sched, dtype, "peaked decode", limit=limit, num_pages=30)
    # the plain model one position off in the temperature's step is far beyond the float32 limit (the step changes the
    # sharpness of a softmax that is peaked already, which moves the logits by thousandths: float32 is the judge of it)
    w = u.as_float64(weights)
    base = plain.forward(cfg, w, reqs["long"])
    off = plain.forward(u.changed(cfg, 0, left__q_temp={"coef": 0.8, "every": 51}), w, reqs["long"])
    assert float(u.row_errors(off, base).max()) > 10 * u.EDGE_LIMIT["float32"]


def test_a_state_written_far_back(tmp_path_factory):
    """Heads that never forget (decay 1, a forget gate near one, a recurrence gate near zero): what token 3 wrote is
    read 200 tokens later, through portions and decoded tokens; with the token changed the last logits move."""
    cfg = u.config([u.lightning_layer(heads=2, dim=8, vdim=8, decay=[1.0, 0.999]), u.rglru_layer(width=32, blocks=2, conv=2),
                    u.parallel_layer(heads=2, kv_heads=1, dim=8, vdim=8, r_heads=2, r_dim=8, r_vdim=8)], width=32, max_positions=300)

    def slow(w):
        w["l1.mix.lam"] = torch.full_like(w["l1.mix.lam"], -9.0)
        w["l2.mix.right.f.b"] = torch.full_like(w["l2.mix.right.f.b"], 9.0)

    weights, model = model_for(tmp_path_factory, "far_state", cfg, 9, "float32", change=slow)
    tokens = u.random_tokens(cfg["vocab"], 210, 8)
    sched = [[("a", 2)], [("a", 60)], [("a", 1)], [("a", 100)]] + [[("a", 1)]] * 47
    run_and_check(cfg, weights, model, {"a": tokens}, sched, "float32", "far state", limit=u.EDGE_LIMIT["float32"])
    w = u.as_float64(weights)
    other = list(tokens)
    other[3] = (other[3] + 1) % cfg["vocab"]
    moved = u.row_errors(plain.forward(cfg, w, other)[-1:], plain.forward(cfg, w, tokens)[-1:])
    assert float(moved) > 100 * u.LIMIT["float32"], "the last token does not see the third"


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_long_decoding_on_the_matrix_units(tmp_path_factory, dtype):
    """Sizes that take the bfloat16 kernels' matrix-unit paths (head sizes in multiples of 16, widths in multiples of
    64, pages of 64): a prompt, then 140 tokens one by one from recorded steps, two requests decoding side by side."""
    weights, model = model_for(tmp_path_factory, "mfma", u.CFG_MFMA, 17, dtype)
    reqs = {"x": u.random_tokens(u.CFG_MFMA["vocab"], 300, 3), "y": u.random_tokens(u.CFG_MFMA["vocab"], 150, 4)}
    sched = [[("x", 160)], [("y", 10)]] + [[("x", 1), ("y", 1)]] * 140
    run_and_check(u.CFG_MFMA, weights, model, reqs, sched, dtype, "long decode", block_size=64, num_pages=10)
    whole = [[("x", 300), ("y", 150)]]
    run_and_check(u.CFG_MFMA, weights, model, reqs, whole, dtype, "whole", block_size=64, num_pages=10)
    cut = [[("x", 130), ("y", 3)], [("x", 2), ("y", 140)], [("x", 150), ("y", 7)], [("x", 18)]]
    run_and_check(u.CFG_MFMA, weights, model, reqs, cut, dtype, "portions", block_size=64, num_pages=10)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_sizes_that_fit_no_vector(tmp_path_factory, dtype):
    """Head sizes, widths and a vocabulary that are no multiples of 16, 8 or 4: the kernels' guarded paths."""
    cfg = u.config([u.parallel_layer(heads=3, kv_heads=3, dim=10, vdim=14, scale=0.6, every=4, r_heads=5, r_dim=6, r_vdim=10, mlp=u.moe(3, 2, 22, 1.2)),
                    u.lightning_layer(heads=5, dim=6, vdim=10, mlp=u.dense(30)),
                    u.rglru_layer(width=42, blocks=7, conv=5, mlp=u.moe(9, 4, 10, 2.0))], width=70, vocab=151, taps=5)
    weights, model = model_for(tmp_path_factory, "odd", cfg, 13, dtype)
    reqs = {"a": u.random_tokens(151, 45, 1), "b": u.random_tokens(151, 20, 2)}
    sched = [[("a", 30), ("b", 2)], [("a", 1), ("b", 17)]] + [[("a", 1), ("b", 1)]] + [[("a", 1)]] * 13
    run_and_check(cfg, weights, model, reqs, sched, dtype, "odd sizes")


# ---------------------------------------------------------------------------
# through the engine's own entry points: scheduler, sampling, recorded steps, command line, replay
# ---------------------------------------------------------------------------
def plain_greedy(cfg, weights, prompt, n):
    tokens, w = list(prompt), u.as_float64(weights)
    for _ in range(n):
        tokens.append(int(plain.forward(cfg, w, tokens)[-1].argmax()))
    return tokens[len(prompt):]


def test_greedy_generation_through_the_engine(tmp_path_factory):
    from ferrox_amd.engine.api import Engine
    weights, model = model_for(tmp_path_factory, "main", u.CFG_MAIN, 3, "float32")
    prompts = [u.random_tokens(u.CFG_MAIN["vocab"], n, 90 + n) for n in (3, 30, 1, 47)]
    want = [plain_greedy(u.CFG_MAIN, weights, p, 12) for p in prompts]
    assert len({t for w in want for t in w}) >= 6, "the expected continuations say too little"
    # steps of at most 16 tokens: prompts are cut into portions that run beside other requests' decoded tokens
    engine = Engine(model=model, block_size=16, num_pages=32, max_seqs=3, max_tokens_per_step=16, prefill_chunk=16)
    assert engine.generate(prompts, max_new_tokens=12, temperature=0.0, ignore_eos=True) == want
    # too few pages for all at once: requests wait, or are preempted and recomputed (their states start again)
    small = Engine(model=model, block_size=16, num_pages=6, max_seqs=4, max_tokens_per_step=32, prefill_chunk=32)
    assert small.generate(prompts, max_new_tokens=12, temperature=0.0, ignore_eos=True) == want


def test_command_line_and_replay(tmp_path_factory):
    import json
    import os
    import subprocess
    import sys

    import numpy as np
    from conftest import ROOT
    weights = u.make_weights(u.CFG_MAIN, 3)
    folder = u.write_model(str(tmp_path_factory.mktemp("panarax_cli")), u.CFG_MAIN, weights)
    prompt = u.random_tokens(u.CFG_MAIN["vocab"], 9, 77)
    want = plain_greedy(u.CFG_MAIN, weights, prompt, 6)
    out = subprocess.run([sys.executable, os.path.join(ROOT, "bin", "ferrox-amd"), "-m", folder, "--tokens",
                          ",".join(map(str, prompt)), "-n", "6", "--temp", "0", "--repeat-penalty", "1.0", "--ignore-eos", "--dtype", "float32",
                          "--block-size", "16", "--num-pages", "16"],
                         capture_output=True, text=True, timeout=300)
    assert out.returncode == 0, out.stderr[-2000:]
    assert ",".join(map(str, want)) in out.stdout.replace(" ", ""), (out.stdout[-500:], want)
    # random weights of the named shape, cut to three layers, through the command line
    out = subprocess.run([sys.executable, os.path.join(ROOT, "bin", "ferrox-amd"), "--random-weights", "--config", "panarax-2k", "--layers", "3",
                          "--tokens", "1,2,3,4,5", "-n", "4", "--temp", "0", "--ignore-eos", "--num-pages", "8"],
                         capture_output=True, text=True, timeout=300)
    assert out.returncode == 0, out.stderr[-2000:]
    # the step-by-step replay: two requests, a portion beside a single token, logits at chosen places
    a, b = u.random_tokens(u.CFG_MAIN["vocab"], 30, 1), u.random_tokens(u.CFG_MAIN["vocab"], 4, 2)
    steps = [{"step": 0, "entries": [{"id": "a", "tokens": a[:17], "want": [0, 16]}], "end": []},
             {"step": 1, "entries": [{"id": "a", "tokens": a[17:29], "want": []}, {"id": "b", "tokens": b[:3], "want": [2]}], "end": []},
             {"step": 2, "entries": [{"id": "b", "tokens": b[3:], "want": [0]}, {"id": "a", "tokens": a[29:], "want": [0]}], "end": ["a", "b"]}]
    out_dir = str(tmp_path_factory.mktemp("panarax_replay"))
    run = subprocess.run([sys.executable, os.path.join(ROOT, "bin", "trace_run"), "--model", folder, "--dtype", "float32",
                          "--out", out_dir, "--max-tokens", "128"], input="\n".join(json.dumps(s) for s in steps) + "\n",
                         capture_output=True, text=True, timeout=300)
    assert run.returncode == 0, run.stderr[-2000:]
    assert [line for line in run.stdout.splitlines() if line.startswith("done")] == ["done 0", "done 1", "done 2"]
    w = u.as_float64(weights)
    la, lb = plain.forward(u.CFG_MAIN, w, a), plain.forward(u.CFG_MAIN, w, b)
    V = u.CFG_MAIN["vocab"]
    for step, want_rows in ((0, [la[0], la[16]]), (1, [lb[2]]), (2, [lb[3], la[29]])):
        got = torch.from_numpy(np.fromfile(os.path.join(out_dir, f"{step}.f32"), dtype="<f4").reshape(-1, V))
        assert float(u.row_errors(got, torch.stack(want_rows)).max()) <= u.LIMIT["float32"], step


def test_replay_of_a_model_that_keeps_no_pages(tmp_path_factory):
    """Layers of recurrent mixers alone: the cache manager has no group of pages, requests hold state slots only."""
    import json
    import os
    import subprocess
    import sys

    import numpy as np
    from conftest import ROOT
    cfg = u.config([u.rglru_layer(mlp=u.moe(4, 2, 16, 1.0)), u.lightning_layer(mlp=u.dense(24))], taps=2)
    weights = u.make_weights(cfg, 5)
    folder = u.write_model(str(tmp_path_factory.mktemp("panarax_no_pages")), cfg, weights)
    a, b = u.random_tokens(cfg["vocab"], 70, 1), u.random_tokens(cfg["vocab"], 9, 2)
    steps = [{"step": 0, "entries": [{"id": "a", "tokens": a[:65], "want": [64]}], "end": []},
             {"step": 1, "entries": [{"id": "a", "tokens": a[65:66], "want": [0]}, {"id": "b", "tokens": b[:8], "want": []}], "end": []},
             {"step": 2, "entries": [{"id": "b", "tokens": b[8:], "want": [0]}, {"id": "a", "tokens": a[66:], "want": [3]}], "end": ["a", "b"]},
             {"step": 3, "entries": [{"id": "c", "tokens": b, "want": [8]}], "end": ["c"]}]       # the slot that b left
    out_dir = str(tmp_path_factory.mktemp("panarax_no_pages_out"))
    run = subprocess.run([sys.executable, os.path.join(ROOT, "bin", "trace_run"), "--model", folder, "--dtype", "float32",
                          "--out", out_dir, "--max-tokens", "192", "--max-seqs", "2"], input="\n".join(json.dumps(s) for s in steps) + "\n",
                         capture_output=True, text=True, timeout=300)
    assert run.returncode == 0, run.stderr[-2000:]
    w = u.as_float64(weights)
    la, lb = plain.forward(cfg, w, a), plain.forward(cfg, w, b)
    V = cfg["vocab"]
    for step, want_rows in ((0, [la[64]]), (1, [la[65]]), (2, [lb[8], la[69]]), (3, [lb[8]])):
        got = torch.from_numpy(np.fromfile(os.path.join(out_dir, f"{step}.f32"), dtype="<f4").reshape(-1, V))
        assert float(u.row_errors(got, torch.stack(want_rows)).max()) <= u.LIMIT["float32"], step
