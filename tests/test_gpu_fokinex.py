"""Fokinex on the GPU against the plain model (`plain_fokinex`): every mechanism alone, the new kernels alone, whole
prompts, decoding through cache and state, portions down to two tokens, unequal batches, pages and slots used again,
keys at the edges of the windows and of pages, far keys, a state written far back, long decoding, other sizes, and
generation through the engine's entry points."""
import math

import pytest
import torch

import fokinex_util as u
import plain_fokinex as plain

pytestmark = pytest.mark.gpu

_models = {}


def model_for(tmp_path_factory, name, cfg, seed, dtype, change=None):
    """(weights as the plain model reads them, loaded engine model); made once per (name, dtype)."""
    from ferrox_amd.engine.loading import load_model
    key = (name, dtype)
    if key not in _models:
        weights = u.make_weights(cfg, seed)
        if change:
            change(weights)
        folder = u.write_model(str(tmp_path_factory.mktemp(f"fokinex_{name}")), cfg, weights)
        _models[key] = (weights, load_model(folder, dtype, "cuda:0"))
    return _models[key]


def runner_of(model, block_size=16, num_pages=24, max_seqs=4, **kw):
    from ferrox_amd.engine.runner import ModelRunner
    return ModelRunner(model, block_size=block_size, num_pages=num_pages, max_seqs=max_seqs, **kw)


def run_and_check(cfg, weights, model, requests, schedule, dtype, what, limit=None, **runner_kw):
    runner = runner_of(model, **runner_kw)
    got, _ = u.run_schedule(runner, requests, schedule)
    for key in runner.manager.groups:
        assert runner.manager.n_free_pages(key) == runner_kw.get("num_pages", 24), "pages were lost"
    return u.check_against_plain(cfg, weights, requests, got, dtype, what, limit)


# ---------------------------------------------------------------------------
# each mechanism alone: models of one layer (two where a layer reads another's latents)
# ---------------------------------------------------------------------------
SINGLE = {
    "latent_no_mask": u.config([u.latent_layer(heads=2, dim=16, rot_dim=8, vdim=16, q_rank=16, kv_rank=16, window=0, scale=0.6)], emb_scale=None),
    "latent_window": u.config([u.latent_layer(heads=4, dim=8, rot_dim=4, vdim=24, q_rank=12, kv_rank=40, window=10, scale=0.5)]),
    "latent_stretched": u.config([u.latent_layer(heads=3, dim=16, rot_dim=16, vdim=8, q_rank=24, kv_rank=24, window=30, scale=0.5, base=100.0,
                                                 scaling=(5.0, 30, 6.0, 0.7))]),
    "latent_part_rotated": u.config([u.latent_layer(heads=2, dim=8, rot_dim=12, vdim=8, q_rank=8, kv_rank=16, window=15, rot_dims=6, base=30.0)]),
    "latent_not_rotated": u.config([u.latent_layer(heads=2, dim=8, rot_dim=8, vdim=8, q_rank=8, kv_rank=16, window=15, rot_dims=0)]),
    "latent_no_rotated_part": u.config([u.latent_layer(heads=2, dim=16, rot_dim=0, vdim=8, q_rank=8, kv_rank=16, window=15)]),
    "latent_shared": u.config([u.latent_layer(heads=4, dim=8, rot_dim=8, vdim=16, q_rank=12, kv_rank=24, window=12, mlp=u.dense(24)),
                               u.latent_layer(heads=2, dim=16, rot_dim=8, vdim=8, q_rank=20, kv_rank=24, window=30, kv_from=0)]),
    "latent_wide": u.config([u.latent_layer(heads=3, dim=16, rot_dim=32, vdim=24, q_rank=24, kv_rank=272, window=19, scale=0.4, mlp=u.dense(32)),
                             u.latent_layer(heads=2, dim=8, rot_dim=32, vdim=16, q_rank=16, kv_rank=272, window=40, scale=0.4, kv_from=0)]),
    "latent_one_head": u.config([u.latent_layer(heads=1, dim=32, rot_dim=4, vdim=32, q_rank=16, kv_rank=24, window=5, scale=0.3)]),
    "left_alone": u.config([u.parallel_layer(heads=4, kv_heads=2, dim=16, window=9, scale=0.5, softcap=3.0, left_scale=1.3, right_scale=0.0)]),
    "left_no_cap_no_mask": u.config([u.parallel_layer(heads=3, kv_heads=3, dim=8, window=0, scale=0.8, softcap=None, left_scale=1.0, right_scale=0.0)]),
    "left_one_kv_head": u.config([u.parallel_layer(heads=6, kv_heads=1, dim=8, window=21, scale=0.7, softcap=50.0, left_scale=0.5, right_scale=0.0)]),
    "right_alone": u.config([u.parallel_layer(left_scale=0.0, right_scale=0.9, r_heads=4, r_kv_heads=1, r_dim=8, r_vdim=12, conv=5)]),
    "right_one_tap": u.config([u.parallel_layer(left_scale=0.0, right_scale=1.0, r_heads=2, r_kv_heads=2, r_dim=24, r_vdim=8, conv=1)]),
    "side_by_side": u.config([u.parallel_layer(mlp=u.dense(32))]),
    "no_feed_forward": u.config([u.latent_layer(mlp=None), u.parallel_layer(mlp=None)]),
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


# ---------------------------------------------------------------------------
# the kernels alone
# ---------------------------------------------------------------------------
def attention_reference(q, k, v, scale, window, sinks, gate, softcap, slopes):
    """float64 attention of one sequence from position 0: q [n, H, D], k [n, G, D], v [n, G, V]."""
    n, H, _ = q.shape
    G = k.shape[1]
    see = plain.window_visible(n, window)
    dist = (torch.arange(n)[:, None] - torch.arange(n)[None, :]).double()
    out = torch.zeros(n, H, v.shape[2], dtype=torch.float64)
    for h in range(H):
        s = (q[:, h].double() @ k[:, h // (H // G)].double().T) * scale
        if softcap:
            s = softcap * torch.tanh(s / softcap)
        if slopes is not None:
            s = s - float(slopes[h]) * dist
        s = s.masked_fill(~see, -math.inf)
        if sinks is not None:
            out[:, h] = plain.softmax_with_sink(s, sinks[h].double()) @ v[:, h // (H // G)].double()
        else:
            out[:, h] = torch.softmax(s, -1) @ v[:, h // (H // G)].double()
    if gate is not None:
        out = out * torch.sigmoid(gate.double()).view(n, H, -1)
    return out


@pytest.mark.parametrize("dtype,hd,vd,bs,G", [
    ("float32", 24, 24, 16, 2), ("bfloat16", 64, 64, 64, 2), ("bfloat16", 128, 128, 64, 1), ("bfloat16", 48, 48, 16, 2),
    ("bfloat16", 32, 32, 16, 4), ("bfloat16", 20, 20, 16, 2), ("bfloat16", 144, 128, 64, 1), ("bfloat16", 80, 64, 16, 1),
    ("float32", 40, 32, 16, 1), ("bfloat16", 256, 192, 64, 1), ("bfloat16", 160, 160, 16, 2), ("bfloat16", 256, 256, 16, 1),
    ("bfloat16", 208, 64, 64, 1), ("bfloat16", 288, 256, 16, 1), ("float32", 320, 272, 64, 1)])
def test_attention_kernels_with_capped_scores_and_distance_slopes(dtype, hd, vd, bs, G):
    """The attention kernels alone with a cap on the scores, a penalty per head for distance, a sink and a gate, and
    with value heads narrower than key heads over one shared key head (what latent attention asks of them): a prompt
    of 333 positions written into scattered pages, read as one portion, as a portion deep in the sequence and as
    single queries, under a window and without one."""
    from ferrox_amd import ops
    dt = getattr(torch, dtype)
    gen = torch.Generator().manual_seed(hd + vd)
    n, H = 333, 4
    q = torch.randn(n, H, hd, generator=gen).to(dt)
    k = torch.randn(n, G, hd, generator=gen).to(dt)
    v = torch.randn(n, G, vd, generator=gen).to(dt)
    gate = torch.randn(n, H * vd, generator=gen).to(dt)
    sinks = torch.randn(H, generator=gen) + 1.0
    slopes = torch.tensor([2.0 ** (-8.0 * (h + 1) / H) for h in range(H)])
    n_blocks = -(-n // bs)
    order = torch.randperm(n_blocks + 3, generator=gen)[:n_blocks].to(torch.int32)
    k_pages = torch.full((n_blocks + 3, G, bs, hd), float("nan")).to(dt)
    v_pages = torch.full((n_blocks + 3, G, vd, bs), float("nan")).to(dt)
    for t in range(n):
        k_pages[order[t // bs], :, t % bs] = k[t]
        v_pages[order[t // bs], :, :, t % bs] = v[t]
    dev = dict(device="cuda")
    qd, gd, kp, vp = q.view(n, -1).cuda(), gate.cuda(), k_pages.cuda(), v_pages.cuda()
    positions = torch.arange(n, dtype=torch.int32, **dev)
    tol = 2e-5 if dtype == "float32" else 2e-2
    table = order.view(1, -1).cuda()
    item = lambda x: torch.tensor(x, dtype=torch.int32, **dev)      # noqa: E731
    for window, cap, slope, sink, gated in ((40, 1.5, True, False, True), (0, 0.7, True, True, False), (100, 0.0, True, False, False),
                                            (64, 2.0, False, True, True), (70, 0.0, False, True, False)):
        want = attention_reference(q, k, v, 0.25, window, sinks if sink else None, gate if gated else None, cap,
                                   slopes if slope else None).view(n, -1)
        common = (H, G, hd, bs, window, 0.25)
        extra = dict(v_dim=vd, sinks=sinks.cuda() if sink else None, gate=gd if gated else None, softcap=cap,
                     slopes=slopes.cuda() if slope else None)
        for first in (0, 200):
            starts = list(range(first, n, 64))
            out = torch.zeros(n, H * vd, dtype=dt, **dev)
            ops.attention_tiles(qd, out, kp, vp, table, positions, item([0] * len(starts)), item(starts),
                                item([min(64, n - s) for s in starts]), *common, tile_q=64, **extra)
            err = (out[first:].double().cpu() - want[first:]).abs().max()
            assert float(err) < tol, (window, cap, slope, first, float(err))
        toks = [0, 1, 63, 64, 200, 263, 264, 332]
        for chunk in (None, 64):
            out = torch.zeros(n, H * vd, dtype=dt, **dev)
            ops.attention_decode(qd, out, kp, vp, table, positions, torch.zeros(len(toks), dtype=torch.int32, **dev),
                                 item(toks), *common, max_kv_len=n, chunk=chunk, **extra)
            err = (out[toks].double().cpu() - want[toks]).abs().max()
            assert float(err) < tol, (window, cap, slope, "decode", chunk, float(err))


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_latent_cache_write_and_query_rotation(dtype):
    """The launch that norms a latent, turns the shared key part and writes both pages, and the one that turns the
    queries' rotated parts, against the plain formulas: positions deep in a sequence, scattered pages, fewer rotated
    dimensions than the part has, a magnitude."""
    from ferrox_amd import ops
    dt = getattr(torch, dtype)
    gen = torch.Generator().manual_seed(5)
    T, R, P, rot, bs, H, D = 37, 24, 12, 8, 16, 3, 10
    freqs, mag = plain.scaled_rotation(rot, 50.0, dict(zip(("factor", "original", "fast", "slow"), (3.0, 40, 4.0, 0.5))))
    down = torch.randn(T, 5 + R + P, generator=gen)
    w = (1.0 + 0.2 * torch.randn(R, generator=gen)).to(dt)
    pos = torch.tensor([900 + 3 * t for t in range(T)], dtype=torch.int32)
    n_pages = (900 + 3 * T) // bs + 2
    table = torch.randperm(n_pages, generator=gen).to(torch.int32).view(1, -1)
    kp = torch.zeros(n_pages + 1, 1, bs, R + P, dtype=dt, device="cuda")
    vp = torch.zeros(n_pages + 1, 1, R, bs, dtype=dt, device="cuda")
    inv = ops.rotary_frequencies("cuda", rot, 50.0, tuple(freqs))
    # (the first five columns stand for the queries' latent, which the same launch norms with a weight of its own)
    wq = (1.0 + 0.2 * torch.randn(5, generator=gen)).to(dt)
    down_d = down.cuda()
    assert ops.latent_kv_write(down_d[:, 5:], w.cuda(), 1e-5, pos.cuda(), torch.zeros(T, dtype=torch.int32, device="cuda"),
                               table.cuda(), kp, vp, R, P, rot, bs, inv, mag) is None
    kp_alone, vp_alone = kp.clone(), vp.clone()
    kp.zero_(), vp.zero_()
    cq = ops.latent_kv_write(down_d[:, 5:], w.cuda(), 1e-5, pos.cuda(), torch.zeros(T, dtype=torch.int32, device="cuda"),
                             table.cuda(), kp, vp, R, P, rot, bs, inv, mag, q_latent=(down_d, wq.cuda(), 3e-5))
    assert torch.equal(kp, kp_alone) and torch.equal(vp, vp_alone)
    assert cq.shape == (T, 5) and cq.dtype == dt
    want_q = plain.rms_norm(down[:, :5].double(), wq.double(), 3e-5)
    assert float((cq.double().cpu() - want_q).abs().max()) < (1e-5 if dtype == "float32" else 2e-2)
    c = plain.rms_norm(down[:, 5:5 + R].double(), w.double(), 1e-5)
    kr = plain.rotate_pairs(down[:, 5 + R:].double(), pos.tolist(), freqs, mag)
    tol = 1e-5 if dtype == "float32" else 2e-2
    for t in range(T):
        page, slot = int(table[0, int(pos[t]) // bs]), int(pos[t]) % bs
        row = kp[page, 0, slot].double().cpu()
        assert float((row[:R] - c[t]).abs().max()) < tol and float((row[R:] - kr[t]).abs().max()) < tol, t
        assert torch.equal(vp[page, 0, :, slot], kp[page, 0, slot, :R]), t          # the values are the latent, the same bits
    q = torch.randn(T, H * (D + P), generator=gen).to(dt)
    q_lat = torch.zeros(T, H * (R + P), dtype=dt, device="cuda")
    ops.latent_q_rot(q.cuda(), q_lat, pos.cuda(), H, D, P, rot, R, inv, mag)
    want = plain.rotate_pairs(q.double().view(T, H, D + P)[..., D:], pos.tolist(), freqs, mag)
    got = q_lat.double().cpu().view(T, H, R + P)
    assert float((got[..., R:] - want).abs().max()) < tol and float(got[..., :R].abs().max()) == 0.0


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_small_kernels_of_the_side_by_side_layer(dtype):
    """Norms over a whole projection with keys that are their own values; a norm over the first columns of wider
    rows; one decay per head; the head norm with a silu gate; the embedding's constant."""
    from ferrox_amd import ops
    dt = getattr(torch, dtype)
    gen = torch.Generator().manual_seed(9)
    tol = 1e-5 if dtype == "float32" else 2e-2
    T, H, G, hd, bs = 21, 3, 2, 12, 8
    qk = torch.randn(T, (H + G) * hd + 3, generator=gen)
    wq, wk = (1 + 0.2 * torch.randn(H * hd, generator=gen)).to(dt), (1 + 0.2 * torch.randn(G * hd, generator=gen)).to(dt)
    pos = torch.arange(40, 40 + T, dtype=torch.int32)
    table = torch.randperm(10, generator=gen).to(torch.int32).view(1, -1)
    kp = torch.zeros(11, G, bs, hd, dtype=dt, device="cuda")
    vp = torch.zeros(11, G, hd, bs, dtype=dt, device="cuda")
    q_out = torch.zeros(T, H * hd, dtype=dt, device="cuda")
    ops.span_norm_kv_write(qk.cuda(), q_out, wq.cuda(), wk.cuda(), 1e-5, pos.cuda(), torch.zeros(T, dtype=torch.int32, device="cuda"),
                           table.cuda(), kp, vp, H, G, hd, bs)
    assert float((q_out.double().cpu() - plain.rms_norm(qk[:, :H * hd].double(), wq.double(), 1e-5)).abs().max()) < tol
    k_want = plain.rms_norm(qk[:, H * hd:(H + G) * hd].double(), wk.double(), 1e-5).view(T, G, hd)
    for t in range(T):
        page, slot = int(table[0, int(pos[t]) // bs]), int(pos[t]) % bs
        assert float((kp[page, :, slot].double().cpu() - k_want[t]).abs().max()) < tol
        assert float((vp[page, :, :, slot].double().cpu() - qk[t, H * hd:(H + G) * hd].double().view(G, hd)).abs().max()) < tol
    # a norm over the first 17 of 29 columns
    rows = torch.randn(9, 29, generator=gen)
    w17 = (1 + 0.2 * torch.randn(17, generator=gen)).to(dt)
    got = ops.rmsnorm(rows.cuda(), w17.cuda(), 1e-5, dt, width=17)
    assert float((got.double().cpu() - plain.rms_norm(rows[:, :17].double(), w17.double(), 1e-5)).abs().max()) < tol
    if dtype == "bfloat16":
        return
    # one decay per head, handed to all its key channels
    Hh, Gg, D = 4, 2, 8
    qc, kc = torch.randn(T, Gg * D, generator=gen), torch.randn(T, Gg * D, generator=gen)
    a, b = torch.randn(T, Hh, generator=gen), torch.randn(T, Hh, generator=gen)
    A_log, dt_bias = torch.randn(Hh, generator=gen) - 1.0, torch.randn(Hh, generator=gen)
    qn, kn, decay, beta, kq = ops.delta_prepare(qc.cuda(), kc.cuda(), a.cuda(), b.cuda(), A_log.cuda(), dt_bias.cuda(), Hh, Gg, D, per_head=True)
    want = torch.exp(-torch.exp(A_log.double()) * torch.nn.functional.softplus(a.double() + dt_bias.double()))
    assert float((decay.double().cpu().view(T, Hh, D) - want[:, :, None]).abs().max()) < 1e-6
    assert float((kn.double().cpu() - plain.unit(kc.double().view(T, Gg, D)).view(T, -1)).abs().max()) < 1e-6
    assert float((beta.double().cpu() - torch.sigmoid(b.double())).abs().max()) < 1e-6
    # head norm times silu(gate)
    V = 10
    o, g = torch.randn(T, Hh * V, generator=gen), torch.randn(T, Hh * V, generator=gen)
    wn = 1 + 0.2 * torch.randn(V, generator=gen)
    y = ops.gated_head_norm(o.cuda(), g.cuda(), wn.cuda(), 1e-5, Hh, V, torch.float32, gate_activation="silu")
    o3 = o.double().view(T, Hh, V)
    want = (o3 / torch.sqrt((o3 * o3).mean(-1, keepdim=True) + 1e-5) * wn.double()).view(T, -1) * plain.silu(g.double())
    assert float((y.double().cpu() - want).abs().max()) < 1e-5
    # the embedding's constant
    table_e = torch.randn(30, 16, generator=gen)
    ids = torch.tensor([3, 29, 0], dtype=torch.int32)
    assert torch.allclose(ops.embed(table_e.cuda(), ids.cuda(), scale=7.5).cpu(), table_e[ids.long()] * 7.5)


# ---------------------------------------------------------------------------
# schedules over the main configuration
# ---------------------------------------------------------------------------
LENGTHS = [1, 2, 23, 50, 97]       # a single token, two, around the windows, across pages


def main_requests():
    return {f"r{n}": u.random_tokens(u.CFG_MAIN["vocab"], n, 40 + n) for n in LENGTHS}


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_whole_prompts_and_decoding(tmp_path_factory, dtype):
    weights, model = model_for(tmp_path_factory, "main", u.CFG_MAIN, 3, dtype)
    reqs = main_requests()
    run_and_check(u.CFG_MAIN, weights, model, reqs, [[(r, len(t))] for r, t in reqs.items()], dtype, "whole")
    # most of a prompt in one step, the last 40 tokens (or all but one) one by one: the windows of 9 to 37 positions
    # pass over decoded tokens, across the page borders at 16, 32, ...; the delta rule's state is carried on
    sched = []
    for r, t in reqs.items():
        first = max(1, len(t) - 40)
        sched += [[(r, first)]] + [[(r, 1)]] * (len(t) - first)
    run_and_check(u.CFG_MAIN, weights, model, reqs, sched, dtype, "decode")
    # token by token from the first token on: the first tokens of a sequence, a convolution that looks before the start
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


def test_one_slot_and_few_pages_for_requests_in_a_row(tmp_path_factory):
    """One slot and three pages of 16: every request takes the slot, the state and the pages that the one before
    left.  Windows of 20 and 12 hold a 150-token request in three pages, in portions of at most 8; the pages behind
    the windows go back as they pass, and come again for later positions."""
    cfg = u.config([u.latent_layer(heads=2, dim=8, rot_dim=4, vdim=8, q_rank=8, kv_rank=12, window=11, scale=0.8, mlp=u.dense(16)),
                    u.parallel_layer(heads=2, kv_heads=1, dim=8, window=12, scale=0.8, r_heads=2, r_kv_heads=1, r_dim=8, r_vdim=8, conv=4),
                    u.latent_layer(heads=4, dim=8, rot_dim=4, vdim=8, q_rank=8, kv_rank=12, window=20, scale=0.8, kv_from=0)], width=32)
    weights, model = model_for(tmp_path_factory, "giveback", cfg, 8, "float32")
    reqs = {"z": u.random_tokens(cfg["vocab"], 150, 2), "y": u.random_tokens(cfg["vocab"], 60, 3), "x": u.random_tokens(cfg["vocab"], 5, 4)}
    sched = [[("z", 8)]] * 17 + [[("z", 1)]] * 14 + [[("y", 7)]] * 8 + [[("y", 2)]] * 2 + [[("x", 2)], [("x", 1)], [("x", 2)]]
    run_and_check(cfg, weights, model, reqs, sched, "float32", "give back", num_pages=3, max_seqs=1)


# ---------------------------------------------------------------------------
# where a fault hides behind random weights: peaked attention, a state written far back
# ---------------------------------------------------------------------------
@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_keys_at_the_edges_stand_out(tmp_path_factory, dtype):
    """A large score scale makes the softmax pick single keys, so that a key just inside a window that is missed, or
    one just outside that is seen, moves the logits far beyond rounding.  The plain model itself must tell the cases
    apart.  Prompts end and decoding runs on both sides of the windows' edges as they pass the page borders (16, 32,
    ...), and far from the start."""
    scale, bar = {"float32": (2.5, 0.1), "bfloat16": (1.0, 0.05)}[dtype]
    cfg = u.config([u.latent_layer(heads=4, dim=16, rot_dim=8, vdim=16, q_rank=24, kv_rank=32, window=30, scale=scale / 4, base=100.0, scaling=u.STRETCH, mlp=u.dense(32)),
                    u.parallel_layer(heads=4, kv_heads=2, dim=16, window=21, scale=scale * 4, softcap=40.0, right_scale=0.3),
                    u.latent_layer(heads=2, dim=16, rot_dim=8, vdim=16, q_rank=24, kv_rank=32, window=47, scale=scale / 4, base=100.0, scaling=u.STRETCH, kv_from=0)], width=64)

    def no_sink(w):      # (a sink that takes no weight: the keys alone share the softmax, one of them stands out)
        for i in (0, 2):
            w[f"l{i}.mix.sink"] = w[f"l{i}.mix.sink"] - 8.0

    weights, model = model_for(tmp_path_factory, "peaked" + dtype, cfg, 21, dtype, change=no_sink)
    tokens = u.random_tokens(cfg["vocab"], 150, 5)
    right = plain.forward(cfg, weights, tokens)
    for layer, key, size in ((0, "mask", 29), (0, "mask", 31), (1, "left__mask", 20), (1, "left__mask", 22), (2, "mask", 46), (2, "mask", 48)):
        other = u.changed(cfg, layer, **{key: {"size": size}})
        assert float(u.row_errors(plain.forward(other, weights, tokens), right).max()) > bar, (layer, size)
    reqs = {"p": tokens}
    for first in (1, 2, 20, 21, 22, 29, 30, 31, 46, 47, 48, 63, 64, 65, 120):
        steps = min(14, 150 - first)
        sched = [[("p", first)]] + [[("p", 1)]] * steps
        if 150 - first - steps:
            sched.append([("p", 150 - first - steps)])
        run_and_check(cfg, weights, model, reqs, sched, dtype, f"edge {first}", limit=u.EDGE_LIMIT[dtype])


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_a_far_key_among_hundreds(tmp_path_factory, dtype):
    """A latent layer without a mask under a peaked softmax: queries deep in a 600-token sequence pick keys hundreds
    of positions back (the plain model without the keys beyond 400 positions differs far beyond the limit), across
    ten pages of 64, whole, in portions, and decoded one by one; a second layer reads the same latents under a window."""
    scale, bar = {"float32": (0.7, 0.1), "bfloat16": (0.3, 0.05)}[dtype]
    cfg = u.config([u.latent_layer(heads=4, dim=16, rot_dim=8, vdim=16, q_rank=24, kv_rank=32, window=0, scale=scale, base=10000.0, mlp=u.dense(64)),
                    u.latent_layer(heads=2, dim=16, rot_dim=8, vdim=16, q_rank=24, kv_rank=32, window=70, scale=scale, base=10000.0, kv_from=0)], width=64)

    def no_sink(w):
        for i in range(2):
            w[f"l{i}.mix.sink"] = w[f"l{i}.mix.sink"] - 8.0

    weights, model = model_for(tmp_path_factory, "far" + dtype, cfg, 23, dtype, change=no_sink)
    tokens = u.random_tokens(cfg["vocab"], 600, 6)
    near = u.changed(cfg, 0, mask={"size": 400})
    moved = u.row_errors(plain.forward(near, weights, tokens)[400:], plain.forward(cfg, weights, tokens)[400:])
    assert float(moved.max()) > bar, float(moved.max())
    reqs = {"f": tokens}
    for what, sched in (("whole", [[("f", 600)]]), ("decode", [[("f", 560)]] + [[("f", 1)]] * 40),
                        ("portions", [[("f", 37)]] * 16 + [[("f", 8)]])):
        run_and_check(cfg, weights, model, reqs, sched, dtype, "far " + what, limit=u.EDGE_LIMIT[dtype], block_size=64, num_pages=10)


def test_a_state_written_far_back(tmp_path_factory):
    """A delta rule that barely decays: what the first tokens wrote is read 150 tokens later.  Changing the first
    token must move the last position's logits in the plain model, and the engine must follow it whole, in portions
    and token by token."""
    cfg = u.config([u.parallel_layer(left_scale=0.0, right_scale=1.0, r_heads=2, r_kv_heads=1, r_dim=16, r_vdim=16, conv=3, mlp=u.dense(32))], width=32)

    def slow(w):
        w["l0.mix.right.A_log"] = torch.full_like(w["l0.mix.right.A_log"], -7.0)

    weights, model = model_for(tmp_path_factory, "slow", cfg, 31, "float32", change=slow)
    tokens = u.random_tokens(cfg["vocab"], 150, 8)
    other = [(tokens[0] + 1) % cfg["vocab"]] + tokens[1:]
    moved = u.row_errors(plain.forward(cfg, weights, other)[-1:], plain.forward(cfg, weights, tokens)[-1:])
    assert float(moved.max()) > 1e-3, float(moved.max())
    reqs = {"s": tokens}
    for what, sched in (("whole", [[("s", 150)]]), ("portions", [[("s", 7)]] * 21 + [[("s", 3)]]), ("decode", [[("s", 100)]] + [[("s", 1)]] * 50)):
        run_and_check(cfg, weights, model, reqs, sched, "float32", "far state " + what)


def test_a_sink_that_takes_nearly_all(tmp_path_factory):
    """Sinks far above every score (the heads' outputs nearly vanish) and far below (no sink at all): neither
    overflows, both match the plain model."""
    cfg = SINGLE["latent_window"]
    for name, shift in (("high_sink", 60.0), ("low_sink", -90.0)):
        def change(w, shift=shift):
            w["l0.mix.sink"] = (w["l0.mix.sink"].float() + shift).to(torch.bfloat16)
        weights, model = model_for(tmp_path_factory, name, cfg, 12, "float32", change=change)
        reqs = {"a": u.random_tokens(cfg["vocab"], 40, 4)}
        run_and_check(cfg, weights, model, reqs, [[("a", 25)]] + [[("a", 1)]] * 15, "float32", name)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_long_decoding_on_the_matrix_units(tmp_path_factory, dtype):
    """Sizes that take the bfloat16 kernels' matrix-unit paths (head sizes in multiples of 16, widths in multiples of
    64, pages of 64): a prompt, then 140 tokens one by one from recorded steps, the windows passing page borders, and
    two requests decoding side by side."""
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
    """Head sizes, ranks, widths and a vocabulary that are no multiples of 16, 8 or 4: the kernels' guarded paths."""
    cfg = u.config([u.latent_layer(heads=3, dim=10, rot_dim=6, vdim=14, q_rank=18, kv_rank=22, window=7, scale=0.6, rot_dims=6, base=20.0, mlp=u.dense(30)),
                    u.parallel_layer(heads=3, kv_heads=3, dim=18, window=19, scale=0.5, softcap=7.0, r_heads=6, r_kv_heads=2, r_dim=10, r_vdim=10, conv=5, mlp=u.dense(22)),
                    u.latent_layer(heads=5, dim=6, rot_dim=6, vdim=6, q_rank=13, kv_rank=22, window=0, scale=0.5, rot_dims=6, base=20.0, kv_from=0)], width=70, vocab=151)
    weights, model = model_for(tmp_path_factory, "odd", cfg, 13, dtype)
    reqs = {"a": u.random_tokens(151, 45, 1), "b": u.random_tokens(151, 20, 2)}
    sched = [[("a", 30), ("b", 2)], [("a", 1), ("b", 17)]] + [[("a", 1), ("b", 1)]] + [[("a", 1)]] * 13
    run_and_check(cfg, weights, model, reqs, sched, dtype, "odd sizes")


# ---------------------------------------------------------------------------
# through the engine's own entry points: scheduler, sampling, recorded steps, command line, replay
# ---------------------------------------------------------------------------
def plain_greedy(cfg, weights, prompt, n):
    tokens = list(prompt)
    for _ in range(n):
        tokens.append(int(plain.forward(cfg, weights, tokens)[-1].argmax()))
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
    folder = u.write_model(str(tmp_path_factory.mktemp("fokinex_cli")), u.CFG_MAIN, weights)
    prompt = u.random_tokens(u.CFG_MAIN["vocab"], 9, 77)
    want = plain_greedy(u.CFG_MAIN, weights, prompt, 6)
    out = subprocess.run([sys.executable, os.path.join(ROOT, "bin", "ferrox-amd"), "-m", folder, "--tokens",
                          ",".join(map(str, prompt)), "-n", "6", "--temp", "0", "--repeat-penalty", "1.0", "--ignore-eos", "--dtype", "float32",
                          "--block-size", "16", "--num-pages", "16"],
                         capture_output=True, text=True, timeout=300)
    assert out.returncode == 0, out.stderr[-2000:]
    assert ",".join(map(str, want)) in out.stdout.replace(" ", ""), (out.stdout[-500:], want)
    # the step-by-step replay: two requests, a portion beside a single token, logits at chosen places
    a, b = u.random_tokens(u.CFG_MAIN["vocab"], 30, 1), u.random_tokens(u.CFG_MAIN["vocab"], 4, 2)
    steps = [{"step": 0, "entries": [{"id": "a", "tokens": a[:17], "want": [0, 16]}], "end": []},
             {"step": 1, "entries": [{"id": "a", "tokens": a[17:29], "want": []}, {"id": "b", "tokens": b[:3], "want": [2]}], "end": []},
             {"step": 2, "entries": [{"id": "b", "tokens": b[3:], "want": [0]}, {"id": "a", "tokens": a[29:], "want": [0]}], "end": ["a", "b"]}]
    out_dir = str(tmp_path_factory.mktemp("fokinex_replay"))
    run = subprocess.run([sys.executable, os.path.join(ROOT, "bin", "trace_run"), "--model", folder, "--dtype", "float32",
                          "--out", out_dir, "--max-tokens", "128"], input="\n".join(json.dumps(s) for s in steps) + "\n",
                         capture_output=True, text=True, timeout=300)
    assert run.returncode == 0, run.stderr[-2000:]
    assert [line for line in run.stdout.splitlines() if line.startswith("done")] == ["done 0", "done 1", "done 2"]
    la, lb = plain.forward(u.CFG_MAIN, weights, a), plain.forward(u.CFG_MAIN, weights, b)
    V = u.CFG_MAIN["vocab"]
    for step, want_rows in ((0, [la[0], la[16]]), (1, [lb[2]]), (2, [lb[3], la[29]])):
        got = torch.from_numpy(np.fromfile(os.path.join(out_dir, f"{step}.f32"), dtype="<f4").reshape(-1, V))
        assert float(u.row_errors(got, torch.stack(want_rows)).max()) <= u.LIMIT["float32"], step
