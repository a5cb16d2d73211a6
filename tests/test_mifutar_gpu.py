"""The Mifutar design on the GPU: every new kernel alone against its plain PyTorch version (tests/emu_ops.py), and
the model through the engine's own step function, cache and state manager, graphs and scheduler against the plain
implementation (tests/plain_mifutar.py), in float32 and bfloat16."""
import json

import pytest
import torch

import helpers
import mifutar_cases as cases
import plain_mifutar as plain
from emu_ops import EmuOps

pytestmark = pytest.mark.gpu
DEV = "cuda:0"
TOL = {"float32": 1e-4, "bfloat16": 3e-2}       # plain.logit_error of a whole model
emu = EmuOps()


def _ops():
    from tempura_amd.kernels import ops
    return ops


@pytest.fixture(scope="module")
def dirs(tmp_path_factory):
    root = tmp_path_factory.mktemp("mifutar_gpu")
    return {name: cases.write_model(name, str(root / name)) for name in cases.CASES}


def _close(got, want, tol):
    got, want = got.double().cpu(), want.double().cpu()
    assert got.shape == want.shape
    err = float((got - want).abs().max() / max(1e-30, float(want.abs().max())))
    assert err <= tol, f"relative error {err:.3e} > {tol:.1e}"


# ---- kernels alone ------------------------------------------------------------------------------
@pytest.mark.parametrize("hidden,streams", [(64, 1), (37, 3), (256, 4), (1030, 2)])
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_embed_with_positions_and_streams(hidden, streams, dtype):
    ops = _ops()
    g = torch.Generator().manual_seed(1)
    table = torch.randn(90, hidden, generator=g).to(dtype)
    tok = torch.randint(0, 90, (33,), generator=g, dtype=torch.int32)
    pos = torch.tensor([0, 1, 2, 3, 17, 500, 4095, 100000, 1 << 19] + list(range(24)), dtype=torch.int32)
    inv = torch.pow(torch.tensor(10000.0, dtype=torch.float64), -2.0 * torch.arange((hidden + 1) // 2, dtype=torch.float64) / hidden)
    got = ops.embed(tok.to(DEV), table.to(DEV), pos.to(DEV), inv.to(DEV), streams)
    want = emu.embed(tok, table, pos, inv, streams)
    assert got.shape == (33, streams * hidden)
    assert float((got.cpu().double() - want.double()).abs().max()) < 2e-6


@pytest.mark.parametrize("S,W", [(1, 48), (3, 64), (4, 256), (5, 33), (16, 40), (2, 5000)])
@pytest.mark.parametrize("out_dtype", [torch.float32, torch.bfloat16])
def test_stream_step(S, W, out_dtype):
    ops = _ops()
    g = torch.Generator().manual_seed(S * 1000 + W)
    n = 9
    h = torch.randn(n, S * W, generator=g)
    y = torch.randn(n, W, generator=g)
    mix, oc, ic = torch.randn(S, S, generator=g), torch.randn(S, generator=g), torch.randn(S, generator=g)
    nw = torch.randn(W, generator=g)
    tol = 2e-6 if out_dtype == torch.float32 else 1e-2
    # close a sublayer and open the next
    h_ref = h.clone()
    want = emu.stream_step(h_ref, S, y, mix, oc, ic, nw, 1e-5, out_dtype)
    h_dev = h.to(DEV)
    got = ops.stream_step(h_dev, S, y.to(DEV), mix.to(DEV), oc.to(DEV), ic.to(DEV), nw.to(DEV), 1e-5, out_dtype)
    _close(h_dev, h_ref, 2e-6)
    _close(got, want, tol)
    # update only; identity wiring (the plain residual sum) when no coefficients are given
    h_ref2, h_dev2 = h.clone(), h.to(DEV)
    emu.stream_step(h_ref2, S, y)
    assert ops.stream_step(h_dev2, S, y.to(DEV)) is None
    _close(h_dev2, h_ref2, 2e-6)
    # the sum of the copies at chosen rows, normed, nothing written
    rows = torch.tensor([7, 0, 3], dtype=torch.int32)
    before = h_dev2.clone()
    got = ops.stream_step(h_dev2, S, norm_weight=nw.to(DEV), eps=1e-6, out_dtype=out_dtype, rows=rows.to(DEV), write_back=False)
    _close(got, emu.stream_step(h_ref2, S, norm_weight=nw, eps=1e-6, out_dtype=out_dtype, rows=rows, write_back=False), tol)
    assert torch.equal(before, h_dev2)
    assert ops.stream_step(h_dev2, S, out_dtype=out_dtype, rows=rows[:0].to(DEV), write_back=False).shape == (0, W)


@pytest.mark.parametrize("out_dtype", [torch.float32, torch.bfloat16])
def test_gated_act_with_limits(out_dtype):
    ops = _ops()
    gu = torch.randn(7, 2 * 45, generator=torch.Generator().manual_seed(2)) * 3
    gu16 = torch.randn(7, 2 * 48, generator=torch.Generator().manual_seed(5)) * 3
    for slope, limit, off in [(1.702, 1.25, 1.0), (1.0, 0.0, 0.0), (0.5, 0.25, -2.0)]:
        got = ops.gated_act(gu.to(DEV), out_dtype, slope, limit, off)
        _close(got, emu.gated_act(gu, out_dtype, slope, limit, off), 2e-6 if out_dtype == torch.float32 else 1e-2)
        got = ops.gated_act(gu16.to(DEV), out_dtype, slope, limit, off, interleaved=True)       # eight gate, eight up columns in turn
        _close(got, emu.gated_act(gu16, out_dtype, slope, limit, off, interleaved=True), 2e-6 if out_dtype == torch.float32 else 1e-2)
    logits = torch.randn(3, 11)
    _close(ops.scale_(logits.to(DEV), 0.375), logits * 0.375, 0)


def _paged(n_ctx, kvh, d, ps, dtype, g):
    """A cache of one request whose pages are scattered, and the keys it holds."""
    pages = (n_ctx + ps - 1) // ps
    order = torch.randperm(pages + 3, generator=g)[:pages].to(torch.int32)
    k_cache = torch.zeros(pages + 4, kvh, ps, d, dtype=dtype)
    v_cache = torch.zeros(pages + 4, kvh, d, ps, dtype=dtype)
    return order, k_cache, v_cache


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("heads,kvh,d,ps", [(4, 2, 16, 16), (3, 3, 10, 8), (6, 2, 96, 16), (2, 1, 64, 32)])
def test_biased_keys_as_values_into_the_cache(dtype, heads, kvh, d, ps):
    ops = _ops()
    g = torch.Generator().manual_seed(heads * 100 + d)
    n = 21
    rows = torch.randn(n, (heads + kvh) * d, generator=g)
    qb, kb = torch.randn(heads * d, generator=g), torch.randn(kvh * d, generator=g)
    order, kc, vc = _paged(40, kvh, d, ps, dtype, g)
    slots = torch.tensor([int(order[(5 + t) // ps]) * ps + (5 + t) % ps for t in range(n)], dtype=torch.int32)
    kd, vd = kc.to(DEV), vc.to(DEV)
    q = ops.qk_store(rows.to(DEV), qb.to(DEV), kb.to(DEV), slots.to(DEV), heads, kvh, d, kd, vd, dtype)
    qr = emu.qk_store(rows, qb, kb, slots, heads, kvh, d, kc, vc, dtype)
    tol = 0 if dtype == torch.float32 else 1e-2
    _close(q, qr, tol)
    _close(kd, kc, tol)
    _close(vd, vc, tol)
    assert torch.equal(kd.cpu()[slots.long() // ps, :, slots.long() % ps], vd.cpu()[slots.long() // ps, :, :, slots.long() % ps])
    # queries alone (a call that reads another call's cache)
    q2 = ops.qk_store(rows[:, : heads * d].contiguous().to(DEV), qb.to(DEV), None, None, heads, kvh, d, None, None, dtype)
    _close(q2, qr, tol)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("heads,kvh,d,ps,window,L", [(4, 2, 16, 16, 7, 7), (3, 3, 10, 8, 20, 12), (6, 2, 96, 16, 100, 90),
                                                   (2, 1, 64, 16, 0, 30), (4, 4, 32, 16, 33, 33), (8, 2, 128, 16, 100, 64),
                                                   (2, 1, 64, 16, 0, 1500), (5, 1, 128, 32, 120, 121)])
def test_attention_with_distance_bias_and_a_key_that_stands_out(dtype, heads, kvh, d, ps, window, L):
    """Portions behind a cached prefix and single tokens in one batch.  One key is made to dominate the scores of
    the queries that may see it: at the window's last place for one request, one place outside it for another, and
    at the very first position (far away) without a window."""
    ops = _ops()
    g = torch.Generator().manual_seed(d + window)
    ctxs, qlens = [150, 64, 97, 1], [37, 1, 1, 1]
    n = sum(qlens)
    r = len(ctxs)
    width = max((c + ps - 1) // ps for c in ctxs)
    total_pages = sum((c + ps - 1) // ps for c in ctxs)
    perm = torch.randperm(total_pages + 2, generator=g).to(torch.int32)
    kc = torch.zeros(total_pages + 3, kvh, ps, d, dtype=dtype)
    vc = torch.zeros(total_pages + 3, kvh, d, ps, dtype=dtype)
    tables = torch.full((r, width), -1, dtype=torch.int32)
    q = (torch.randn(n, heads, d, generator=g) * 0.5).to(dtype)
    used = 0
    cu = [0]
    for i, (c, ql) in enumerate(zip(ctxs, qlens)):
        npg = (c + ps - 1) // ps
        tables[i, :npg] = perm[used: used + npg]
        used += npg
        keys = torch.randn(c, kvh, d, generator=g) * 0.5
        # the stand-out key: as seen from the request's last query
        last = c - 1
        if window > 0 and last - (window - 1) >= 0:
            place = last - (window - 1) if i % 2 == 0 else last - window       # just inside / just outside
        else:
            place = 0
        if place >= 0:
            # (every head of the last query looks the same way; the key lies four times as far that way)
            way = torch.randn(d, generator=g)
            way = way / way.norm() * d ** 0.5
            q[cu[-1] + ql - 1] = way.to(dtype)
            keys[place] = 4.0 * way
        for j in range(c):
            pg = int(tables[i, j // ps])
            kc[pg, :, j % ps] = keys[j].to(dtype)
            vc[pg, :, :, j % ps] = keys[j].to(dtype)
        cu.append(cu[-1] + ql)
    bias = torch.randn(heads, L, generator=g)
    cu_t, ctx_t = torch.tensor(cu, dtype=torch.int32), torch.tensor(ctxs, dtype=torch.int32)
    token_req = torch.tensor([i for i, ql in enumerate(qlens) for _ in range(ql)], dtype=torch.int32)
    scale = d ** -0.5
    want = emu.paged_attention(q, kc, vc, tables, cu_t, ctx_t, token_req, scale, window, max(qlens), max(ctxs), dist_bias=bias)
    for singles in (0, 3):        # every request as a portion; the single tokens through the kernel for decoding
        got = ops.paged_attention(q.to(DEV), kc.to(DEV), vc.to(DEV), tables.to(DEV), cu_t.to(DEV), ctx_t.to(DEV), token_req.to(DEV),
                                  scale, window, max(qlens), max(ctxs), num_single=singles, dist_bias=bias.to(DEV))
        _close(got, want, 2e-5 if dtype == torch.float32 else 2e-2)
    # and the stand-out key does decide where it is seen (the first request; the second has it one place outside)
    assert float((want.double()[cu[1] - 1]).abs().max()) > 2.0
    if window > 0 and ctxs[1] - 1 - window >= 0:
        assert float((want.double()[cu[2] - 1]).abs().max()) < 2.0


@pytest.mark.parametrize("channels,taps", [(40, 4), (7, 1), (130, 2), (300, 5)])
def test_causal_conv_carries_its_inputs(channels, taps):
    ops = _ops()
    g = torch.Generator().manual_seed(channels)
    col0, width = 11, 11 + channels + 6
    w, b = torch.randn(taps, channels, generator=g), torch.randn(channels, generator=g)
    row = (taps - 1) * channels + 13
    state = torch.randn(5, row, generator=g)
    runs = [3, 1, 2, 9]                                     # shorter than, equal to and longer than taps - 1
    slots = torch.tensor([4, 0, 2, 1], dtype=torch.int32)
    cu = torch.tensor([0, 3, 4, 6, 15], dtype=torch.int32)
    token_req = torch.tensor([i for i, l in enumerate(runs) for _ in range(l)], dtype=torch.int32)
    proj = torch.randn(15, width, generator=g)
    s_ref, s_dev = state.clone(), state.to(DEV)
    for _ in range(3):                                      # three steps in a row: what one leaves the next reads
        want = emu.causal_conv(proj, col0, channels, w, b, s_ref, cu, token_req, slots, 4)
        got = ops.causal_conv(proj.to(DEV), col0, channels, w.to(DEV), b.to(DEV), s_dev, cu.to(DEV), token_req.to(DEV), slots.to(DEV), 4)
        _close(got, want, 2e-6)
        _close(s_dev, s_ref, 0)
        proj = proj * 0.9 + 0.1
    assert torch.equal(s_dev.cpu()[3], state[3])            # a slot of no request is left alone


@pytest.mark.parametrize("H,P,N,G", [(4, 8, 16, 2), (2, 24, 5, 1), (6, 40, 56, 2), (3, 64, 128, 3), (1, 40, 600, 1), (8, 16, 32, 1)])
def test_selective_scan_and_its_state(H, P, N, G):
    ops = _ops()
    g = torch.Generator().manual_seed(H * 10 + N)
    inner, ch = H * P, H * P + 2 * G * N
    runs = [70, 1, 5, 2]
    n = sum(runs)
    cu = torch.tensor([0, 70, 71, 76, 78], dtype=torch.int32)
    slots = torch.tensor([2, 5, 0, 3], dtype=torch.int32)
    off = 17
    state = torch.randn(7, off + H * N * P, generator=g) * 0.5
    xbc = torch.randn(n, ch, generator=g) * 0.7
    proj = torch.randn(n, 9 + H + 3, generator=g)
    dt_bias, a_log, d_skip = torch.randn(H, generator=g) - 0.5, torch.log(torch.rand(H, generator=g) * 2 + 0.05), torch.randn(H, generator=g)
    s_ref, s_dev = state.clone(), state.to(DEV)
    want = emu.ssm_scan(xbc, proj, 9, dt_bias, a_log, d_skip, s_ref, off, cu, slots, 4, H, P, N, G)
    got = ops.ssm_scan(xbc.to(DEV), proj.to(DEV), 9, dt_bias.to(DEV), a_log.to(DEV), d_skip.to(DEV), s_dev, off, cu.to(DEV),
                       slots.to(DEV), 4, H, P, N, G)
    _close(got, want, 2e-5)
    _close(s_dev, s_ref, 2e-5)
    assert torch.equal(s_dev.cpu()[:, :off], state[:, :off]) and torch.equal(s_dev.cpu()[1], state[1])
    # a run cut in two gives the same bits as the run whole
    s_two = state.to(DEV)
    cut = 33
    cu_a = torch.tensor([0, cut], dtype=torch.int32).to(DEV)
    cu_b = torch.tensor([0, 70 - cut], dtype=torch.int32).to(DEV)
    one = slots[:1].to(DEV)
    ya = ops.ssm_scan(xbc[:cut].to(DEV), proj[:cut].to(DEV), 9, dt_bias.to(DEV), a_log.to(DEV), d_skip.to(DEV), s_two, off, cu_a, one, 1, H, P, N, G)
    yb = ops.ssm_scan(xbc[cut:70].contiguous().to(DEV), proj[cut:70].contiguous().to(DEV), 9, dt_bias.to(DEV), a_log.to(DEV), d_skip.to(DEV),
                      s_two, off, cu_b, one, 1, H, P, N, G)
    assert torch.equal(torch.cat([ya, yb]), got[:70]) and torch.equal(s_two[2], s_dev[2])


@pytest.mark.parametrize("H,P,N,G", [(4, 8, 16, 2), (3, 40, 24, 1), (8, 64, 128, 4)])
def test_long_runs_in_pieces_side_by_side(H, P, N, G):
    """Runs long enough to be cut into pieces that run side by side, beside short ones and a single token, from states
    that are not zero: the same result as token by token, up to rounding."""
    ops = _ops()
    g = torch.Generator().manual_seed(H + N)
    inner, ch = H * P, H * P + 2 * G * N
    runs = [700, 1, 300, 2, 129]
    n = sum(runs)
    cu = torch.tensor([0, 700, 701, 1001, 1003, 1132], dtype=torch.int32)
    slots = torch.tensor([1, 4, 0, 3, 2], dtype=torch.int32)
    state = torch.randn(6, 5 + H * N * P, generator=g) * 0.5
    xbc = torch.randn(n, ch, generator=g) * 0.7
    proj = torch.randn(n, H + 2, generator=g)
    dt_bias, a_log, d_skip = torch.randn(H, generator=g) - 1.5, torch.log(torch.rand(H, generator=g) * 0.5 + 0.05), torch.randn(H, generator=g)
    s_ref, s_dev = state.clone(), state.to(DEV)
    want = emu.ssm_scan(xbc, proj, 1, dt_bias, a_log, d_skip, s_ref, 5, cu, slots, 5, H, P, N, G)
    got = ops.ssm_scan(xbc.to(DEV), proj.to(DEV), 1, dt_bias.to(DEV), a_log.to(DEV), d_skip.to(DEV), s_dev, 5, cu.to(DEV),
                       slots.to(DEV), 5, H, P, N, G, max_run=700)
    _close(got, want, 2e-5)
    _close(s_dev, s_ref, 2e-5)
    assert torch.equal(s_dev.cpu()[5], state[5]) and torch.equal(s_dev.cpu()[:, :5], state[:, :5])


@pytest.mark.parametrize("inner,groups", [(32, 1), (48, 3), (320, 2), (4096, 4)])
@pytest.mark.parametrize("out_dtype", [torch.float32, torch.bfloat16])
def test_gated_group_norm(inner, groups, out_dtype):
    ops = _ops()
    g = torch.Generator().manual_seed(inner)
    y, proj, w = torch.randn(6, inner, generator=g), torch.randn(6, 5 + inner + 2, generator=g), torch.randn(inner, generator=g)
    got = ops.gated_group_norm(y.to(DEV), proj.to(DEV), 5, w.to(DEV), 1e-5, groups, out_dtype)
    _close(got, emu.gated_group_norm(y, proj, 5, w, 1e-5, groups, out_dtype), 2e-6 if out_dtype == torch.float32 else 1e-2)


# ---- the model through the step function --------------------------------------------------------
def _runner(dirs, name, dtype, max_tokens, page_size=16, max_requests=4, use_graph=False):
    from tempura_amd.engine.loading import load_model
    from tempura_amd.engine.runner import ModelRunner
    model = load_model(dirs[name], dtype, DEV)
    return ModelRunner(model, page_size, (max_tokens + page_size - 1) // page_size, max_requests=max_requests, use_graph=use_graph)


_REFS = {}


def _ref(name, rid):
    if (name, rid) not in _REFS:
        _REFS[(name, rid)] = plain.forward(cases.config_json(name), cases.make_weights(name), cases.requests(name)[rid])
    return _REFS[(name, rid)]


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", ["mix", "ssm", "attn", "wide"])
@pytest.mark.parametrize("mode", ["whole", "bulk_tail", "portions", "mixed"])
def test_every_cutting_matches_plain(dirs, name, mode, dtype):
    reqs = cases.requests(name)
    lengths = cases.LENGTHS[name]
    if mode == "mixed":
        max_tokens = sum(sorted(helpers.roundup(n, 64) for n in lengths.values())[-2:]) + 64
        steps = helpers.schedule_mixed(lengths, max_tokens, seed=11)
    else:
        max_tokens = max(helpers.roundup(n, 64) for n in lengths.values())
        steps = {"whole": helpers.schedule_whole, "bulk_tail": lambda l: helpers.schedule_bulk_tail(l, tail=40),
                 "portions": lambda l: helpers.schedule_portions(l, sizes=(7, 2, 16, 3, 2, 31, 5, 2, 64, 9, 2, 17))}[mode](lengths)
    runner = _runner(dirs, name, dtype, max_tokens)
    got = helpers.run_schedule(runner, reqs, steps)
    for rid in reqs:
        err = plain.logit_error(got[rid], _ref(name, rid))
        assert err < TOL[dtype], f"{name}/{mode}/{dtype}: request {rid}: error {err:.3e}"
    assert not runner.cache.live_requests()
    assert runner.cache.free_pages() == [p.num_pages for p in runner.cache.pools]


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_cutting_changes_rounding_only(dirs, dtype):
    """The same request whole, in portions and beside others: differences far below the distance to the plain result."""
    reqs = cases.requests("wide")
    lengths = cases.LENGTHS["wide"]
    runs = []
    for steps in (helpers.schedule_whole(lengths), helpers.schedule_portions(lengths, sizes=(2, 9, 33, 2, 16, 5)),
                  helpers.schedule_mixed(lengths, 448, seed=3)):
        runs.append(helpers.run_schedule(_runner(dirs, "wide", dtype, 448), reqs, steps))
    for rid in reqs:
        for other in runs[1:]:
            assert plain.logit_error(other[rid], runs[0][rid]) < (2e-5 if dtype == "float32" else 2e-2), rid


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_window_edge_decides_on_the_gpu(dirs, tmp_path, dtype):
    from tempura_amd.engine.loading import load_model
    from tempura_amd.engine.runner import ModelRunner, StepEntry
    cfg = cases.config_json("wide")
    W = cases.make_weights("wide")
    for li in (0, 2):
        m = cases.CASES["wide"]["layers"][li]["mixer"]
        edge = plain.distance_bucket(m["mask"]["size"] - 1, m["_rows"], m["bias_max"])
        W[f"l{li}.mix.rel"] = W[f"l{li}.mix.rel"].clone()
        W[f"l{li}.mix.rel"][edge] += 14.0
    folder = cases.write_model("wide", str(tmp_path / "edge"), weights=W)
    toks = cases.tokens("wide", 110, 3)
    ref = plain.forward(cfg, W, toks)
    # (a bias of 14 on one key also magnifies what rounding q and k to bfloat16 does to that score)
    tol = {"float32": 1e-4, "bfloat16": 5e-2}[dtype]
    for delta in (-1, 1):
        off = json.loads(json.dumps(cfg))
        for li in (0, 2):
            off["layers"][li]["mixer"]["mask"]["size"] += delta
        assert plain.logit_error(plain.forward(off, W, toks)[60:], ref[60:]) > 4 * tol
    runner = ModelRunner(load_model(folder, dtype, DEV), 16, 16, max_requests=2)
    runner.add_request("r")
    a = runner.step([StepEntry("r", toks[:60], list(range(60)))])
    rows = [a.clone()] + [runner.step([StepEntry("r", [t], [0])]).clone() for t in toks[60:]]
    assert plain.logit_error(torch.cat(rows).cpu(), ref) < tol


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_long_prompt_whole_and_in_portions(dirs, dtype):
    """A prompt long enough that the recurrence runs in pieces side by side, whole and in portions that are cut
    inside pieces, pages and windows, then decoded on; far keys and the state of hundreds of tokens decide here."""
    from tempura_amd.engine.runner import StepEntry
    toks = cases.tokens("wide", 560, 77)
    ref = plain.forward(cases.config_json("wide"), cases.make_weights("wide"), toks)
    want_rows = [0, 1, 255, 256, 257, 300, 511, 512, 540, 559]
    for cuts in ([560], [300, 2, 129, 97, 31, 1]):
        runner = _runner(dirs, "wide", dtype, 640)
        runner.add_request("r")
        rows, at = [], 0
        for c in cuts:
            w = [i - at for i in want_rows if at <= i < at + c]
            lg = runner.step([StepEntry("r", toks[at: at + c], w)])
            if w:
                rows.append(lg.cpu().clone())
            at += c
        assert plain.logit_error(torch.cat(rows), ref[want_rows]) < TOL[dtype], cuts


def test_long_decoding_through_a_captured_step(dirs):
    """Two requests decoded token by token for 150 steps through the graph path, state and windows carried along."""
    from tempura_amd.engine.runner import StepEntry
    cfg, W = cases.config_json("wide"), cases.make_weights("wide")
    runner = _runner(dirs, "wide", "float32", 512, use_graph=True)
    assert runner.use_graph, "every part of the design may be captured"
    seqs = {"p": cases.tokens("wide", 170, 41), "q": cases.tokens("wide", 158, 42)}
    start = {"p": 20, "q": 8}
    got = {rid: [] for rid in seqs}
    for rid in seqs:
        runner.add_request(rid)
        got[rid].append(runner.step([StepEntry(rid, seqs[rid][: start[rid]], list(range(start[rid])))]).cpu())
    for i in range(150):
        logits = runner.step([StepEntry(rid, [seqs[rid][start[rid] + i]], [0]) for rid in seqs]).cpu()
        for k, rid in enumerate(seqs):
            got[rid].append(logits[k: k + 1].clone())
    assert runner.graph_steps >= 149
    for rid in seqs:
        assert plain.logit_error(torch.cat(got[rid]), plain.forward(cfg, W, seqs[rid])) < TOL["float32"], rid


@pytest.mark.parametrize("name", ["mix", "wide"])
@pytest.mark.parametrize("use_graph", [False, True])
def test_engine_generates_what_plain_greedy_generates(dirs, name, use_graph):
    from tempura_amd.engine import Engine
    from tempura_amd.sampling import SamplingParams
    cfg, W = cases.config_json(name), cases.make_weights(name)
    prompts = [cases.tokens(name, n, 20 + i) for i, n in enumerate((3, 18, 9, 40, 1))]
    eng = Engine(dirs[name], dtype="float32", page_size=16, kv_pages=24, max_batch_size=3, max_num_batched_tokens=32,
                 prefill_chunk_size=7, device=DEV, use_graph=use_graph)
    outs = eng.generate(prompts, SamplingParams(temperature=0.0, max_new_tokens=12))
    for p, o in zip(prompts, outs):
        assert o == plain.greedy(cfg, W, p, 12)
    if use_graph:
        assert eng.runner.graph_steps > 0


def test_replay_program_on_a_model_folder(dirs, tmp_path):
    """bin/trace_run on a small folder: steps on standard input, logits files out, against the plain result."""
    import os
    import subprocess
    import numpy as np
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    toks = cases.tokens("mix", 30, 5)
    out = tmp_path / "out"
    steps = [{"step": 0, "entries": [{"id": "a", "tokens": toks[:11], "want": [0, 10]}], "end": []},
             {"step": 1, "entries": [{"id": "a", "tokens": toks[11:13], "want": []}], "end": []},
             {"step": 2, "entries": [{"id": "a", "tokens": toks[13:], "want": [16]}, {"id": "b", "tokens": toks[:4], "want": [3]}], "end": ["a", "b"]}]
    p = subprocess.run([os.path.join(root, "bin", "trace_run"), "--model", dirs["mix"], "--dtype", "float32", "--out", str(out),
                        "--max-tokens", "128"], input="".join(json.dumps(s) + "\n" for s in steps), capture_output=True, text=True, timeout=600)
    assert p.returncode == 0, p.stderr[-2000:]
    assert [l for l in p.stdout.splitlines() if l.startswith("done")] == ["done 0", "done 1", "done 2"]
    ref = plain.forward(cases.config_json("mix"), cases.make_weights("mix"), toks)
    vocab = ref.shape[1]
    a = torch.from_numpy(np.fromfile(out / "0.f32", dtype="<f4").reshape(-1, vocab))
    c = torch.from_numpy(np.fromfile(out / "2.f32", dtype="<f4").reshape(-1, vocab))
    assert not (out / "1.f32").exists()
    assert plain.logit_error(torch.cat([a, c]), torch.stack([ref[0], ref[10], ref[29], ref[3]])) < TOL["float32"]


@pytest.mark.parametrize("m", [17, 40, 64, 100, 300, 2048])
def test_gated_product_with_limits_in_the_epilogue(m):
    """The gate/up product that applies the limited activation to its float32 sums, at every number of rows that
    takes another product kernel, against the product and the activation as two steps."""
    ops = _ops()
    g = torch.Generator().manual_seed(m)
    k, inter = 256, 384
    x = (torch.randn(m, k, generator=g) * 1.5).to(torch.bfloat16)
    gate, up = (torch.randn(inter, k, generator=g) * 0.1).to(torch.bfloat16), (torch.randn(inter, k, generator=g) * 0.1).to(torch.bfloat16)
    w = ops.tile_weight(ops.interleave_gate_up(gate.to(DEV), up.to(DEV)))
    for slope, limit, off in [(1.702, 1.25, 1.0), (1.0, 0.0, 0.0), (0.7, 0.4, -0.5)]:
        got = ops.linear_swiglu(x.to(DEV), w, slope=slope, limit=limit, up_offset=off)
        gu = torch.cat([x.double() @ gate.double().T, x.double() @ up.double().T], dim=1)
        want = emu.gated_act(gu, torch.float64, slope, limit, off)
        assert float(want.abs().max()) > 0.3
        _close(got, want, 1e-2)
