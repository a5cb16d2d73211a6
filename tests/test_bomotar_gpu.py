"""The Bomotar design on the GPU: every new kernel alone against its plain PyTorch version (tests/emu_ops.py), and
the model through the engine's own step function, cache and state manager, graphs and scheduler against the plain
implementation (tests/plain_bomotar.py), in float32 and bfloat16."""
import json

import pytest
import torch

import bomotar_cases as cases
import helpers
import plain_bomotar as plain
from emu_ops import EmuOps

pytestmark = pytest.mark.gpu
DEV = "cuda:0"
# plain.logit_error of a whole model: the largest difference of any logit, in units of the logits' spread.  bfloat16
# rounding alone reaches 0.1 in these small models; a lost key, a wrong state or another choice of experts costs
# 0.3 and more (the tests that plant something check that their own premise does)
TOL = {"float32": 1e-4, "bfloat16": 1.5e-1}
emu = EmuOps()


def _ops():
    from tempura_amd.kernels import ops
    return ops


class _Folders:
    """Model folders by case; for bfloat16 runs the routers' choices are no close calls (``apart``)."""

    def __init__(self, root):
        self.root, self.made = root, {}

    def get(self, name, dtype="float32"):
        apart = dtype == "bfloat16"
        if (name, apart) not in self.made:
            self.made[(name, apart)] = cases.write_model(name, str(self.root / f"{name}{int(apart)}"), weights=cases.make_weights(name, apart=apart))
        return self.made[(name, apart)]

    def __getitem__(self, name):
        return self.get(name)


@pytest.fixture(scope="module")
def dirs(tmp_path_factory):
    return _Folders(tmp_path_factory.mktemp("bomotar_gpu"))


def _close(got, want, tol):
    got, want = got.double().cpu(), want.double().cpu()
    assert got.shape == want.shape
    err = float((got - want).abs().max() / max(1e-30, float(want.abs().max())))
    assert err <= tol, f"relative error {err:.3e} > {tol:.1e}"


def _batch(runs, slots):
    """cu_seqlens, token_req, state slots of a batch of runs."""
    cu = torch.tensor([0] + list(torch.tensor(runs).cumsum(0)), dtype=torch.int32)
    token_req = torch.tensor([i for i, l in enumerate(runs) for _ in range(l)], dtype=torch.int32)
    return cu, token_req, torch.tensor(slots, dtype=torch.int32)


# ---- kernels alone ------------------------------------------------------------------------------
@pytest.mark.parametrize("hidden", [64, 37, 1030])
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_embedding_with_a_bigram_row_and_a_carried_token(hidden, dtype):
    ops = _ops()
    g = torch.Generator().manual_seed(hidden)
    vocab, buckets, mp, mc = 90, 53, 1000003, 77
    table, bigram = torch.randn(vocab, hidden, generator=g).to(dtype), torch.randn(buckets + 1, hidden, generator=g).to(dtype)
    runs, slots = [3, 1, 2, 9], [4, 0, 2, 1]
    cu, token_req, sl = _batch(runs, slots)
    state = torch.randint(0, vocab, (6, 1), generator=g, dtype=torch.int32)
    s_ref, s_dev = state.clone(), state.to(DEV)
    pos = torch.tensor([0, 1, 2, 7, 0, 1, 5, 6, 7, 8, 9, 10, 11, 12, 13], dtype=torch.int32)      # two runs start a request
    for _ in range(2):
        tok = torch.randint(0, vocab, (15,), generator=g, dtype=torch.int32)
        want = emu.embed_bigram(tok, table, bigram, pos, token_req, cu, sl, s_ref, 4, mp, mc, buckets)
        got = ops.embed_bigram(tok.to(DEV), table.to(DEV), bigram.to(DEV), pos.to(DEV), token_req.to(DEV), cu.to(DEV), sl.to(DEV), s_dev,
                               4, mp, mc, buckets)
        assert float((got.cpu().double() - want.double()).abs().max()) < 1e-6
        assert torch.equal(s_dev.cpu(), s_ref)
        pos = pos + torch.tensor([3] * 3 + [1] + [2] * 2 + [9] * 9, dtype=torch.int32)
    assert int(s_ref[3]) == int(state[3])


@pytest.mark.parametrize("channels,taps,act,bias", [(40, 4, False, False), (7, 1, True, True), (130, 2, False, True), (300, 5, True, False)])
def test_causal_conv_without_activation_at_an_offset_of_the_state(channels, taps, act, bias):
    ops = _ops()
    g = torch.Generator().manual_seed(channels)
    col0, width, off = 11, 11 + channels + 6, 17
    w, b = torch.randn(taps, channels, generator=g), (torch.randn(channels, generator=g) if bias else None)
    state = torch.randn(5, off + (taps - 1) * channels + 13, generator=g)
    cu, token_req, slots = _batch([3, 1, 2, 9], [4, 0, 2, 1])
    proj = torch.randn(15, width, generator=g)
    s_ref, s_dev = state.clone(), state.to(DEV)
    for _ in range(3):                                      # three steps in a row: what one leaves the next reads
        want = emu.causal_conv(proj, col0, channels, w, b, s_ref, cu, token_req, slots, 4, off, act)
        got = ops.causal_conv(proj.to(DEV), col0, channels, w.to(DEV), None if b is None else b.to(DEV), s_dev, cu.to(DEV),
                              token_req.to(DEV), slots.to(DEV), 4, state_off=off, act=act)
        _close(got, want, 2e-6)
        _close(s_dev, s_ref, 0)
        proj = proj * 0.9 + 0.1
    assert torch.equal(s_dev.cpu()[3], state[3]) and torch.equal(s_dev.cpu()[:, :off], state[:, :off])


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("heads,kvh,d,vd,ps,rd,pad", [(4, 2, 16, 24, 16, 8, 0), (3, 3, 10, 6, 8, 10, 0), (6, 3, 64, 128, 16, 64, 0), (2, 1, 32, 64, 32, 0, 0),
                                                      (2, 2, 8, 8, 16, 4, 0), (6, 3, 64, 128, 16, 64, 128), (4, 1, 32, 64, 16, 16, 64), (2, 2, 16, 96, 16, 8, 96),
                                                      (3, 1, 10, 32, 8, 6, 32)])
@pytest.mark.parametrize("n", [21, 300])
def test_values_of_another_size_into_the_cache_and_out_of_it(dtype, heads, kvh, d, vd, ps, rd, pad, n):
    """Rotation and cache write with values wider or narrower than keys, then attention over them with one far key
    that stands out: the first rows attend from a context of 40 tokens whose third key matches every query.  ``pad``:
    q and the cached keys as wide as the values, zeros behind their own elements (the matrix-core kernels then serve)."""
    ops = _ops()
    g = torch.Generator().manual_seed(heads * 100 + d + n)
    ctx0 = 40
    total = ctx0 + n
    pages = (total + ps - 1) // ps
    order = torch.randperm(pages + 3, generator=g)[:pages].to(torch.int32)
    kc, vc = torch.zeros(pages + 4, kvh, ps, pad or d, dtype=dtype), torch.zeros(pages + 4, kvh, vd, ps, dtype=dtype)
    inv = torch.pow(torch.tensor(10000.0, dtype=torch.float64), -2.0 * torch.arange(rd // 2, dtype=torch.float64) / max(rd, 1)) if rd else None
    kd, vdv = kc.to(DEV), vc.to(DEV)
    qs = []
    for lo, cnt in ((0, ctx0), (ctx0, n)):                    # the context first, then the rows that are graded
        rows = torch.randn(cnt, (heads + kvh) * d + kvh * vd, generator=g)
        if lo == 0:
            rows[2, heads * d: (heads + kvh) * d] *= 6.0      # a key far back that the queries below lean on
        pos = torch.arange(lo, lo + cnt, dtype=torch.int32)
        slots = torch.tensor([int(order[p // ps]) * ps + p % ps for p in range(lo, lo + cnt)], dtype=torch.int32)
        q = ops.rope_kv_write(rows.to(DEV), pos.to(DEV), slots.to(DEV), None if inv is None else inv.to(DEV), rd, 1.25, heads, kvh, d,
                              kd, vdv, dtype, value_dim=vd, pad_dim=pad or None)
        qr = emu.rope_kv_write(rows, pos, slots, inv, rd, 1.25, heads, kvh, d, kc, vc, dtype, value_dim=vd, pad_dim=pad or None)
        assert q.shape == (cnt, heads, pad or d)
        tol = 2e-6 if dtype == torch.float32 else 1e-2
        _close(q, qr, tol)
        qs.append(qr)
    _close(kd, kc, tol)
    _close(vdv, vc, tol)
    table = torch.full((1, pages + 2), -1, dtype=torch.int32)
    table[0, :pages] = order
    cu = torch.tensor([0, n], dtype=torch.int32)
    lens = torch.tensor([total], dtype=torch.int32)
    token_req = torch.zeros(n, dtype=torch.int32)
    got = ops.paged_attention(qs[1].to(DEV), kd, vdv, table.to(DEV), cu.to(DEV), lens.to(DEV), token_req.to(DEV), 0.7, 0, n, total, 0)
    want = emu.paged_attention(qs[1], kc, vc, table, cu, lens, token_req, 0.7, 0, n, total)
    assert got.shape == (n, heads * vd)
    _close(got, want, 2e-5 if dtype == torch.float32 else 2e-2)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_gate_on_the_heads_into_a_wider_buffer(dtype):
    ops = _ops()
    g = torch.Generator().manual_seed(2)
    a = torch.randn(13, 70, generator=g).to(dtype)
    proj = torch.randn(13, 200, generator=g) * 3
    out = torch.full((13, 101), 7.0).to(dtype)
    ref = out.clone()
    dev = out.to(DEV)
    ops.sigmoid_gate(a.to(DEV), proj.to(DEV), 90, 0.6, dev, 20)
    emu.sigmoid_gate(a, proj, 90, 0.6, ref, 20)
    _close(dev, ref, 1e-6 if dtype == torch.float32 else 8e-3)
    ops.sigmoid_gate(a.to(DEV), None, 0, 1.5, dev, 3)
    emu.sigmoid_gate(a, None, 0, 1.5, ref, 3)
    _close(dev, ref, 1e-6 if dtype == torch.float32 else 8e-3)
    assert torch.equal(dev.cpu()[:, :3], out[:, :3])


@pytest.mark.parametrize("width", [48, 256, 1000, 1024, 2048, 4096, 5000, 8192, 8196])
@pytest.mark.parametrize("out_dtype", [None, torch.float32, torch.bfloat16])
def test_norm_of_a_sublayers_output_into_the_stream(width, out_dtype):
    ops = _ops()
    g = torch.Generator().manual_seed(width)
    h, y = torch.randn(9, width, generator=g), torch.randn(9, width, generator=g) * 30
    w, w2 = torch.randn(width, generator=g), torch.randn(width, generator=g)
    h_ref, h_dev = h.clone(), h.to(DEV)
    if out_dtype is None:
        assert ops.norm_add(h_dev, y.to(DEV), w.to(DEV), 1e-5) is None
        emu.norm_add(h_ref, y, w, 1e-5)
    else:
        x = ops.norm_add(h_dev, y.to(DEV), w.to(DEV), 1e-5, w2.to(DEV), 1e-6, out_dtype)
        _close(x, emu.norm_add(h_ref, y, w, 1e-5, w2, 1e-6, out_dtype), 2e-6 if out_dtype == torch.float32 else 8e-3)
    _close(h_dev, h_ref, 1e-6)


@pytest.mark.parametrize("kind", ["gelu_tanh", "silu"])
@pytest.mark.parametrize("out_dtype", [torch.float32, torch.bfloat16])
def test_activation(kind, out_dtype):
    ops = _ops()
    u = torch.cat([torch.linspace(-12, 12, 997), torch.tensor([0.0, -0.0, 1e-20, 80.0, -80.0])]).reshape(2, -1)
    _close(ops.activation(u.to(DEV), kind, out_dtype), emu.activation(u, kind, out_dtype), 2e-6 if out_dtype == torch.float32 else 8e-3)


@pytest.mark.parametrize("E,top,groups,keep", [(6, 2, 3, 2), (8, 4, 4, 3), (4, 1, 1, 1), (12, 3, 2, 1), (5, 5, 1, 1), (64, 6, 8, 4),
                                               (130, 7, 10, 3), (16, 2, 16, 3)])
def test_router_chooses_by_corrected_scores_within_the_best_groups(E, top, groups, keep):
    ops = _ops()
    g = torch.Generator().manual_seed(E * 10 + top)
    n = 77
    logits = torch.randn(n, E + 3, generator=g) * 2
    corr = torch.randn(E, generator=g) * 0.2 - 0.1           # negative choice scores happen
    dense, ids, wts = ops.moe_route(logits.to(DEV), corr.to(DEV), E, top, groups, keep)
    d_ref, i_ref, w_ref = emu.moe_route(logits, corr, E, top, groups, keep)
    assert torch.equal(ids.cpu(), i_ref)
    _close(wts, w_ref, 2e-6)
    _close(dense, d_ref, 2e-6)
    assert int((dense > 0).sum()) == n * top


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_experts_activations_as_rows_of_their_own_times_the_weights(dtype):
    ops = _ops()
    g = torch.Generator().manual_seed(4)
    n, E, ff = 19, 5, 24
    dense = torch.rand(n, E, generator=g) * (torch.rand(n, E, generator=g) > 0.5)
    a = torch.randn(n, E * ff, generator=g).to(dtype)
    got = ops.moe_spread(a.to(DEV), dense.to(DEV), E)
    assert got.shape == (E, n, ff)
    _close(got, emu.moe_spread(a, dense, E), 1e-6 if dtype == torch.float32 else 8e-3)


@pytest.mark.parametrize("n,top,E,width,dtype", [(77, 2, 6, 48, torch.float32), (1000, 4, 8, 64, torch.bfloat16), (5, 1, 4, 32, torch.bfloat16),
                                                  (300, 3, 130, 200, torch.float32)])
def test_rows_in_the_order_of_the_experts_and_back(n, top, E, width, dtype):
    ops = _ops()
    g = torch.Generator().manual_seed(n)
    ids = torch.stack([torch.randperm(E, generator=g)[:top] for _ in range(n)]).to(torch.int32)
    x = torch.randn(n, width, generator=g).to(dtype)
    counts, offsets, rank = ops.moe_plan(ids.to(DEV), E)
    c_ref, o_ref, r_ref = emu.moe_plan(ids, E)
    assert torch.equal(counts.cpu(), c_ref) and torch.equal(offsets.cpu(), o_ref) and torch.equal(rank.cpu(), r_ref)
    xg, row_of = ops.moe_gather(x.to(DEV), ids.to(DEV), rank, offsets)
    xg_ref, row_ref = emu.moe_gather(x, ids, r_ref, o_ref)
    assert torch.equal(row_of.cpu(), row_ref) and torch.equal(xg.cpu(), xg_ref)
    assert sorted(row_ref.reshape(-1).tolist()) == list(range(n * top))
    yg = torch.randn(n * top, width, generator=g)
    wts = torch.rand(n, top, generator=g)
    _close(ops.moe_scatter(yg.to(DEV), row_of, wts.to(DEV)), emu.moe_scatter(yg, row_ref, wts), 2e-6)
    y0 = torch.randn(n, width, generator=g)
    y_dev = y0.to(DEV)
    ops.moe_scatter(yg.to(DEV), row_of, wts.to(DEV), y_dev)
    _close(y_dev, emu.moe_scatter(yg, row_ref, wts, y0.clone()), 2e-6)


@pytest.mark.parametrize("rank,n_out,mode", [(5, 48, "plain"), (24, 256, "decay"), (3, 20, "sigmoid"), (64, 1000, "decay"), (9, 130, "sigmoid")])
def test_second_product_of_a_low_rank_projection(rank, n_out, mode):
    ops = _ops()
    g = torch.Generator().manual_seed(rank)
    n, col0 = 21, 6
    x = torch.randn(n, col0 + rank + 4, generator=g)
    wt = torch.randn(rank, n_out, generator=g) * rank ** -0.5
    per = n_out // 4 if mode == "decay" else 0
    a_log = torch.randn(4, generator=g) if mode == "decay" else None
    bias = torch.randn(n_out, generator=g) - 1.0 if mode == "decay" else None
    got = ops.lowrank_up(x.to(DEV), col0, wt.to(DEV), mode, None if a_log is None else a_log.to(DEV), None if bias is None else bias.to(DEV), per)
    _close(got, emu.lowrank_up(x, col0, wt, mode, a_log, bias, per), 3e-6)


@pytest.mark.parametrize("H,G,D,Dv", [(4, 2, 12, 10), (1, 1, 20, 40), (2, 2, 7, 5), (4, 2, 64, 32), (2, 2, 128, 48), (3, 1, 96, 130), (2, 1, 300, 16),
                                      (8, 8, 32, 64)])
def test_delta_rule_and_its_state(H, G, D, Dv):
    """Runs of one token, a few and many beside each other, three steps in a row from states that are not zero;
    one step's k of one request is scaled up so that its write dominates the read-out that follows."""
    ops = _ops()
    g = torch.Generator().manual_seed(H * 1000 + D)
    runs, slot_list = [3, 1, 40, 9], [4, 0, 2, 1]
    cu, _, slots = _batch(runs, slot_list)
    n = sum(runs)
    off = 23
    state = torch.randn(6, off + H * D * Dv + 5, generator=g) * 0.3
    s_ref, s_dev = state.clone(), state.to(DEV)
    for step in range(3):
        qkv = torch.randn(n, 2 * G * D + H * Dv, generator=g)
        if step == 1:
            qkv[10, G * D: 2 * G * D] *= 9.0
        decay = torch.rand(n, H * D, generator=g) * 0.6 + 0.4
        proj = torch.randn(n, H + 9, generator=g) * 2
        want = emu.delta_scan(qkv, decay, proj, 4, s_ref, off, cu, slots, 4, H, G, D, Dv, D ** -0.5, 1e-6)
        got = ops.delta_scan(qkv.clone().to(DEV), decay.to(DEV), proj.to(DEV), 4, s_dev, off, cu.to(DEV), slots.to(DEV), 4, H, G, D, Dv, D ** -0.5, 1e-6)
        _close(got, want, 2e-5)
        _close(s_dev, s_ref, 2e-5)
    assert torch.equal(s_dev.cpu()[3], state[3]) and torch.equal(s_dev.cpu()[:, :off], state[:, :off])
    assert torch.equal(s_dev.cpu()[:, off + H * D * Dv:], state[:, off + H * D * Dv:])


def test_delta_rule_token_by_token_is_the_run():
    """300 tokens as one run, and the same tokens one a step: the same chain, so the same bits."""
    ops = _ops()
    g = torch.Generator().manual_seed(8)
    H, G, D, Dv, n = 2, 1, 64, 48, 300
    qkv0 = torch.randn(n, 2 * G * D + H * Dv, generator=g).to(DEV)
    qkv = qkv0.clone()
    decay = (torch.rand(n, H * D, generator=g) * 0.3 + 0.7).to(DEV)
    proj = torch.randn(n, H, generator=g).to(DEV)
    one = torch.tensor([0], dtype=torch.int32, device=DEV)
    s1 = torch.zeros(2, H * D * Dv, device=DEV)
    whole = ops.delta_scan(qkv, decay, proj, 0, s1, 0, torch.tensor([0, n], dtype=torch.int32, device=DEV), one, 1, H, G, D, Dv, 0.125, 1e-6)
    s2 = torch.zeros(2, H * D * Dv, device=DEV)
    cu1 = torch.tensor([0, 1], dtype=torch.int32, device=DEV)
    rows = [ops.delta_scan(qkv0[t: t + 1].contiguous(), decay[t: t + 1].contiguous(), proj[t: t + 1].contiguous(), 0, s2, 0, cu1, one, 1,
                           H, G, D, Dv, 0.125, 1e-6) for t in range(n)]
    assert torch.equal(torch.cat(rows), whole) and torch.equal(s1, s2)


@pytest.mark.parametrize("heads,vdim", [(4, 10), (1, 40), (3, 130), (16, 128)])
@pytest.mark.parametrize("out_dtype", [torch.float32, torch.bfloat16])
def test_norm_per_head_with_a_gate(heads, vdim, out_dtype):
    ops = _ops()
    g = torch.Generator().manual_seed(heads + vdim)
    n = 11
    o = torch.randn(n, heads * vdim, generator=g) * 5
    w, gate = torch.randn(vdim, generator=g), torch.rand(n, heads * vdim, generator=g)
    out = torch.zeros(n, heads * vdim + 9).to(out_dtype)
    ref = out.clone()
    dev = out.to(DEV)
    ops.head_norm_gate(o.to(DEV), w.to(DEV), gate.to(DEV), 1e-5, 0.9, heads, dev, 5)
    emu.head_norm_gate(o, w, gate, 1e-5, 0.9, heads, ref, 5)
    _close(dev, ref, 2e-6 if out_dtype == torch.float32 else 8e-3)
    ops.head_norm_gate(o.to(DEV), w.to(DEV), None, 1e-5, 1.0, heads, dev, 0)
    emu.head_norm_gate(o, w, None, 1e-5, 1.0, heads, ref, 0)
    _close(dev, ref, 2e-6 if out_dtype == torch.float32 else 8e-3)


# ---- the model through the step function --------------------------------------------------------
def _runner(folder, dtype, max_tokens, page_size=16, max_requests=4, use_graph=False):
    from tempura_amd.engine.loading import load_model
    from tempura_amd.engine.runner import ModelRunner
    model = load_model(folder, dtype, DEV)
    return ModelRunner(model, page_size, (max_tokens + page_size - 1) // page_size, max_requests=max_requests, use_graph=use_graph)


_REFS = {}


def _ref(name, rid, dtype):
    key = (name, rid, dtype == "bfloat16")
    if key not in _REFS:
        _REFS[key] = plain.forward(cases.config_json(name), cases.make_weights(name, apart=key[2]), cases.requests(name)[rid])
    return _REFS[key]


@pytest.mark.parametrize("name", ["pair", "solo", "wide", "many"])
def test_each_part_alone_matches_its_plain_function(dirs, name):
    import bomotar_mechanisms
    bomotar_mechanisms.check(dirs[name], name, DEV, 2e-5)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", ["pair", "solo", "wide", "many"])
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
    runner = _runner(dirs.get(name, dtype), dtype, max_tokens)
    got = helpers.run_schedule(runner, reqs, steps)
    for rid in reqs:
        err = plain.logit_error(got[rid], _ref(name, rid, dtype))
        assert err < TOL[dtype], f"{name}/{mode}/{dtype}: request {rid}: error {err:.3e}"
    assert not runner.cache.live_requests()
    assert runner.cache.free_pages() == [p.num_pages for p in runner.cache.pools]


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_cutting_changes_rounding_only(dirs, dtype):
    """The same request whole, in portions and beside others: float32 differs in summation order only; bfloat16 runs
    differ by what their roundings differ (other product kernels for other row counts, the routed feed-forward's
    two ways), which stays at half of what a bfloat16 run may differ from the exact result."""
    reqs = cases.requests("wide")
    lengths = cases.LENGTHS["wide"]
    runs = []
    for steps in (helpers.schedule_whole(lengths), helpers.schedule_portions(lengths, sizes=(2, 9, 33, 2, 16, 5)),
                  helpers.schedule_mixed(lengths, 448, seed=3)):
        runs.append(helpers.run_schedule(_runner(dirs.get("wide", dtype), dtype, 448), reqs, steps))
    for rid in reqs:
        for other in runs[1:]:
            assert plain.logit_error(other[rid], runs[0][rid]) < (2e-5 if dtype == "float32" else TOL["bfloat16"] / 2), rid


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_sharp_attention_over_far_keys_on_the_gpu(tmp_path, dtype):
    """Queries many times larger than drawn (a softmax that rests on one or two keys anywhere in the context): a
    prompt of 400 tokens whole, then in portions that end at and beside page borders with decoding behind them."""
    from tempura_amd.engine.runner import StepEntry
    cfg = cases.config_json("wide")
    # (bfloat16: scores as large as the queries carry rounding errors as large, so the queries are 2.5 instead of 6
    # times the drawn ones and the bound is a fifth of what losing the oldest keys costs)
    W = cases.make_weights("wide", sharp=6.0 if dtype == "float32" else 2.5, apart=dtype == "bfloat16")
    folder = cases.write_model("wide", str(tmp_path / "sharp"), weights=W)
    toks = cases.tokens("wide", 400, 5)
    ref = plain.forward(cfg, W, toks)
    # (the premise: what losing the oldest keys costs)
    assert plain.logit_error(plain.forward(cfg, W, toks[200:])[-50:], ref[-50:]) > 1.5
    tol = TOL[dtype] if dtype == "float32" else 0.3
    runner = _runner(folder, dtype, 448 + 448)
    runner.add_request("w")
    whole = runner.step([StepEntry("w", toks, list(range(400)))]).cpu()
    assert plain.logit_error(whole, ref) < tol
    runner.add_request("r")
    rows, at = [], 0
    for c in (16, 15, 2, 31, 257, 40, 3):
        rows.append(runner.step([StepEntry("r", toks[at: at + c], list(range(c)))]).cpu())
        at += c
    rows += [runner.step([StepEntry("r", [t], [0])]).cpu() for t in toks[at:]]
    assert plain.logit_error(torch.cat(rows), ref) < tol


def test_long_decoding_through_a_captured_step(dirs):
    """Two requests decoded token by token for 150 steps through the graph path: pages, carried convolution
    inputs, recurrent states and last tokens all move along."""
    from tempura_amd.engine.runner import StepEntry
    cfg, W = cases.config_json("wide"), cases.make_weights("wide")
    runner = _runner(dirs["wide"], "float32", 512, use_graph=True)
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


@pytest.mark.parametrize("name", ["pair", "wide"])
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
    toks = cases.tokens("pair", 30, 5)
    out = tmp_path / "out"
    steps = [{"step": 0, "entries": [{"id": "a", "tokens": toks[:11], "want": [0, 10]}], "end": []},
             {"step": 1, "entries": [{"id": "a", "tokens": toks[11:13], "want": []}], "end": []},
             {"step": 2, "entries": [{"id": "a", "tokens": toks[13:], "want": [16]}, {"id": "b", "tokens": toks[:4], "want": [3]}], "end": ["a", "b"]}]
    for dtype in ("float32", "bfloat16"):
        p = subprocess.run([os.path.join(root, "bin", "trace_run"), "--model", dirs.get("pair", dtype), "--dtype", dtype, "--out", str(out),
                            "--max-tokens", "128"], input="".join(json.dumps(s) + "\n" for s in steps), capture_output=True, text=True, timeout=600)
        assert p.returncode == 0, p.stderr[-2000:]
        assert [l for l in p.stdout.splitlines() if l.startswith("done")] == ["done 0", "done 1", "done 2"]
        ref = plain.forward(cases.config_json("pair"), cases.make_weights("pair", apart=dtype == "bfloat16"), toks)
        vocab = ref.shape[1]
        a = torch.from_numpy(np.fromfile(out / "0.f32", dtype="<f4").reshape(-1, vocab))
        c = torch.from_numpy(np.fromfile(out / "2.f32", dtype="<f4").reshape(-1, vocab))
        assert plain.logit_error(torch.cat([a, c]), torch.stack([ref[0], ref[10], ref[29], ref[3]])) < TOL[dtype]
