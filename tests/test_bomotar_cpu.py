"""The Bomotar design through the engine's own model, cache and state manager, step function and scheduler on the
host: the kernel operations are replaced by their plain PyTorch stand-ins (tests/emu_ops.py), the expected values
come from the plain implementation in tests/plain_bomotar.py.  A difference here is a fault of the configuration,
the parts, the cache, the state slots or the batch."""
import json

import pytest
import torch

import bomotar_cases as cases
import helpers
import plain_bomotar as plain
from emu_ops import EmuOps

TOL = 2e-5      # float32 storage of activations against float64


@pytest.fixture(autouse=True)
def host_ops():
    from tempura_amd.kernels import ops
    ops.set_backend(EmuOps())
    yield
    ops.set_backend(None)


@pytest.fixture(scope="module")
def dirs(tmp_path_factory):
    root = tmp_path_factory.mktemp("bomotar")
    return {name: cases.write_model(name, str(root / name)) for name in cases.CASES}


def _runner(folder, max_tokens, page_size=16, max_requests=4):
    from tempura_amd.engine.loading import load_model
    from tempura_amd.engine.runner import ModelRunner
    model = load_model(folder, "float32", "cpu")
    return ModelRunner(model, page_size, (max_tokens + page_size - 1) // page_size, max_requests=max_requests)


def _plain(name):
    return cases.config_json(name), cases.make_weights(name)


# ---- configuration ------------------------------------------------------------------------------
def test_config_reads_every_size_and_writes_it_back():
    from tempura_amd.config import BomotarConfig, ConfigError
    from tempura_amd.parts.inventory import expected_weights
    for name in cases.CASES:
        d = cases.config_json(name)
        cfg = BomotarConfig.from_dict(d)
        assert BomotarConfig.from_json(cfg.to_json()) == cfg
        assert cfg.width == d["width"] and cfg.vocab == d["vocab"] and cfg.residual_mult == d.get("residual_mult", 1.0)
        want = {k: tuple(v.shape) for k, v in cases.make_weights(name).items()}
        got = expected_weights(cfg.build_spec())
        assert set(got) == set(want)
        for k, info in got.items():
            assert all(e is None or e == f for e, f in zip(info.shape, want[k])) and len(info.shape) == len(want[k]), k
    spec = BomotarConfig.from_dict(cases.config_json("pair")).build_spec()
    assert len(spec.layers) == 3 and [c.layer for c in spec.order] == [0, 1, 0, 2, 1]
    for change in (lambda c: c["layers"][0].__setitem__("type", "serial"),
                   lambda c: c["layers"][0]["mixer"]["left"].__setitem__("kv_heads", 3),
                   lambda c: c["layers"][0]["mixer"]["right"].pop("vdim"),
                   lambda c: c["layers"][1]["mlp"].__setitem__("kind", "sparse"),
                   lambda c: c["layers"][1]["mlp"]["router"].__setitem__("top", 5),      # more than the kept groups hold
                   lambda c: c["layers"][2].__setitem__("weights_of", 2),
                   lambda c: c["layers"][2]["mixer"].__setitem__("left_scale", 0.5),      # sizes of the layer whose tensors it runs
                   lambda c: c["embedding"].pop("bigram"),
                   lambda c: c["layers"][0]["mixer"]["left"]["rot"].__setitem__("dims", 7)):
        bad = cases.config_json("pair")
        change(bad)
        with pytest.raises(ConfigError):
            BomotarConfig.from_dict(bad)


def test_registry_chooses_the_design_by_config_json(dirs):
    from tempura_amd.config import BomotarConfig, load_config
    assert isinstance(load_config(dirs["solo"]), BomotarConfig)


def test_a_checkpoint_with_a_wrong_tensor_is_refused(dirs, tmp_path):
    from tempura_amd.engine.loading import load_model
    from tempura_amd.weights import WeightsError
    W = cases.make_weights("pair")
    W["l0.mix.right.norm"] = W["l0.mix.right.norm"][:4].contiguous()
    del W["l1.mlp.e3.up"]
    del W["bigram"]
    W["l2.norm1"] = W["l0.norm1"]          # a layer that runs another's tensors has none of its own
    cases.write_model("pair", str(tmp_path / "bad"), weights=W)
    with pytest.raises(WeightsError) as e:
        load_model(str(tmp_path / "bad"), "float32", "cpu")
    assert {"l1.mlp.e3.up", "bigram"} <= set(e.value.missing) and "l0.mix.right.norm" in e.value.wrong_shape
    assert "l2.norm1" in e.value.unexpected


def test_a_layer_run_twice_has_a_cache_and_a_state_of_its_own(dirs):
    runner = _runner(dirs["pair"], 64)
    m = runner.model
    assert len(m.order) == 5 and len({c.cache for c in m.order}) == 5 and all(m.call_writes)
    assert m.layers[m.order[0].layer] is m.layers[m.order[2].layer]
    states = [runner.layer_caches[i].state for i in range(5)]
    assert len({s.data_ptr() for s in states}) == 5
    assert states[0].shape == states[2].shape and states[0].shape != states[3].shape
    assert m.EMBEDDING_STATE in m.state_specs and runner.pools.state[m.EMBEDDING_STATE].dtype == torch.int32


# ---- mechanisms alone, against the plain functions ----------------------------------------------
def test_yarn_frequencies_are_the_plain_ones():
    from tempura_amd.parts.rope import rotary_inv_freq
    for dims, base, sc in [(8, 5000.0, (4.0, 64, 8.0, 1.0)), (64, 800000.0, (5.0, 2048, 24.0, 2.0)), (32, 10000.0, (2.0, 4096, 4.0, 0.5)),
                           (16, 100.0, (16.0, 8, 2.0, 1.0)), (10, 300.0, None)]:
        scaling = None if sc is None else dict(zip(("factor", "original", "fast", "slow"), sc))
        want, _ = plain.yarn_frequencies(dims, base, scaling)
        got = rotary_inv_freq(dims + 6, base, None if sc is None else dict(scaling, type="yarn"), dims)
        assert torch.allclose(got, want, rtol=1e-14, atol=0), (dims, base, sc)


def test_router_stand_in_is_the_plain_router():
    g = torch.Generator().manual_seed(5)
    for E, top, groups in [(6, 2, (3, 2)), (8, 4, (4, 3)), (4, 1, None), (12, 3, (2, 1)), (5, 5, None), (16, 2, (16, 3))]:
        h = torch.randn(40, 24, generator=g, dtype=torch.float64)
        W = {"m.router": torch.randn(E, 24, generator=g, dtype=torch.float64), "m.correction": torch.randn(E, generator=g, dtype=torch.float64) * 0.2 - 0.1}
        r = {"experts": E, "top": top}
        if groups:
            r["groups"] = {"count": groups[0], "keep": groups[1]}
        idx, wts = plain.route(h, W, "m", r)
        dense, ids, w2 = EmuOps().moe_route((h @ W["m.router"].T).float(), W["m.correction"].float(), E, top, groups[0] if groups else 1,
                                            groups[1] if groups else 1)
        assert torch.equal(ids.long().sort(dim=1).values, idx.sort(dim=1).values), (E, top, groups)
        assert torch.allclose(dense.double().sum(1), wts.sum(1), atol=1e-6)
        assert int((dense > 0).sum()) == 40 * top


@pytest.mark.parametrize("name", ["pair", "solo"])
def test_each_part_alone_matches_its_plain_function(dirs, name):
    import bomotar_mechanisms
    bomotar_mechanisms.check(dirs[name], name, "cpu", TOL)


# ---- the model through the step function --------------------------------------------------------
@pytest.mark.parametrize("name", ["pair", "solo"])
@pytest.mark.parametrize("mode", ["whole", "bulk_tail", "portions", "mixed"])
def test_every_cutting_matches_plain(dirs, name, mode):
    cfg, W = _plain(name)
    reqs = cases.requests(name)
    lengths = cases.LENGTHS[name]
    if mode == "mixed":
        max_tokens = sum(sorted(helpers.roundup(n, 64) for n in lengths.values())[-2:]) + 64
        steps = helpers.schedule_mixed(lengths, max_tokens, seed=11)
    else:
        max_tokens = max(helpers.roundup(n, 64) for n in lengths.values())
        steps = {"whole": helpers.schedule_whole, "bulk_tail": lambda l: helpers.schedule_bulk_tail(l, tail=9),
                 "portions": lambda l: helpers.schedule_portions(l, sizes=(7, 2, 16, 3, 2, 5, 2, 9, 2, 17))}[mode](lengths)
    runner = _runner(dirs[name], max_tokens)
    got = helpers.run_schedule(runner, reqs, steps)
    for rid, toks in reqs.items():
        ref = plain.forward(cfg, W, toks)
        bad = helpers.first_difference(got[rid], ref, TOL)
        assert bad is None, f"{name}/{mode}: request {rid} first differs at position {bad}"
    assert not runner.cache.live_requests()
    assert runner.cache.free_pages() == [p.num_pages for p in runner.cache.pools]


def test_residual_after_every_layer_matches_plain(dirs):
    from tempura_amd.engine.runner import StepEntry
    cfg, W = _plain("pair")
    toks = cases.tokens("pair", 19, 7)
    want = []
    plain.forward(cfg, W, toks, want)
    runner = _runner(dirs["pair"], 64)
    seen = {}
    runner.model.observer = lambda i, h: seen.__setitem__(i, h.double().clone())
    runner.add_request("r")
    runner.step([StepEntry("r", toks, [])])
    assert len(want) == 5
    for i, ref in enumerate(want):
        assert float((seen[i + 1] - ref).abs().max() / ref.abs().max()) < TOL, f"after layer {i}"


def test_state_slots_and_pages_are_used_again(dirs):
    """Two state slots and a pool of six pages for five requests one after the other and side by side: a slot's
    or a page's last owner must leave nothing behind (carried convolution inputs, a recurrent state, a last token)."""
    from tempura_amd.engine.runner import StepEntry
    cfg, W = _plain("pair")
    runner = _runner(dirs["pair"], 96, max_requests=2)
    reqs = cases.requests("pair")
    order = ["p2", "p1", "p4", "p0", "p5"]
    slots_seen = []
    for k in range(0, len(order), 2):
        pair = order[k: k + 2]
        for rid in pair:
            runner.add_request(rid)
            slots_seen.append(runner.cache.state_slot(rid))
        done = {rid: 0 for rid in pair}
        got = {rid: [] for rid in pair}
        while any(done[r] < len(reqs[r]) for r in pair):
            batch = []
            for rid in pair:
                c = min(5, len(reqs[rid]) - done[rid])
                if c > 0:
                    batch.append(StepEntry(rid, reqs[rid][done[rid]: done[rid] + c], list(range(c))))
                    done[rid] += c
            logits = runner.step(batch)
            row = 0
            for e in batch:
                got[e.rid].append(logits[row: row + len(e.tokens)].clone())
                row += len(e.tokens)
        for rid in pair:
            runner.end_request(rid)
            ref = plain.forward(cfg, W, reqs[rid])
            assert helpers.first_difference(torch.cat(got[rid]), ref, TOL) is None, rid
    assert len(set(slots_seen)) == 2 and len(slots_seen) == 5


def test_sharp_attention_over_far_keys_and_page_borders(dirs, tmp_path):
    """Queries many times larger than drawn: a query's softmax rests on one or two keys anywhere in its context, so
    a key that is lost, misplaced or read from a wrong page changes the logits beyond any tolerance.  A long prompt
    in portions that end at and beside page borders, then decoding across two more borders."""
    from tempura_amd.engine.runner import StepEntry
    cfg = cases.config_json("pair")
    W = cases.make_weights("pair", sharp=8.0)
    folder = cases.write_model("pair", str(tmp_path / "sharp"), weights=W)
    toks = cases.tokens("pair", 150, 5)
    ref = plain.forward(cfg, W, toks)
    # the test's premise: losing the oldest keys must show (the plain implementation on a prompt without them differs)
    assert plain.logit_error(plain.forward(cfg, W, toks[40:])[-20:], ref[-20:]) > 0.5
    runner = _runner(folder, 192)
    runner.add_request("r")
    rows, at = [], 0
    for c in (16, 15, 2, 31, 17, 32, 3):
        rows.append(runner.step([StepEntry("r", toks[at: at + c], list(range(c)))]))
        at += c
    rows += [runner.step([StepEntry("r", [t], [0])]) for t in toks[at:]]
    assert plain.logit_error(torch.cat(rows), ref) < 1e-4


def test_first_tokens_and_single_token_requests(dirs):
    """From the very first token on, one token a step: the bigram row of a request's first token, zeros before the
    start of every convolution, a state that starts at zero."""
    from tempura_amd.engine.runner import StepEntry
    for name in ("pair", "solo"):
        cfg, W = _plain(name)
        runner = _runner(dirs[name], 64)
        toks = cases.tokens(name, 6, 9)
        ref = plain.forward(cfg, W, toks)
        runner.add_request("x")
        rows = [runner.step([StepEntry("x", [t], [0])]) for t in toks]
        assert plain.logit_error(torch.cat(rows), ref) < 1e-4, name
        # the slot's next owner starts from nothing as well
        runner.end_request("x")
        runner.add_request("y")
        again = runner.step([StepEntry("y", toks[:3], [0, 1, 2])])
        assert plain.logit_error(again, ref[:3]) < 1e-4, name


def test_the_bigram_row_of_a_portions_first_token_is_the_last_tokens_of_the_step_before(dirs):
    """Two requests whose portions alternate: each one's previous token is its own, not its neighbour's in the batch."""
    from tempura_amd.engine.runner import StepEntry
    cfg, W = _plain("solo")
    a, b = cases.tokens("solo", 12, 1), cases.tokens("solo", 9, 2)
    runner = _runner(dirs["solo"], 128)
    runner.add_request("a")
    runner.add_request("b")
    got = {"a": [], "b": []}
    runner.step([StepEntry("a", a[:5], [])])
    got["b"].append(runner.step([StepEntry("b", b[:1], [0])]))
    out = runner.step([StepEntry("b", b[1:4], [0, 1, 2]), StepEntry("a", a[5:6], [0])])
    got["b"].append(out[:3]); got["a"].append(out[3:])
    out = runner.step([StepEntry("a", a[6:], list(range(6))), StepEntry("b", b[4:], list(range(5)))])
    got["a"].append(out[:6]); got["b"].append(out[6:])
    assert plain.logit_error(torch.cat(got["a"]), plain.forward(cfg, W, a)[5:]) < 1e-4
    assert plain.logit_error(torch.cat(got["b"]), plain.forward(cfg, W, b)) < 1e-4


# ---- generation through the engine's entry point and scheduler ----------------------------------
@pytest.mark.parametrize("name", ["pair", "solo"])
def test_engine_generates_what_plain_greedy_generates(dirs, name):
    from tempura_amd.engine import Engine
    from tempura_amd.sampling import SamplingParams
    cfg, W = _plain(name)
    prompts = [cases.tokens(name, n, 20 + i) for i, n in enumerate((3, 18, 9))]
    eng = Engine(dirs[name], dtype="float32", page_size=16, kv_pages=12, max_batch_size=2, max_num_batched_tokens=16,
                 prefill_chunk_size=7, device="cpu", use_graph=False)
    outs = eng.generate(prompts, SamplingParams(temperature=0.0, max_new_tokens=6))
    for p, o in zip(prompts, outs):
        assert o == plain.greedy(cfg, W, p, 6)


def test_command_line_inspects_and_writes_random_folders(dirs, tmp_path, capsys):
    """`tempura inspect` on a folder of the design, and `tempura random-model --config-json` for it (the ranks of the
    low-rank projections named in the file, since no checkpoint is there to say them)."""
    from tempura_amd.cli import main
    from tempura_amd.engine.loading import load_model
    assert main(["inspect", dirs["pair"]]) == 0
    text = capsys.readouterr().out
    assert "Bomotar" in text and "6 experts of 24, 2 a token, 2 of 3 groups" in text and "tensors of layer 0" in text
    cfg = cases.config_json("solo")
    for layer, (ra, rg) in zip(cfg["layers"], ((2, 6), (3, 2))):
        layer["mixer"]["right"]["decay_rank"], layer["mixer"]["right"]["gate_rank"] = ra, rg
    path = tmp_path / "c.json"
    path.write_text(json.dumps(cfg))
    assert main(["random-model", "--config-json", str(path), "--out", str(tmp_path / "rnd"), "--std", "0.3"]) == 0
    model = load_model(str(tmp_path / "rnd"), "float32", "cpu")
    assert model.layers[0].mixer.branches[1].a2_t.shape == (2, 20) and model.layers[1].mixer.branches[1].g2_t.shape == (2, 10)
