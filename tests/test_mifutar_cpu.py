"""The Mifutar design through the engine's own model, cache and state manager, step function and scheduler on the
host: the kernel operations are replaced by their plain PyTorch stand-ins (tests/emu_ops.py), the expected values
come from the plain implementation in tests/plain_mifutar.py.  A difference here is a fault of the configuration,
the parts, the cache, the state slots or the batch."""
import json

import pytest
import torch

import helpers
import mifutar_cases as cases
import plain_mifutar as plain
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
    root = tmp_path_factory.mktemp("mifutar")
    return {name: cases.write_model(name, str(root / name)) for name in cases.CASES}


def _runner(dirs, name, max_tokens, page_size=16, max_requests=4):
    from tempura_amd.engine.loading import load_model
    from tempura_amd.engine.runner import ModelRunner
    model = load_model(dirs[name], "float32", "cpu")
    return ModelRunner(model, page_size, (max_tokens + page_size - 1) // page_size, max_requests=max_requests)


def _plain(name):
    return cases.config_json(name), cases.make_weights(name)


# ---- configuration ------------------------------------------------------------------------------
def test_config_reads_every_size_and_writes_it_back():
    from tempura_amd.config import ConfigError, MifutarConfig
    from tempura_amd.parts.inventory import expected_weights
    for name in cases.CASES:
        d = cases.config_json(name)
        cfg = MifutarConfig.from_dict(d)
        again = MifutarConfig.from_json(cfg.to_json())
        assert again == cfg
        assert cfg.width == d["width"] and cfg.vocab == d["vocab"] and cfg.streams == d.get("streams")
        want = {k: tuple(v.shape) for k, v in cases.make_weights(name).items()}
        got = expected_weights(cfg.build_spec())
        assert set(got) == set(want)
        for k, info in got.items():
            assert all(e is None or e == f for e, f in zip(info.shape, want[k])) and len(info.shape) == len(want[k]), k
    bad = cases.config_json("mix")
    bad["layers"][1]["mixer"]["vdim"] = 8
    with pytest.raises(ConfigError):
        MifutarConfig.from_dict(bad)
    bad = cases.config_json("mix")
    bad["layers"][0]["type"] = "lstm"
    with pytest.raises(ConfigError):
        MifutarConfig.from_dict(bad)
    bad = cases.config_json("mix")
    del bad["layers"][0]["mixer"]["state"]
    with pytest.raises(ConfigError):
        MifutarConfig.from_dict(bad)
    bad = cases.config_json("mix")
    bad["layers"][2]["mlp"]["kind"] = "routed"
    with pytest.raises(ConfigError):
        MifutarConfig.from_dict(bad)


def test_registry_chooses_the_design_by_config_json(dirs):
    from tempura_amd.config import MifutarConfig, load_config
    assert isinstance(load_config(dirs["ssm"]), MifutarConfig)


def test_a_checkpoint_with_a_wrong_tensor_is_refused(dirs, tmp_path):
    from tempura_amd.engine.loading import load_model
    from tempura_amd.weights import WeightsError
    W = cases.make_weights("mix")
    W["l1.mix.rel"] = W["l1.mix.rel"][:, :2].contiguous()          # heads do not fit
    del W["l0.hc1.mix"]
    cases.write_model("mix", str(tmp_path / "bad"), weights=W)
    with pytest.raises(WeightsError) as e:
        load_model(str(tmp_path / "bad"), "float32", "cpu")
    assert "l0.hc1.mix" in e.value.missing and "l1.mix.rel" in e.value.wrong_shape


def test_distance_table_is_the_bucket_rule():
    from tempura_amd.parts.attention import distance_table
    g = torch.Generator().manual_seed(3)
    for rows, far, window in [(6, 12, 7), (5, 16, 20), (8, 64, 500), (4, 30, None), (10, 16, 16), (2, 9, None), (1, 5, 40), (16, 200, 90)]:
        rel = torch.randn(rows, 3, generator=g)
        table = distance_table(rel, far, window)
        reach = 400 if window is None else window
        for n in range(reach):
            want = rel[plain.distance_bucket(n, rows, far) if rows > 1 else 0]
            assert torch.equal(table[:, min(n, table.shape[1] - 1)], want), (rows, far, window, n)


# ---- the model through the step function --------------------------------------------------------
@pytest.mark.parametrize("name", ["mix", "ssm", "attn"])
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
    runner = _runner(dirs, name, max_tokens)
    got = helpers.run_schedule(runner, reqs, steps)
    for rid, toks in reqs.items():
        ref = plain.forward(cfg, W, toks)
        bad = helpers.first_difference(got[rid], ref, TOL)
        assert bad is None, f"{name}/{mode}: request {rid} first differs at position {bad}"
    assert not runner.cache.live_requests()
    assert runner.cache.free_pages() == [p.num_pages for p in runner.cache.pools]


def test_residual_after_every_layer_matches_plain(dirs):
    from tempura_amd.engine.runner import StepEntry
    cfg, W = _plain("mix")
    toks = cases.tokens("mix", 19, 7)
    want = []
    plain.forward(cfg, W, toks, want)
    runner = _runner(dirs, "mix", 64)
    seen = {}
    runner.model.observer = lambda i, h: seen.__setitem__(i, h.double().clone())
    runner.add_request("r")
    runner.step([StepEntry("r", toks, [])])
    for i, ref in enumerate(want):
        assert float((seen[i + 1] - ref).abs().max() / ref.abs().max()) < TOL, f"after layer {i}"


def test_state_slots_and_pages_are_used_again(dirs):
    """Two state slots and a pool of six pages for five requests one after the other and side by side: a slot's
    or a page's last owner must leave nothing behind."""
    from tempura_amd.engine.runner import StepEntry
    cfg, W = _plain("mix")
    runner = _runner(dirs, "mix", 96, max_requests=2)
    reqs = cases.requests("mix")
    order = ["m2", "m1", "m4", "m0", "m5"]
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


def test_window_edge_decides(dirs, tmp_path):
    """The distance table gives the key at the window's last place a bias that outweighs everything else: a window
    one key too short or too long changes the result beyond any tolerance, in a prompt and in decoding."""
    from tempura_amd.engine.loading import load_model
    from tempura_amd.engine.runner import ModelRunner, StepEntry
    cfg = cases.config_json("mix")
    W = cases.make_weights("mix")
    for li in (1, 3):
        m = cases.CASES["mix"]["layers"][li]["mixer"]
        edge = plain.distance_bucket(m["mask"]["size"] - 1, m["_rows"], m["bias_max"])
        assert edge != plain.distance_bucket(0, m["_rows"], m["bias_max"])
        W[f"l{li}.mix.rel"] = W[f"l{li}.mix.rel"].clone()
        W[f"l{li}.mix.rel"][edge] += 14.0
    folder = cases.write_model("mix", str(tmp_path / "edge"), weights=W)
    toks = cases.tokens("mix", 45, 3)
    ref = plain.forward(cfg, W, toks)
    # the plain implementation with windows one off must differ visibly, or the test would prove nothing
    for delta in (-1, 1):
        off = json.loads(json.dumps(cfg))
        for li in (1, 3):
            off["layers"][li]["mixer"]["mask"]["size"] += delta
        assert plain.logit_error(plain.forward(off, W, toks)[25:], ref[25:]) > 0.05
    model = load_model(folder, "float32", "cpu")
    runner = ModelRunner(model, 16, 8, max_requests=2)
    runner.add_request("r")
    a = runner.step([StepEntry("r", toks[:30], list(range(30)))])
    rows = [a] + [runner.step([StepEntry("r", [t], [0])]) for t in toks[30:]]
    assert plain.logit_error(torch.cat(rows), ref) < 1e-4


def test_first_tokens_and_single_token_requests(dirs):
    from tempura_amd.engine.runner import StepEntry
    for name in ("mix", "ssm", "attn"):
        cfg, W = _plain(name)
        runner = _runner(dirs, name, 64)
        toks = cases.tokens(name, 4, 9)
        ref = plain.forward(cfg, W, toks)
        runner.add_request("x")
        rows = [runner.step([StepEntry("x", [t], [0])]) for t in toks]          # from the very first token on, one by one
        assert plain.logit_error(torch.cat(rows), ref) < 1e-4, name


# ---- generation through the engine's entry point and scheduler ----------------------------------
@pytest.mark.parametrize("name", ["mix", "ssm"])
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
    """`tempura inspect` on a folder of the design, and `tempura random-model --config-json` for it (the rows of
    the distance table named in the file, since no checkpoint is there to say them)."""
    from tempura_amd.cli import main
    from tempura_amd.engine.loading import load_model
    assert main(["inspect", dirs["mix"]]) == 0
    text = capsys.readouterr().out
    assert "Mifutar" in text and "mamba2 4 heads of 8" in text and "window 7" in text
    cfg = cases.config_json("attn")
    for layer, rows in zip(cfg["layers"], (8, 4, 10)):
        layer["mixer"]["bias_buckets"] = rows
    path = tmp_path / "c.json"
    path.write_text(json.dumps(cfg))
    assert main(["random-model", "--config-json", str(path), "--out", str(tmp_path / "rnd"), "--std", "0.3"]) == 0
    model = load_model(str(tmp_path / "rnd"), "float32", "cpu")
    assert model.layers[2].mixer.dist_table.shape[0] == 6 and model.streams == 1
    # connection tensors are drawn around the plain residual sum
    assert abs(float(model.layers[0].mixer_link.mix[0, 0]) - 1.0) < 1.5
