"""Each mechanism of the Bomotar design alone: the framework's part, taken out of a loaded model and run on random
rows through the step's own context and cache, against the plain function of tests/plain_bomotar.py for it.  Used by
the host tests (over the stand-in operations) and by the GPU tests (over the kernels)."""
from __future__ import annotations

import torch

import bomotar_cases as cases
import plain_bomotar as plain


def _err(got, ref):
    got, ref = got.double().cpu(), ref.double()
    return float((got - ref).abs().max() / ref.abs().max())


def check(folder: str, name: str, device: str, tol: float, seed: int = 0) -> None:
    """Asserts, for every layer of case ``name`` that has tensors of its own: the left and the right mixer alone (as
    a prompt of 37 tokens in two portions), the feed-forward, and the embedding across a step's border."""
    from tempura_amd.engine.loading import load_model
    from tempura_amd.engine.runner import ModelRunner, StepEntry
    cfg, W = cases.config_json(name), cases.make_weights(name)
    W64 = {k: v.double() for k, v in W.items()}
    model = load_model(folder, "float32", device)
    runner = ModelRunner(model, 16, 8, max_requests=2)
    get = lambda key, optional=False: W[key]
    g = torch.Generator().manual_seed(seed)
    n, cut = 37, 21
    toks = cases.tokens(name, n, 3)
    eps = float(cfg["norm"]["eps"])
    own = [i for i, l in enumerate(cfg["layers"]) if l.get("weights_of") is None]
    x = torch.randn(n, cfg["width"], generator=g)
    runner.add_request("r")
    outs = {}
    for lo, hi in ((0, cut), (cut, n)):
        tok_dev, ctx = runner._pack_step([StepEntry("r", toks[lo:hi], [])])
        runner._clear_state([s for s, q, c in zip(ctx.state_slot_list, ctx.q_lens, ctx.ctx_lens) if c == q])
        rows = x[lo:hi].to(device)
        emb = model.embedding.forward(tok_dev, ctx.positions, 1, ctx=ctx, state=runner.pools.state[model.EMBEDDING_STATE])
        outs.setdefault("embed", []).append(emb.cpu())
        for k, i in enumerate(own):
            block = model.layers[k]
            cache = runner.layer_caches[[c.layer for c in model.order].index(k)]
            for side, branch in zip(("left", "right"), block.mixer.branches):
                if lo == 0:
                    branch.load_weights(get)      # (the branch as a mixer of its own: its own two products)
                outs.setdefault((i, side), []).append(branch.forward(rows, ctx, cache).cpu())
            if block.ffn is not None:
                outs.setdefault((i, "ffn"), []).append(block.ffn.forward(rows, ctx).cpu())
        runner.cache.commit_many(["r"], ctx.q_lens)
    bg = cfg["embedding"]["bigram"]
    ref = plain.embed_tokens(toks, W64["embed"], W64["bigram"], bg["mul_prev"], bg["mul_cur"], bg["buckets"])
    assert _err(torch.cat(outs["embed"]), ref) < tol, "embedding"
    xd, pos = x.double(), torch.arange(n)
    for i in own:
        layer, p = cfg["layers"][i], f"l{i}"
        ref = plain.left_mixer(xd, W64, p + ".mix.left", layer["mixer"]["left"], pos)
        assert _err(torch.cat(outs[(i, "left")]), ref) < tol, f"layer {i}: left mixer"
        ref = plain.right_mixer(xd, W64, p + ".mix.right", layer["mixer"]["right"], eps)
        assert _err(torch.cat(outs[(i, "right")]), ref) < tol, f"layer {i}: right mixer"
        mlp = layer["mlp"]
        if mlp is not None:
            ref = plain.dense_mlp(xd, W64, p + ".mlp") if mlp["kind"] == "dense" else plain.moe_mlp(xd, W64, p + ".mlp", mlp)
            assert _err(torch.cat(outs[(i, "ffn")]), ref) < tol, f"layer {i}: feed-forward"
