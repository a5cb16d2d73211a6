"""Small Bomotar configurations and random weights of the tests' own making (stored as bfloat16 values, so that the
float32 and the bfloat16 engine and the plain implementation all read the same numbers)."""
from __future__ import annotations

import json
import os
from typing import Dict, List

import torch


def _left(heads, kv, dim, vdim, conv, rot_dims=None, base=10000.0, scaling=None, scale=None):
    m = {"heads": heads, "kv_heads": kv, "dim": dim, "vdim": vdim, "conv": conv, "scale": scale if scale is not None else dim ** -0.5}
    if rot_dims:
        m["rot"] = {"dims": rot_dims, "base": base}
        if scaling:
            m["rot"]["scaling"] = dict(zip(("factor", "original", "fast", "slow"), scaling))
    return m


def _right(heads, kv, dim, vdim, conv, ra, rg):
    return {"heads": heads, "kv_heads": kv, "dim": dim, "vdim": vdim, "conv": conv, "_ranks": (ra, rg)}


def _dense(ff):
    return {"kind": "dense", "ff": ff}


def _moe(ff, experts, top, groups=None):
    r = {"experts": experts, "top": top}
    if groups:
        r["groups"] = {"count": groups[0], "keep": groups[1]}
    return {"kind": "moe", "expert": {"ff": ff}, "router": r}


def _layer(left, right, mlp, ls=1.0, rs=1.0, weights_of=None):
    d = {"type": "parallel", "mixer": {"left": left, "right": right, "left_scale": ls, "right_scale": rs}, "mlp": mlp}
    if weights_of is not None:
        d["weights_of"] = weights_of
    return d


def _case(vocab, width, layers, buckets, mp, mc, mult=None, eps=1e-6):
    d = {"architecture": "Bomotar", "vocab": vocab, "width": width, "norm": {"eps": eps},
         "embedding": {"bigram": {"buckets": buckets, "mul_prev": mp, "mul_cur": mc}}, "layers": layers}
    if mult is not None:
        d["residual_mult"] = mult
    return d


_PA = (_left(4, 2, 16, 24, 3, rot_dims=8, base=5000.0, scaling=(4.0, 64, 8.0, 1.0), scale=0.3), _right(4, 2, 12, 10, 2, 5, 7))
_PB = (_left(3, 3, 10, 6, 2, rot_dims=10, base=300.0), _right(2, 1, 20, 18, 4, 9, 3))

_MA = (_left(8, 2, 48, 96, 2, rot_dims=24, base=1e5, scaling=(3.0, 256, 8.0, 1.0), scale=0.2), _right(6, 3, 80, 40, 5, 12, 20))
_MB = (_left(4, 4, 32, 32, 3, rot_dims=32, base=2e4), _right(4, 1, 48, 96, 2, 6, 10))

#: name -> config.json content ("_ranks": ranks of the right mixer's low-rank projections, sizes only the tensors say)
CASES: Dict[str, dict] = {
    # two kinds of layers, each run twice (the second time with a cache and state of its own), a layer without a
    # feed-forward between them; partial rotation with scaling; values wider than keys; grouped key heads
    "pair": _case(70, 48, [_layer(*_PA, _dense(80), 0.55, 1.3),
                           _layer(*_PB, _moe(24, 6, 2, (3, 2)), 1.1, 0.8),
                           _layer(*_PA, _dense(80), 0.55, 1.3, weights_of=0),
                           _layer(_left(2, 1, 8, 8, 5), _right(3, 3, 6, 14, 1, 4, 4), None, 0.9, 0.7),
                           _layer(*_PB, _moe(24, 6, 2, (3, 2)), 1.1, 0.8, weights_of=1)], 53, 31, 7, mult=0.7, eps=1e-5),
    # one layer kind, no residual constant, no groups, one expert a token, one tap on the left (no carried
    # inputs), unrotated keys beside full rotation, a key size that fills no power of two
    "solo": _case(40, 32, [_layer(_left(2, 2, 8, 8, 1, rot_dims=8, base=100.0), _right(1, 1, 20, 40, 4, 2, 6), _moe(16, 4, 1)),
                           _layer(_left(4, 1, 6, 12, 4), _right(2, 2, 7, 5, 3, 3, 2), _dense(44))], 17, 3, 5),
    # sizes the matrix-core kernels take: heads of 64 with values of 64, heads of 32 with values of 64, a recurrence
    # with keys of 64 and of 128, eight experts in four groups
    "wide": _case(96, 128, [_layer(_left(4, 2, 64, 64, 4, rot_dims=32, base=500000.0, scaling=(6.0, 128, 16.0, 2.0), scale=0.11),
                                   _right(4, 2, 64, 32, 3, 16, 16), _dense(256), 0.7, 0.85),
                            _layer(_left(2, 1, 32, 64, 3, rot_dims=32, base=10000.0), _right(2, 2, 128, 48, 4, 8, 24),
                                   _moe(64, 8, 3, (4, 2)), 1.0, 0.5),
                            _layer(_left(4, 2, 64, 64, 4, rot_dims=32, base=500000.0, scaling=(6.0, 128, 16.0, 2.0), scale=0.11),
                                   _right(4, 2, 64, 32, 3, 16, 16), _dense(256), 0.7, 0.85, weights_of=0)], 211, 13, 29, mult=0.6),
    # five layers of three kinds: keys of 48 under values of 96 and of 64 under 128 (padded onto the matrix cores in
    # bfloat16), four query heads a key head, a recurrence with keys of 80 (no power of two) and five taps, sixteen
    # experts in eight groups, three a token; a width that is no power of two
    "many": _case(300, 192, [_layer(*_MA, _moe(40, 16, 3, (8, 3)), 0.8, 1.2), _layer(*_MB, _dense(200), 1.0, 0.4),
                             _layer(*_MA, _moe(40, 16, 3, (8, 3)), 0.8, 1.2, weights_of=0), _layer(*_MB, _dense(200), 1.0, 0.4, weights_of=1),
                             _layer(_left(2, 1, 64, 128, 4, rot_dims=16, base=777.0, scaling=(2.0, 64, 4.0, 0.5)),
                                    _right(2, 2, 32, 32, 3, 4, 4), None, 0.5, 0.5)], 997, 101, 13, mult=0.3),
}


def config_json(name: str) -> dict:
    """The case as config.json would hold it (without the tests' private keys)."""
    cfg = json.loads(json.dumps(CASES[name]))
    for layer in cfg["layers"]:
        layer["mixer"]["right"].pop("_ranks", None)
    return cfg


def make_weights(name: str, seed: int = 0, sharp: float = 1.0, apart: bool = False) -> Dict[str, torch.Tensor]:
    """bfloat16 tensors by checkpoint name, drawn so that every mechanism matters to the logits.  ``sharp``
    multiplies the attention's query projections: with large values a query's softmax rests on one or two keys
    somewhere in its context, far ones as often as near ones.  ``apart``: the routers' corrections lie 1.5 apart,
    more than two scores can differ, so that no choice of experts is a close call (for runs in bfloat16, whose
    rounding would flip close calls; the scores still weigh the chosen experts)."""
    cfg = CASES[name]
    g = torch.Generator().manual_seed(seed)
    W: Dict[str, torch.Tensor] = {}

    def normal(*shape, std=1.0, mean=0.0):
        return torch.randn(*shape, generator=g, dtype=torch.float64) * std + mean

    width = cfg["width"]
    bg = cfg["embedding"]["bigram"]
    W["embed"] = normal(cfg["vocab"], width)
    W["bigram"] = normal(bg["buckets"] + 1, width, std=0.7)
    W["head"] = normal(cfg["vocab"], width, std=width ** -0.5)
    W["final.norm"] = normal(width, std=0.2, mean=1.0)
    for i, layer in enumerate(cfg["layers"]):
        if layer.get("weights_of") is not None:
            continue
        p = f"l{i}"
        for nm in ("norm1", "norm1b"):
            W[f"{p}.{nm}"] = normal(width, std=0.2, mean=1.0)
        a, r = layer["mixer"]["left"], layer["mixer"]["right"]
        H, G, D, Dv, K = a["heads"], a["kv_heads"], a["dim"], a["vdim"], a["conv"]
        q = f"{p}.mix.left"
        W[q + ".q"] = normal(H * D, width, std=sharp * 1.5 * width ** -0.5)
        W[q + ".k"] = normal(G * D, width, std=1.5 * width ** -0.5)
        W[q + ".v"] = normal(G * Dv, width, std=width ** -0.5)
        for nm, ch in (("q", H * D), ("k", G * D), ("v", G * Dv)):
            W[f"{q}.{nm}.conv"] = normal(ch, K, std=0.4) + torch.cat([torch.zeros(ch, K - 1, dtype=torch.float64), torch.ones(ch, 1, dtype=torch.float64)], 1)
        W[q + ".g"] = normal(H * Dv, width, std=width ** -0.5)
        W[q + ".o"] = normal(width, H * Dv, std=(H * Dv) ** -0.5)
        H, G, D, Dv, K = r["heads"], r["kv_heads"], r["dim"], r["vdim"], r["conv"]
        ra, rg = r["_ranks"]
        q = f"{p}.mix.right"
        W[q + ".q"] = normal(G * D, width, std=width ** -0.5)
        W[q + ".k"] = normal(G * D, width, std=width ** -0.5)
        W[q + ".v"] = normal(H * Dv, width, std=width ** -0.5)
        for nm, ch in (("q", G * D), ("k", G * D), ("v", H * Dv)):
            W[f"{q}.{nm}.conv"] = normal(ch, K, std=0.5)
        W[q + ".b"] = normal(H, width, std=width ** -0.5)
        W[q + ".A_log"] = torch.log(torch.rand(H, generator=g, dtype=torch.float64) * 1.5 + 0.05)
        W[q + ".dt_bias"] = normal(H * D, std=0.8, mean=-1.5)
        W[q + ".a1"] = normal(ra, width, std=width ** -0.5)
        W[q + ".a2"] = normal(H * D, ra, std=ra ** -0.5)
        W[q + ".g1"] = normal(rg, width, std=width ** -0.5)
        W[q + ".g2"] = normal(H * Dv, rg, std=rg ** -0.5)
        W[q + ".norm"] = normal(Dv, std=0.2, mean=1.0)
        W[q + ".o"] = normal(width, H * Dv, std=(H * Dv) ** -0.5)
        mlp = layer["mlp"]
        if mlp is None:
            continue
        for nm in ("norm2", "norm2b"):
            W[f"{p}.{nm}"] = normal(width, std=0.2, mean=1.0)
        if mlp["kind"] == "dense":
            W[f"{p}.mlp.up"] = normal(mlp["ff"], width, std=1.5 * width ** -0.5)
            W[f"{p}.mlp.down"] = normal(width, mlp["ff"], std=mlp["ff"] ** -0.5)
        else:
            E, ff = mlp["router"]["experts"], mlp["expert"]["ff"]
            W[f"{p}.mlp.router"] = normal(E, width, std=2.0 * width ** -0.5)
            # (corrections as large as the scores' differences: the choice and the weights then often disagree,
            # and some choice scores are negative)
            W[f"{p}.mlp.correction"] = normal(E, std=0.15, mean=-0.05)
            if apart:
                W[f"{p}.mlp.correction"] = (torch.randperm(E, generator=g).to(torch.float64) - E / 2) * 1.5
            for e in range(E):
                W[f"{p}.mlp.e{e}.gate"] = normal(ff, width, std=1.5 * width ** -0.5)
                W[f"{p}.mlp.e{e}.up"] = normal(ff, width, std=1.5 * width ** -0.5)
                W[f"{p}.mlp.e{e}.down"] = normal(width, ff, std=ff ** -0.5)
    return {k: v.to(torch.bfloat16) for k, v in W.items()}


def write_model(name: str, folder: str, seed: int = 0, weights=None) -> str:
    from tempura_amd.weights import write_safetensors
    os.makedirs(folder, exist_ok=True)
    with open(os.path.join(folder, "config.json"), "w") as f:
        json.dump(config_json(name), f)
    W = weights if weights is not None else make_weights(name, seed)
    write_safetensors(os.path.join(folder, "model.safetensors"), W.items(), metadata={"format": "pt"})
    return folder


def tokens(name: str, n: int, seed: int) -> List[int]:
    g = torch.Generator().manual_seed(4321 + seed)
    return torch.randint(0, CASES[name]["vocab"], (n,), generator=g).tolist()


#: request lengths per case: one token, a few, around pages' edges, long
LENGTHS = {"pair": {"p0": 1, "p1": 6, "p2": 23, "p3": 49, "p4": 33, "p5": 16},
           "solo": {"s0": 2, "s1": 31, "s2": 17, "s3": 1, "s4": 40},
           "wide": {"w0": 5, "w1": 70, "w2": 33, "w3": 129, "w4": 48},
           "many": {"n0": 1, "n1": 37, "n2": 150, "n3": 64}}


def requests(name: str) -> Dict[str, List[int]]:
    return {rid: tokens(name, n, i) for i, (rid, n) in enumerate(LENGTHS[name].items())}
