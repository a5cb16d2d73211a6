"""Small Mifutar configurations and random weights of the tests' own making (stored as bfloat16 values, so that
the float32 and the bfloat16 engine and the plain implementation all read the same numbers)."""
from __future__ import annotations

import json
import math
import os
from typing import Dict, List

import torch


def _mamba(heads, vdim, state, groups, conv, norm_groups):
    return {"heads": heads, "vdim": vdim, "state": state, "groups": groups, "conv": conv, "norm_groups": norm_groups}


def _attn(heads, kv, dim, window, rows, far, scale=None):
    m = {"heads": heads, "kv_heads": kv, "dim": dim, "vdim": dim, "scale": scale if scale is not None else dim ** -0.5,
         "bias_max": far, "_rows": rows}
    if window is not None:
        m["mask"] = {"size": window}
    return m


def _layer(kind, mixer, ff=None, limit=1.0):
    return {"type": kind, "mixer": mixer, "mlp": None if ff is None else {"ff": ff, "kind": "dense", "limit": limit}}


#: name -> config.json content ("_rows": rows of an attention layer's distance table, a size only the tensor says)
CASES: Dict[str, dict] = {
    # both mixers, three streams, a layer without feed-forward, odd sizes, a window shorter than a page and one
    # that ends inside the second page
    "mix": {"architecture": "Mifutar", "vocab": 50, "width": 64, "streams": 3, "logit_scale": 0.75, "norm": {"eps": 1e-5},
            "layers": [_layer("mamba2", _mamba(4, 8, 16, 2, 3, 1), 96, 1.0),
                       _layer("attention", _attn(4, 2, 16, 7, 6, 12)),
                       _layer("mamba2", _mamba(2, 24, 5, 1, 2, 2), 80, 0.5),
                       _layer("attention", _attn(3, 3, 10, 20, 5, 16, scale=0.4), 72, 2.0)]},
    # no streams key: the plain residual sum; state-space layers only (no paged cache at all); one tap, five taps
    "ssm": {"architecture": "Mifutar", "vocab": 40, "width": 48, "logit_scale": 1.0, "norm": {"eps": 1e-6},
            "layers": [_layer("mamba2", _mamba(3, 16, 8, 3, 1, 3), 64, 3.0),
                       _layer("mamba2", _mamba(6, 4, 40, 2, 5, 1)),
                       _layer("mamba2", _mamba(1, 32, 12, 1, 4, 4), 56, 0.8)]},
    # one stream with connection tensors of size one; attention only: one key/value head, a window longer than any
    # prompt here, no window at all, and a window of exactly one page
    "attn": {"architecture": "Mifutar", "vocab": 60, "width": 32, "streams": 1, "logit_scale": 2.0, "norm": {"eps": 1e-6},
             "layers": [_layer("attention", _attn(4, 1, 8, 500, 8, 64), 48, 1.0),
                        _layer("attention", _attn(2, 2, 12, None, 4, 30), 44, 1.25),      # (44: no multiple of eight)
                        _layer("attention", _attn(6, 3, 6, 16, 10, 16))]},
    # MFMA-friendly sizes: heads of 32 and 64, state 64, pages of 16 with windows at and beside page borders
    "wide": {"architecture": "Mifutar", "vocab": 96, "width": 128, "streams": 2, "logit_scale": 0.25, "norm": {"eps": 1e-5},
             "layers": [_layer("attention", _attn(4, 2, 32, 33, 14, 40), 256, 1.75),
                        _layer("mamba2", _mamba(4, 32, 64, 2, 4, 2), 192, 1.25),
                        _layer("attention", _attn(2, 1, 64, 48, 12, 100), 128, 1.0),
                        _layer("mamba2", _mamba(8, 16, 32, 1, 4, 1))]},
}


def config_json(name: str) -> dict:
    """The case as config.json would hold it (without the tests' private keys)."""
    cfg = json.loads(json.dumps(CASES[name]))
    for layer in cfg["layers"]:
        layer["mixer"].pop("_rows", None)
    return cfg


def make_weights(name: str, seed: int = 0) -> Dict[str, torch.Tensor]:
    """bfloat16 tensors by checkpoint name, drawn so that every mechanism matters to the logits."""
    cfg = CASES[name]
    g = torch.Generator().manual_seed(seed)
    W: Dict[str, torch.Tensor] = {}

    def normal(*shape, std=1.0, mean=0.0):
        return torch.randn(*shape, generator=g, dtype=torch.float64) * std + mean

    width, S = cfg["width"], cfg.get("streams")
    W["embed"] = normal(cfg["vocab"], width)
    W["head"] = normal(cfg["vocab"], width, std=width ** -0.5)
    W["final.norm"] = normal(width, std=0.2)
    for i, layer in enumerate(cfg["layers"]):
        p, m = f"l{i}", layer["mixer"]
        W[f"{p}.norm1"] = normal(width, std=0.2)
        if layer["type"] == "attention":
            H, G, d = m["heads"], m["kv_heads"], m["dim"]
            W[f"{p}.mix.q"] = normal(H * d, width, std=width ** -0.5)
            W[f"{p}.mix.k"] = normal(G * d, width, std=width ** -0.5)
            W[f"{p}.mix.q.b"] = normal(H * d, std=0.3)
            W[f"{p}.mix.k.b"] = normal(G * d, std=0.3)
            W[f"{p}.mix.rel"] = normal(m["_rows"], H)
            W[f"{p}.mix.o"] = normal(width, H * d, std=(H * d) ** -0.5)
        else:
            H, P, N, G, K = m["heads"], m["vdim"], m["state"], m["groups"], m["conv"]
            inner, ch = H * P, H * P + 2 * G * N
            W[f"{p}.mix.in"] = normal(2 * inner + 2 * G * N + H, width, std=width ** -0.5)
            W[f"{p}.mix.conv"] = normal(ch, K, std=0.5)
            W[f"{p}.mix.conv.b"] = normal(ch, std=0.2)
            W[f"{p}.mix.dt_bias"] = normal(H, std=0.7, mean=-0.5)
            W[f"{p}.mix.A_log"] = torch.log(torch.rand(H, generator=g, dtype=torch.float64) * 2.0 + 0.05)
            W[f"{p}.mix.D"] = normal(H, std=0.3, mean=1.0)
            W[f"{p}.mix.norm"] = normal(inner, std=0.2, mean=1.0)
            W[f"{p}.mix.o"] = normal(width, inner, std=inner ** -0.5)
        if S is not None:
            for q in (1, 2):
                if q == 2 and layer["mlp"] is None:
                    continue
                W[f"{p}.hc{q}.in"] = normal(S, std=0.3, mean=1.0 / S)
                W[f"{p}.hc{q}.out"] = normal(S, std=0.3, mean=1.0)
                W[f"{p}.hc{q}.mix"] = torch.eye(S, dtype=torch.float64) + normal(S, S, std=0.2)
        if layer["mlp"] is not None:
            ff = layer["mlp"]["ff"]
            W[f"{p}.norm2"] = normal(width, std=0.2)
            W[f"{p}.mlp.gate"] = normal(ff, width, std=1.5 * width ** -0.5)      # (wide enough that the limits bite)
            W[f"{p}.mlp.up"] = normal(ff, width, std=1.5 * width ** -0.5)
            W[f"{p}.mlp.down"] = normal(width, ff, std=ff ** -0.5)
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
    g = torch.Generator().manual_seed(1234 + seed)
    return torch.randint(0, CASES[name]["vocab"], (n,), generator=g).tolist()


#: request lengths per case: one token, a few, around pages' and windows' edges, long
LENGTHS = {"mix": {"m0": 1, "m1": 6, "m2": 23, "m3": 49, "m4": 33, "m5": 16},
           "ssm": {"s0": 2, "s1": 31, "s2": 17, "s3": 1, "s4": 40},
           "attn": {"a0": 3, "a1": 35, "a2": 17, "a3": 16, "a4": 52},
           "wide": {"w0": 5, "w1": 70, "w2": 33, "w3": 129, "w4": 48}}


def requests(name: str) -> Dict[str, List[int]]:
    return {rid: tokens(name, n, i) for i, (rid, n) in enumerate(LENGTHS[name].items())}
