"""The Mifutar design written out plainly: whole sequences, no cache, float64, one function per mechanism.

Nothing here is shared with the product path; the functions take the configuration as the plain dict that
config.json holds and the weights as a dict of tensors by checkpoint name.  Notation: T tokens, width W,
S streams; a mixer's tensors are ``<layer>.mix.<name>``, a feed-forward's ``<layer>.mlp.<name>``.
"""
from __future__ import annotations

import math
from typing import Dict, List, Optional

import torch

F = torch.float64


def unit_rms(x: torch.Tensor, eps: float) -> torch.Tensor:
    """x / sqrt(mean(x^2) + eps) over the last dimension."""
    return x / torch.sqrt((x * x).mean(dim=-1, keepdim=True) + eps)


def offset_norm(x: torch.Tensor, w: torch.Tensor, eps: float) -> torch.Tensor:
    """The layer norm of the design: unit root mean square, times (1 + w)."""
    return unit_rms(x, eps) * (1.0 + w)


def sinusoid(T: int, width: int, start: int = 0) -> torch.Tensor:
    """[T, width]: entry 2i of position p is sin(p * 10000^(-2i / width)), entry 2i + 1 its cosine."""
    out = torch.zeros(T, width, dtype=F)
    for t in range(T):
        p = start + t
        for j in range(width):
            ang = p * 10000.0 ** (-2.0 * (j // 2) / width)
            out[t, j] = math.cos(ang) if j % 2 else math.sin(ang)
    return out


def distance_bucket(n: int, rows: int, far: int) -> int:
    """Row of the distance table that distance n reads (exact below half of the rows, then logarithmic up to ``far``)."""
    half = rows // 2
    if n < half:
        return n
    return min(rows - 1, half + int(math.floor(math.log(n / half) / math.log(far / half) * (rows - half))))


def windowed_attention(m: dict, W: Dict[str, torch.Tensor], p: str, h: torch.Tensor) -> torch.Tensor:
    """Grouped-query attention whose values are its keys, with projection biases, a learned bias by distance
    and a sliding window; softmax over the visible keys; output projection."""
    T = h.shape[0]
    H, G, d = m["heads"], m["kv_heads"], m["dim"]
    q = (h @ W[p + ".q"].T + W[p + ".q.b"]).reshape(T, H, d)
    k = (h @ W[p + ".k"].T + W[p + ".k.b"]).reshape(T, G, d)
    rel = W[p + ".rel"]
    rows, far = rel.shape[0], m["bias_max"]
    window = m["mask"]["size"] if m.get("mask") else None
    out = torch.zeros(T, H, d, dtype=F)
    for i in range(T):
        first = 0 if window is None else max(0, i - window + 1)
        for hd in range(H):
            g = hd // (H // G)
            score = (k[first: i + 1, g] @ q[i, hd]) * m["scale"]
            for j in range(first, i + 1):
                score[j - first] = score[j - first] + rel[distance_bucket(i - j, rows, far), hd]
            out[i, hd] = torch.softmax(score, dim=0) @ k[first: i + 1, g]
    return out.reshape(T, H * d) @ W[p + ".o"].T


def causal_conv_silu(x: torch.Tensor, w: torch.Tensor, b: torch.Tensor) -> torch.Tensor:
    """Per channel: sum over taps of w[c, k] * x[t - (taps - 1 - k), c] (zeros before the start), plus b, then SiLU."""
    T, taps = x.shape[0], w.shape[1]
    padded = torch.cat([torch.zeros(taps - 1, x.shape[1], dtype=F), x], dim=0)
    out = torch.stack([(padded[t: t + taps] * w.T).sum(dim=0) + b for t in range(T)]) if T else x
    return out * torch.sigmoid(out)


def selective_scan(x, Bm, Cm, dt, a_log, d_skip):
    """x [T, H, P], Bm/Cm [T, H, N] (already spread over the heads), dt [T, H] (after softplus).
    S_t = exp(-exp(a_log) dt_t) S_(t-1) + dt_t B_t x_t^T ;  y_t = S_t^T C_t + d_skip x_t."""
    T, H, P = x.shape
    N = Bm.shape[2]
    S = torch.zeros(H, N, P, dtype=F)
    y = torch.zeros(T, H, P, dtype=F)
    for t in range(T):
        for hd in range(H):
            S[hd] = math.exp(-math.exp(float(a_log[hd])) * float(dt[t, hd])) * S[hd] + dt[t, hd] * torch.outer(Bm[t, hd], x[t, hd])
            y[t, hd] = S[hd].T @ Cm[t, hd] + d_skip[hd] * x[t, hd]
    return y


def mamba2(m: dict, W: Dict[str, torch.Tensor], p: str, h: torch.Tensor, eps: float) -> torch.Tensor:
    T = h.shape[0]
    H, P, N, G = m["heads"], m["vdim"], m["state"], m["groups"]
    inner = H * P
    proj = h @ W[p + ".in"].T
    z = proj[:, :inner]
    xbc = causal_conv_silu(proj[:, inner: 2 * inner + 2 * G * N], W[p + ".conv"], W[p + ".conv.b"])
    dt = torch.nn.functional.softplus(proj[:, 2 * inner + 2 * G * N:] + W[p + ".dt_bias"])
    x = xbc[:, :inner].reshape(T, H, P)
    Bm = xbc[:, inner: inner + G * N].reshape(T, G, N).repeat_interleave(H // G, dim=1)
    Cm = xbc[:, inner + G * N:].reshape(T, G, N).repeat_interleave(H // G, dim=1)
    y = selective_scan(x, Bm, Cm, dt, W[p + ".A_log"], W[p + ".D"]).reshape(T, inner)
    y = y * (z * torch.sigmoid(z))
    parts = m["norm_groups"]
    y = unit_rms(y.reshape(T, parts, inner // parts), eps).reshape(T, inner) * W[p + ".norm"]
    return y @ W[p + ".o"].T


def limited_glu(m: dict, W: Dict[str, torch.Tensor], p: str, h: torch.Tensor) -> torch.Tensor:
    lim = m["limit"]
    g = torch.clamp(h @ W[p + ".gate"].T, max=lim)
    u = torch.clamp(h @ W[p + ".up"].T, min=-lim, max=lim)
    return (g * torch.sigmoid(1.702 * g) * (u + 1.0)) @ W[p + ".down"].T


def forward(cfg: dict, weights: Dict[str, torch.Tensor], tokens: List[int], layers_out: Optional[list] = None) -> torch.Tensor:
    """Logits [T, vocab] of one whole sequence."""
    W = {k: v.to(F) for k, v in weights.items()}
    T, width, eps = len(tokens), cfg["width"], cfg["norm"]["eps"]
    x = W["embed"][torch.tensor(tokens, dtype=torch.long)] + sinusoid(T, width)
    S = cfg.get("streams")
    xs = [x.clone() for _ in range(S or 1)]
    for li, layer in enumerate(cfg["layers"]):
        p = f"l{li}"
        for q, kind in ((1, "mix"), (2, "mlp")):
            if kind == "mlp" and layer.get("mlp") is None:
                continue
            if S is None:
                u = xs[0]
            else:
                u = sum(W[f"{p}.hc{q}.in"][a] * xs[a] for a in range(S))
            hn = offset_norm(u, W[f"{p}.norm{q}"], eps)
            if kind == "mlp":
                y = limited_glu(layer["mlp"], W, p + ".mlp", hn)
            elif layer["type"] == "attention":
                y = windowed_attention(layer["mixer"], W, p + ".mix", hn)
            else:
                y = mamba2(layer["mixer"], W, p + ".mix", hn, eps)
            if S is None:
                xs = [xs[0] + y]
            else:
                mix, out = W[f"{p}.hc{q}.mix"], W[f"{p}.hc{q}.out"]
                xs = [sum(mix[a, b] * xs[a] for a in range(S)) + out[b] * y for b in range(S)]
        if layers_out is not None:
            layers_out.append(sum(xs))
    xf = offset_norm(sum(xs), W["final.norm"], eps)
    return (xf @ W["head"].T) * cfg.get("logit_scale", 1.0)


def greedy(cfg: dict, weights: Dict[str, torch.Tensor], prompt: List[int], n_new: int) -> List[int]:
    """n_new tokens, each the (last) largest logit of the whole sequence so far run anew."""
    toks, out = list(prompt), []
    for _ in range(n_new):
        row = forward(cfg, weights, toks)[-1]
        v = row.shape[0]
        nxt = v - 1 - int(torch.argmax(torch.flip(row, dims=[0])))
        toks.append(nxt)
        out.append(nxt)
    return out


def logit_error(got: torch.Tensor, want: torch.Tensor) -> float:
    """Largest row error: root mean square over the vocabulary of the difference with its mean taken off,
    relative to the root mean square of the wanted logits (mean taken off, over all rows)."""
    d = got.to(F) - want.to(F)
    d = d - d.mean(dim=-1, keepdim=True)
    w = want.to(F) - want.to(F).mean(dim=-1, keepdim=True)
    return float(d.pow(2).mean(dim=-1).sqrt().max() / w.pow(2).mean().sqrt())
