"""The Bomotar design written out plainly in float64, one function per mechanism, token by token where the design
is recurrent.  It shares no code with the product: tensors come as a dict name -> tensor, the configuration as the
dict that config.json holds.  Slow on purpose.

Notation: x is the residual stream [T, W]; h a sublayer's normed input; a mixer named ``parallel`` runs a softmax
attention ("left") and a gated delta-rule recurrence ("right") on the same h and adds the two with fixed scales.
"""
from __future__ import annotations

import math

import torch

F64 = torch.float64


def rms_norm(x, w, eps):
    return x / torch.sqrt((x * x).mean(dim=-1, keepdim=True) + eps) * w


def gelu_tanh(z):
    return 0.5 * z * (1.0 + torch.tanh(math.sqrt(2.0 / math.pi) * (z + 0.044715 * z ** 3)))


def silu(z):
    return z * torch.sigmoid(z)


def embed_tokens(tokens, embed, bigram, mul_prev, mul_cur, buckets):
    """Row of the token plus a row of the bigram table chosen by a hash of (previous, current); a sequence's first
    token reads the table's last row."""
    out = []
    for t, tok in enumerate(tokens):
        row = buckets if t == 0 else (tokens[t - 1] * mul_prev + tok * mul_cur) % buckets
        out.append(embed[tok] + bigram[row])
    return torch.stack(out)


def short_conv(u, w):
    """u [T, C], w [C, taps]: y_t = sum_j w[:, j] * u_(t - taps + 1 + j), zeros before the start."""
    T, C = u.shape
    taps = w.shape[1]
    padded = torch.cat([torch.zeros(taps - 1, C, dtype=u.dtype), u], dim=0)
    y = torch.zeros_like(u)
    for j in range(taps):
        y = y + padded[j: j + T] * w[:, j]
    return y


def yarn_frequencies(dims, base, scaling):
    """(frequencies [dims / 2], magnitude of cos and sin)."""
    i = torch.arange(dims // 2, dtype=F64)
    f = base ** (-2.0 * i / dims)
    if scaling is None:
        return f, 1.0
    factor, original = float(scaling["factor"]), float(scaling["original"])

    def corr(turns):
        return dims * math.log(original / (2.0 * math.pi * turns)) / (2.0 * math.log(base))
    lo = max(math.floor(corr(float(scaling["fast"]))), 0)
    hi = min(math.ceil(corr(float(scaling["slow"]))), dims - 1)
    ramp = torch.clamp((i - lo) / max(hi - lo, 0.001), 0.0, 1.0)
    return f / factor * ramp + f * (1.0 - ramp), 0.1 * math.log(factor) + 1.0


def rotate(x, positions, freqs, mag, dims):
    """x [T, heads, D]: the first ``dims`` elements of every head rotate, element i with element i + dims / 2."""
    half = dims // 2
    ang = positions.to(F64)[:, None] * freqs[None, :]
    c, s = (torch.cos(ang) * mag)[:, None, :], (torch.sin(ang) * mag)[:, None, :]
    u, v = x[..., :half], x[..., half:dims]
    return torch.cat([u * c - v * s, v * c + u * s, x[..., dims:]], dim=-1)


def softmax_attention(q, k, v, scale):
    """q [T, H, D], k [T, G, D], v [T, G, Dv], causal, grouped: query head h reads key/value head h // (H / G)."""
    T, H, _ = q.shape
    G = k.shape[1]
    out = torch.zeros(T, H, v.shape[2], dtype=F64)
    for h in range(H):
        g = h // (H // G)
        s = (q[:, h] @ k[:, g].T) * scale
        s = s.masked_fill(torch.triu(torch.ones(T, T, dtype=torch.bool), diagonal=1), float("-inf"))
        out[:, h] = torch.softmax(s, dim=-1) @ v[:, g]
    return out


def left_mixer(h, W, p, c, positions):
    """Softmax attention with short convolutions behind the projections, partial rotation and an output gate."""
    T = h.shape[0]
    H, G, D, Dv = c["heads"], c["kv_heads"], c["dim"], c["vdim"]
    q = short_conv(h @ W[p + ".q"].T, W[p + ".q.conv"]).reshape(T, H, D)
    k = short_conv(h @ W[p + ".k"].T, W[p + ".k.conv"]).reshape(T, G, D)
    v = short_conv(h @ W[p + ".v"].T, W[p + ".v.conv"]).reshape(T, G, Dv)
    rot = c.get("rot")
    if rot is not None:
        f, mag = yarn_frequencies(rot["dims"], float(rot["base"]), rot.get("scaling"))
        q, k = rotate(q, positions, f, mag, rot["dims"]), rotate(k, positions, f, mag, rot["dims"])
    a = softmax_attention(q, k, v, float(c["scale"])).reshape(T, H * Dv)
    a = a * torch.sigmoid(h @ W[p + ".g"].T)
    return a @ W[p + ".o"].T


def delta_rule(q, k, v, beta, decay):
    """Per head, token by token: S <- decay * S (rows are key channels); u = beta (v - S^T k); S <- S + k u^T;
    o = S^T q.  q, k, decay [T, H, D]; v [T, H, Dv]; beta [T, H]."""
    T, H, D = q.shape
    Dv = v.shape[2]
    S = torch.zeros(H, D, Dv, dtype=F64)
    out = torch.zeros(T, H, Dv, dtype=F64)
    for t in range(T):
        S = decay[t][:, :, None] * S
        u = beta[t][:, None] * (v[t] - torch.einsum("hdv,hd->hv", S, k[t]))
        S = S + k[t][:, :, None] * u[:, None, :]
        out[t] = torch.einsum("hdv,hd->hv", S, q[t])
    return out


def right_mixer(h, W, p, c, eps):
    """Gated delta rule with a decay per head and key channel, a norm per head and a low-rank output gate."""
    T = h.shape[0]
    H, G, D, Dv = c["heads"], c["kv_heads"], c["dim"], c["vdim"]
    q = silu(short_conv(h @ W[p + ".q"].T, W[p + ".q.conv"])).reshape(T, G, D)
    k = silu(short_conv(h @ W[p + ".k"].T, W[p + ".k.conv"])).reshape(T, G, D)
    v = silu(short_conv(h @ W[p + ".v"].T, W[p + ".v.conv"])).reshape(T, H, Dv)
    q = q / torch.sqrt((q * q).sum(-1, keepdim=True) + 1e-6) * D ** -0.5
    k = k / torch.sqrt((k * k).sum(-1, keepdim=True) + 1e-6)
    q, k = q.repeat_interleave(H // G, dim=1), k.repeat_interleave(H // G, dim=1)
    beta = torch.sigmoid(h @ W[p + ".b"].T)
    step = torch.nn.functional.softplus((h @ W[p + ".a1"].T) @ W[p + ".a2"].T + W[p + ".dt_bias"]).reshape(T, H, D)
    decay = torch.exp(-torch.exp(W[p + ".A_log"])[None, :, None] * step)
    o = delta_rule(q, k, v, beta, decay)
    o = o / torch.sqrt((o * o).mean(-1, keepdim=True) + eps) * W[p + ".norm"]
    o = o.reshape(T, H * Dv) * torch.sigmoid((h @ W[p + ".g1"].T) @ W[p + ".g2"].T)
    return o @ W[p + ".o"].T


def parallel_mixer(h, W, p, c, eps, positions):
    return float(c["left_scale"]) * left_mixer(h, W, p + ".left", c["left"], positions) + \
        float(c["right_scale"]) * right_mixer(h, W, p + ".right", c["right"], eps)


def dense_mlp(h, W, p):
    return gelu_tanh(h @ W[p + ".up"].T) @ W[p + ".down"].T


def route(h, W, p, r):
    """(chosen experts [T, top], their weights [T, top]): softmax scores; the choice adds a correction and is
    limited to the best groups; the weights are the scores themselves."""
    E, top = r["experts"], r["top"]
    s = torch.softmax(h @ W[p + ".router"].T, dim=-1)
    choice = s + W[p + ".correction"]
    groups = r.get("groups")
    if groups is not None:
        per = E // groups["count"]
        best = choice.reshape(-1, groups["count"], per).max(dim=-1).values
        keep = torch.topk(best, groups["keep"], dim=-1).indices
        allowed = torch.zeros(h.shape[0], groups["count"], dtype=torch.bool)
        allowed.scatter_(1, keep, True)
        choice = choice.masked_fill(~allowed.repeat_interleave(per, dim=1), float("-inf"))
    idx = torch.topk(choice, top, dim=-1).indices
    return idx, torch.gather(s, 1, idx)


def moe_mlp(h, W, p, mlp):
    idx, wts = route(h, W, p, mlp["router"])
    out = torch.zeros(h.shape[0], W[p + ".e0.down"].shape[0], dtype=F64)
    for t in range(h.shape[0]):
        for e, w in zip(idx[t].tolist(), wts[t]):
            q = f"{p}.e{e}"
            out[t] += w * ((silu(h[t] @ W[q + ".gate"].T) * (h[t] @ W[q + ".up"].T)) @ W[q + ".down"].T)
    return out


def forward(config, weights, tokens, layer_outputs=None):
    """Logits [T, vocab] of one whole sequence; ``layer_outputs`` (a list) receives the residual stream after
    every layer run."""
    W = {k: v.to(F64) for k, v in weights.items()}
    eps = float(config["norm"]["eps"])
    m = float(config.get("residual_mult", 1.0))
    bg = config["embedding"]["bigram"]
    x = embed_tokens(list(tokens), W["embed"], W["bigram"], bg["mul_prev"], bg["mul_cur"], bg["buckets"])
    positions = torch.arange(len(tokens))
    for i, layer in enumerate(config["layers"]):
        p = f"l{layer.get('weights_of', i)}"
        y = parallel_mixer(rms_norm(x, W[p + ".norm1"], eps), W, p + ".mix", layer["mixer"], eps, positions)
        x = x + m * rms_norm(y, W[p + ".norm1b"], eps)
        mlp = layer.get("mlp")
        if mlp is not None:
            h = rms_norm(x, W[p + ".norm2"], eps)
            y = dense_mlp(h, W, p + ".mlp") if mlp.get("kind", "dense") == "dense" else moe_mlp(h, W, p + ".mlp", mlp)
            x = x + m * rms_norm(y, W[p + ".norm2b"], eps)
        if layer_outputs is not None:
            layer_outputs.append(x.clone())
    return rms_norm(x, W["final.norm"], eps) @ W["head"].T


def greedy(config, weights, prompt, n_new):
    """The tokens that greedy decoding appends to ``prompt`` (the whole sequence is run anew for every token)."""
    toks = list(prompt)
    for _ in range(n_new):
        toks.append(int(torch.argmax(forward(config, weights, toks)[-1])))
    return toks[len(prompt):]


def logit_error(got, ref):
    """Largest difference between two sets of logits after taking each row's mean off, relative to the reference's
    spread."""
    g, r = got.to(F64), ref.to(F64)
    d = (g - g.mean(-1, keepdim=True)) - (r - r.mean(-1, keepdim=True))
    return float(d.abs().max() / r.std())
