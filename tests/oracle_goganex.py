"""A plain, slow float64 statement of the Goganex decoder, one function per mechanism, written
from the design's equations and sharing no code with the package. ``P`` maps checkpoint tensor
names to float64 tensors, ``cfg`` is the checkpoint's config.json as a dict.

Notation: n tokens, width W; a head's query / key size D, value size E; H query heads over G
key / value heads, query head i reading key / value head i // (H / G).
"""
import math

import torch


def unit_rms(x, eps):
    """x divided by its root mean square over the last axis, eps inside the root."""
    return x / torch.sqrt((x * x).mean(-1, keepdim=True) + eps)


def rms_norm(x, w, eps):
    return unit_rms(x, eps) * w


def token_shift(h, mu):
    """Row t becomes h_t + (h_(t-1) - h_t) * mu, with h_(-1) = 0; the rows on the right-hand side
    are the ones that came in."""
    before = torch.cat([torch.zeros_like(h[:1]), h[:-1]])
    return h + (before - h) * mu


def frequencies(rot):
    """base^(-2i / dims), i < dims / 2, each rescaled by its wavelength L = 2 pi / f when
    ``scaling`` = (factor, low, high, original) is given: unchanged for L < original / high,
    f / factor for L > original / low, and in between a blend with weight
    s = (original / L - low) / (high - low) on the unchanged one."""
    n = rot["dims"] // 2
    out = []
    sc = rot.get("scaling")
    for i in range(n):
        f = rot["base"] ** (-2.0 * i / rot["dims"])
        if sc:
            L = 2 * math.pi / f
            if L > sc["original"] / sc["low"]:
                f = f / sc["factor"]
            elif L >= sc["original"] / sc["high"]:
                s = (sc["original"] / L - sc["low"]) / (sc["high"] - sc["low"])
                f = (1 - s) * f / sc["factor"] + s * f
        out.append(f)
    return torch.tensor(out, dtype=torch.float64)


def rotate_pairs(x, positions, freqs):
    """x [n, heads, D]: entries (2i, 2i + 1) = (a, b) of the token at position p become
    (a cos t - b sin t, b cos t + a sin t), t = p f_i; entries from 2 len(freqs) on stay."""
    out = x.clone()
    for i, f in enumerate(freqs.tolist()):
        t = positions.double() * f
        c, s = torch.cos(t)[:, None], torch.sin(t)[:, None]
        a, b = x[..., 2 * i], x[..., 2 * i + 1]
        out[..., 2 * i] = a * c - b * s
        out[..., 2 * i + 1] = b * c + a * s
    return out


def causal_attention(q, k, v, scale, temp=None, sink=0.0):
    """q [n, H, D], k [n, G, D], v [n, G, E] of ONE sequence from position 0. Token t sees tokens
    0 .. t; weights exp(s_j) / (sink + sum_j exp(s_j)) with s_j = q_t . k_j * scale * temp[head]
    (``sink`` = 1 is a key of score 0 that has no value). Returns [n, H, E]."""
    n, H, _ = q.shape
    G = k.shape[1]
    out = torch.zeros(n, H, v.shape[2], dtype=torch.float64)
    for i in range(H):
        g = i // (H // G)
        for t in range(n):
            s = (k[:t + 1, g] @ q[t, i]) * scale * (float(temp[i]) if temp is not None else 1.0)
            e = torch.exp(s)
            out[t, i] = (e / (sink + e.sum())) @ v[:t + 1, g]
    return out


def attention_mixer(h, P, p, m, eps, kind):
    """``kind`` 'attention': rotary pairs, then unit-RMS queries and keys, a temperature per head,
    a sink of score 0. ``kind`` 'left' (of a parallel layer): no positions, the values are the
    projected keys before their norm, an ordinary softmax."""
    n = h.shape[0]
    H, G, D, E = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    q = (h @ P[p + "q"].T).reshape(n, H, D)
    k = (h @ P[p + "k"].T).reshape(n, G, D)
    if kind == "attention":
        v = (h @ P[p + "v"].T).reshape(n, G, E)
        f = frequencies(m["rot"])
        pos = torch.arange(n)
        q, k = rotate_pairs(q, pos, f), rotate_pairs(k, pos, f)
        temp, sink = P[p + "temp"], 1.0
    else:
        v, temp, sink = k.clone(), None, 0.0
    o = causal_attention(unit_rms(q, eps), unit_rms(k, eps), v, m["scale"], temp, sink)
    return o.reshape(n, H * E) @ P[p + "o"].T


def min_gru(h, P, p):
    """z = sigmoid(Wz h + bz); u = Wx h + bx; candidate c = u + 1/2 for u >= 0, sigmoid(u) below;
    S_t = (1 - z_t) S_(t-1) + z_t c_t from S = 0; output Wo (S_t * silu(Wg h))."""
    z = torch.sigmoid(h @ P[p + "z"].T + P[p + "z.b"])
    u = h @ P[p + "x"].T + P[p + "x.b"]
    c = torch.where(u >= 0, u + 0.5, torch.sigmoid(u))
    g = h @ P[p + "g"].T
    S = torch.zeros(z.shape[1], dtype=torch.float64)
    rows = []
    for t in range(h.shape[0]):
        S = (1 - z[t]) * S + z[t] * c[t]
        rows.append(S * g[t] * torch.sigmoid(g[t]))
    return torch.stack(rows) @ P[p + "o"].T


def feed_forward(h, P, p, limit):
    g = torch.clamp(h @ P[p + "gate"].T, max=limit)
    u = torch.clamp(h @ P[p + "up"].T, -limit, limit)
    return (g * torch.sigmoid(1.702 * g) * (u + 1)) @ P[p + "down"].T


def layer_runs(cfg):
    """Checkpoint layer index of every layer run, in order: layers start .. stop - 1 of ``loop``
    are run ``times`` times in a row."""
    n = len(cfg["layers"])
    lp = cfg.get("loop")
    if not lp:
        return list(range(n))
    return list(range(lp["start"])) + list(range(lp["start"], lp["stop"])) * lp["times"] + list(range(lp["stop"], n))


def forward(tokens, P, cfg, return_layers=False):
    """Logits [n, vocab] of one sequence from position 0 (and the residual stream after every run)."""
    eps = cfg["norm"]["eps"]
    x = P["embed"][torch.tensor(tokens)] * cfg["embedding"]["scale"]
    kept = []
    for i in layer_runs(cfg):
        e, p = cfg["layers"][i], f"l{i}."
        h = token_shift(rms_norm(x, P[p + "norm1"], eps), P[p + "shift"])
        if e["type"] == "attention":
            x = x + attention_mixer(h, P, p + "mix.", e["mixer"], eps, "attention")
        else:
            a = attention_mixer(h, P, p + "mix.left.", e["mixer"]["left"], eps, "left")
            b = min_gru(h, P, p + "mix.right.")
            x = x + 0.5 * (rms_norm(a, P[p + "mix.left.out"], eps) + rms_norm(b, P[p + "mix.right.out"], eps))
        if e.get("mlp"):
            x = x + feed_forward(rms_norm(x, P[p + "norm2"], eps), P, p + "mlp.", e["mlp"]["limit"])
        kept.append(x.clone())
    logits = rms_norm(x, P["final.norm"], eps) @ P["head"].T
    return (logits, kept) if return_layers else logits
