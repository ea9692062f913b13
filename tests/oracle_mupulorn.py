"""Plain, slow statement of the Mupulorn decoder, one function per mechanism (the tests' oracle).

Whole sequences only, no cache and no batching; every function takes and returns tensors of one
dtype (the tests use float64). Nothing here is shared with the package's model code.

Notation: ``x`` [T, W] is the residual stream, ``P`` a dict name -> tensor with the checkpoint's
names, ``cfg`` the parsed ``config.json``.
"""
from __future__ import annotations

import math

import torch


def scalar_rms_norm(x, g, eps):
    """x / rms(x) times ONE learned number."""
    return x / torch.sqrt((x * x).mean(-1, keepdim=True) + eps) * g


def weighted_rms_norm(x, w, eps):
    return x / torch.sqrt((x * x).mean(-1, keepdim=True) + eps) * w


def input_conv(h, w):
    """h + causal depthwise convolution of h over time; ``w`` [W, taps], tap ``taps-1`` is the
    current token, zeros before the sequence's start."""
    T, W = h.shape
    taps = w.shape[1]
    out = h.clone()
    for t in range(T):
        for j in range(taps):
            s = t - (taps - 1) + j
            if s >= 0:
                out[t] = out[t] + w[:, j] * h[s]
    return out


def rotate_pairs(v, pos, base, dims):
    """Interleaved rotary embedding on the first ``dims`` entries of the last axis; ``v`` [T, ..., D]."""
    out = v.clone()
    for t in range(v.shape[0]):
        for i in range(dims // 2):
            a = float(pos[t]) * base ** (-2.0 * i / dims)
            c, s = math.cos(a), math.sin(a)
            u, w = v[t, ..., 2 * i].clone(), v[t, ..., 2 * i + 1].clone()
            out[t, ..., 2 * i] = u * c - w * s
            out[t, ..., 2 * i + 1] = w * c + u * s
    return out


def sink_softmax_attention(q, k, v, sink, scale):
    """Causal attention of one head with a sink in the softmax denominator. q, k [T, Dk], v [T, Dv]."""
    T = q.shape[0]
    out = torch.zeros(T, v.shape[1], dtype=q.dtype)
    for i in range(T):
        s = (k[:i + 1] @ q[i]) * scale
        m = torch.maximum(s.max(), sink)
        e = torch.exp(s - m)
        den = e.sum() + torch.exp(sink - m)
        out[i] = (e / den) @ v[:i + 1]
    return out


def latent_qkv(h, P, pre, m, eps):
    """Per-head queries and keys [H, T, dim + rot_dim] (rotated parts last) and values [H, T, vdim]."""
    T = h.shape[0]
    H, D, R, Dv, C = m["heads"], m["dim"], m["rot_dim"], m["vdim"], m["kv_rank"]
    pos = torch.arange(T)
    cq = weighted_rms_norm(h @ P[pre + "dq"].T, P[pre + "dq.norm"], eps)
    q = (cq @ P[pre + "uq"].T).view(T, H, D + R)
    dkv = h @ P[pre + "dkv"].T
    c = weighted_rms_norm(dkv[:, :C], P[pre + "dkv.norm"], eps)
    k_rot = rotate_pairs(dkv[:, C:], pos, m["rot"]["base"], m["rot"]["dims"])
    q_rot = rotate_pairs(q[:, :, D:], pos, m["rot"]["base"], m["rot"]["dims"])
    kn = (c @ P[pre + "uk"].T).view(T, H, D)
    vv = (c @ P[pre + "uv"].T).view(T, H, Dv)
    qs = torch.stack([torch.cat([q[:, hh, :D], q_rot[:, hh]], -1) for hh in range(H)])
    ks = torch.stack([torch.cat([kn[:, hh], k_rot], -1) for hh in range(H)])
    return qs, ks, vv.transpose(0, 1)


def latent_attention(h, P, pre, m, eps):
    """The mixer: low-rank queries, one shared latent for keys and values, a rotated key part
    shared by all heads, a per-head sink, an output gate."""
    qs, ks, vs = latent_qkv(h, P, pre, m, eps)
    heads = [sink_softmax_attention(qs[hh], ks[hh], vs[hh], P[pre + "sink"][hh], m["scale"])
             for hh in range(m["heads"])]
    o = torch.cat(heads, -1) * torch.sigmoid(h @ P[pre + "g"].T)
    return o @ P[pre + "o"].T


def poly_norm(z, coef, eps):
    def n(u):
        return u / torch.sqrt((u * u).mean(-1, keepdim=True) + eps)
    return coef[0] * n(z) + coef[1] * n(z * z) + coef[2] * n(z * z * z) + coef[3]


def dense_ff(h, P, pre, eps):
    return poly_norm(h @ P[pre + "up"].T, P[pre + "act"], eps) @ P[pre + "down"].T


def source_layer(cfg, i):
    while "weights_of" in cfg["layers"][i]:
        i = cfg["layers"][i]["weights_of"]
    return i


def layer(x, P, cfg, i):
    eps = cfg["norm"]["eps"]
    L = cfg["layers"][i]
    p = "l%d." % source_layer(cfg, i)
    h = input_conv(scalar_rms_norm(x, P[p + "norm1"], eps), P[p + "canon1"])
    x = x + scalar_rms_norm(latent_attention(h, P, p + "mix.", L["mixer"], eps), P[p + "norm1b"], eps)
    if L.get("mlp") is not None:
        h = input_conv(scalar_rms_norm(x, P[p + "norm2"], eps), P[p + "canon2"])
        x = x + scalar_rms_norm(dense_ff(h, P, p + "mlp.", eps), P[p + "norm2b"], eps)
    return x


def forward(tokens, P, cfg, return_layers=False):
    """Logits [T, vocab] of one whole sequence (and the residual stream after every layer)."""
    x = P["embed"][torch.as_tensor(tokens)]
    per_layer = []
    for i in range(len(cfg["layers"])):
        x = layer(x, P, cfg, i)
        per_layer.append(x)
    y = scalar_rms_norm(x, P["final.norm"], cfg["norm"]["eps"]) @ P["head"].T * cfg["logit_scale"]
    cap = cfg["logit_softcap"]
    y = cap * torch.tanh(y / cap)
    return (y, torch.stack(per_layer)) if return_layers else y
