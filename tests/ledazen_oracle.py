"""Slow, plain oracle of the Ledazen decoder: one function per mechanism, token-by-token
loops, no paging, no batching, no kernels.  It shares no code with the package: the tests
compare the engine (its cache, state slots, scheduler and kernels) against these functions.

Everything runs in one dtype (float64 by default) on whole sequences; ``params`` is a dict
name -> tensor with the checkpoint's tensor names, ``cfg`` the parsed config.json dict.
"""
from __future__ import annotations

import math

import torch


def unit_rms(x, eps):
    """x / sqrt(mean(x^2) + eps) over the last axis."""
    return x / torch.sqrt((x * x).mean(-1, keepdim=True) + eps)


def norm_one_plus(x, w, eps):
    return unit_rms(x, eps) * (1.0 + w)


def norm_plain(x, w, eps):
    return unit_rms(x, eps) * w


def silu(x):
    return x / (1.0 + torch.exp(-x))


def softplus(x):
    return torch.where(x > 30.0, x, torch.log1p(torch.exp(torch.clamp(x, max=30.0))))


def embed_tokens(ids, table, pair_table, buckets, mul_prev, mul_cur):
    """Token embedding plus the hashed previous/current pair embedding (last row of the pair
    table for the first token of a sequence)."""
    rows = []
    for i, t in enumerate(ids):
        r = buckets if i == 0 else (ids[i - 1] * mul_prev + t * mul_cur) % buckets
        rows.append(table[t] + pair_table[r])
    return torch.stack(rows)


def rotate_pairs(x, pos, dims, base):
    """x [T, heads, d]: rotate interleaved pairs (2i, 2i+1), i < dims/2, by pos * base^(-2i/dims);
    channels >= dims pass through."""
    out = x.clone()
    for i in range(dims // 2):
        f = base ** (-2.0 * i / dims)
        a = pos.to(x.dtype) * f
        c, s = torch.cos(a)[:, None], torch.sin(a)[:, None]
        u, v = x[..., 2 * i], x[..., 2 * i + 1]
        out[..., 2 * i] = u * c - v * s
        out[..., 2 * i + 1] = v * c + u * s
    return out


def sink_attention(q, k, v, scale):
    """q [T, H, d], k [T, G, d], v [T, G, dv]; causal; one extra key of score 0 and no value
    in every softmax denominator."""
    T, H, _ = q.shape
    G = k.shape[1]
    rep = H // G
    out = torch.zeros(T, H, v.shape[-1], dtype=q.dtype)
    for h in range(H):
        g = h // rep
        for i in range(T):
            s = (k[: i + 1, g] @ q[i, h]) * scale
            m = torch.clamp(s.max(), min=0.0)
            e = torch.exp(s - m)
            den = e.sum() + math.exp(-float(m))
            out[i, h] = (e[:, None] * v[: i + 1, g]).sum(0) / den
    return out


def causal_conv(x, w):
    """x [T, C], w [C, taps] (last tap = current token), zeros before the start."""
    T, C = x.shape
    taps = w.shape[1]
    out = torch.zeros_like(x)
    for t in range(T):
        for j in range(taps):
            src = t - (taps - 1) + j
            if src >= 0:
                out[t] += w[:, j] * x[src]
    return out


def unit_vector(x):
    return x / torch.sqrt((x * x).sum(-1, keepdim=True) + 1e-6)


def delta_rule(q, k, v, beta, decay):
    """Gated delta rule per head.  q, k [T, H, d] (already normalised / scaled), v [T, H, dv],
    beta [T, H], decay [T, H] (one per head) or [T, H, d] (one per key channel).
    S starts at zero; per token: S = decay * S; u = beta (v - S^T k); S += k u^T; o = S^T q."""
    T, H, d = q.shape
    dv = v.shape[-1]
    out = torch.zeros(T, H, dv, dtype=q.dtype)
    for h in range(H):
        S = torch.zeros(d, dv, dtype=q.dtype)
        for t in range(T):
            g = decay[t, h]
            S = S * (g[:, None] if g.dim() == 1 else g)
            u = beta[t, h] * (v[t, h] - S.t() @ k[t, h])
            S = S + torch.outer(k[t, h], u)
            out[t, h] = S.t() @ q[t, h]
    return out


def delta_mixer(h, p, pre, m, eps, channel_decay):
    """The recurrent mixer.  ``channel_decay`` False: decay logits from one projection ('a'),
    output gate silu(W_g h).  True: decay logits per key channel from the low-rank pair
    a1/a2, output gate sigmoid(W_g2 W_g1 h)."""
    T = h.shape[0]
    H, G, d, dv = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    rep = H // G

    def proj_conv(name):
        return silu(causal_conv(h @ p[pre + name].t(), p[pre + name + ".conv"]))

    q = proj_conv("q").view(T, G, d)
    k = proj_conv("k").view(T, G, d)
    v = proj_conv("v").view(T, H, dv)
    q = unit_vector(q) * d ** -0.5
    k = unit_vector(k)
    q = q.repeat_interleave(rep, 1)
    k = k.repeat_interleave(rep, 1)
    beta = torch.sigmoid(h @ p[pre + "b"].t())
    rate = torch.exp(p[pre + "A_log"])
    if channel_decay:
        a = (h @ p[pre + "a1"].t()) @ p[pre + "a2"].t() + p[pre + "dt_bias"]
        decay = torch.exp(-rate[None, :, None] * softplus(a.view(T, H, d)))
        gate = torch.sigmoid((h @ p[pre + "g1"].t()) @ p[pre + "g2"].t())
    else:
        a = h @ p[pre + "a"].t() + p[pre + "dt_bias"]
        decay = torch.exp(-rate[None, :] * softplus(a))
        gate = silu(h @ p[pre + "g"].t())
    o = delta_rule(q, k, v, beta, decay)
    o = unit_rms(o, eps) * p[pre + "norm"]
    o = o * gate.view(T, H, dv)
    return o.reshape(T, H * dv) @ p[pre + "o"].t()


def softmax_mixer(h, p, pre, m, eps):
    T = h.shape[0]
    H, G, d, dv = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    q = (h @ p[pre + "q"].t()).view(T, H, d)
    k = (h @ p[pre + "k"].t()).view(T, G, d)
    v = (h @ p[pre + "v"].t()).view(T, G, dv)
    q = norm_plain(q, p[pre + "q.norm"], eps)
    k = norm_plain(k, p[pre + "k.norm"], eps)
    pos = torch.arange(T)
    q = rotate_pairs(q, pos, m["rot"]["dims"], m["rot"]["base"])
    k = rotate_pairs(k, pos, m["rot"]["dims"], m["rot"]["base"])
    o = sink_attention(q, k, v, m["scale"])
    return o.reshape(T, H * dv) @ p[pre + "o"].t()


def feed_forward(h, p, pre):
    z = torch.relu(h @ p[pre + "up"].t())
    return (z * z) @ p[pre + "down"].t()


def forward(cfg, params, ids, dtype=torch.float64, return_layers=False):
    """Logits [T, vocab] of one whole sequence (and the residual stream after every layer)."""
    p = {k: (v.to(dtype) if v.is_floating_point() else v) for k, v in params.items()}
    eps = cfg["norm"]["eps"]
    bg = cfg["embedding"]["bigram"]
    x = embed_tokens(list(ids), p["embed"], p["bigram"], bg["buckets"], bg["mul_prev"],
                     bg["mul_cur"])
    layers = []
    for i, L in enumerate(cfg["layers"]):
        pre = f"l{i}."
        h = norm_one_plus(x, p[pre + "norm1"], eps)
        m = L["mixer"]
        if L["type"] == "delta":
            mix = delta_mixer(h, p, pre + "mix.", m, eps, channel_decay=False)
        elif L["type"] == "parallel":
            mix = (m["left_scale"] * softmax_mixer(h, p, pre + "mix.left.", m["left"], eps)
                   + m["right_scale"] * delta_mixer(h, p, pre + "mix.right.", m["right"], eps,
                                                    channel_decay=True))
        else:
            raise ValueError(L["type"])
        ff = feed_forward(h, p, pre + "mlp.") if L.get("mlp") else 0.0
        x = x + (mix + ff)
        layers.append(x)
    logits = norm_one_plus(x, p["final.norm"], eps) @ p["head"].t()
    return (logits, torch.stack(layers)) if return_layers else logits
