"""Slow float64 oracle of the Soselix decoder: one function per mechanism, token-by-token
loops, dense attention with per-head keys and values (no absorption, no paging, no batching).
Shares no code with the package; tests compare the engine and the kernels against it.
"""
import math

import torch

F64 = torch.float64


def silu(z):
    return z * torch.sigmoid(z)


def softplus(z):
    return torch.log1p(torch.exp(-z.abs())) + z.clamp_min(0)


def rms(x, eps):
    return x / torch.sqrt((x * x).mean(-1, keepdim=True) + eps)


def norm_scalar(x, g, eps):
    """RMS norm whose weight is one number."""
    return rms(x, eps) * g


def norm_plain(x, w, eps):
    return rms(x, eps) * w


def rotate_half(x, pos, dims, base):
    """x [T, ..., r]: channel i < dims / 2 pairs with channel i + dims / 2; channels >= dims
    pass unchanged.  pos: float64 [T]."""
    half = dims // 2
    freq = torch.tensor([base ** (-2.0 * i / dims) for i in range(half)], dtype=F64)
    ang = pos.to(F64)[:, None] * freq[None]
    shape = [x.shape[0]] + [1] * (x.dim() - 2) + [half]
    c, s = torch.cos(ang).view(shape), torch.sin(ang).view(shape)
    u, v = x[..., :half], x[..., half:dims]
    return torch.cat([u * c - v * s, v * c + u * s, x[..., dims:]], -1)


def sink_softmax_attention(q, k, v, scale, sink):
    """q [T, H, d], k [T, H, d], v [T, H, dv] of one sequence, causal; ``sink`` [H] adds
    exp(sink) to every denominator (None: no sink)."""
    T, H, _ = q.shape
    out = torch.zeros(T, H, v.shape[-1], dtype=F64)
    for t in range(T):
        for h in range(H):
            sc = (k[:t + 1, h] @ q[t, h]) * scale
            m = sc.max() if sink is None else torch.maximum(sc.max(), sink[h])
            e = torch.exp(sc - m)
            den = e.sum() + (0.0 if sink is None else torch.exp(sink[h] - m))
            out[t, h] = (e / den) @ v[:t + 1, h]
    return out


def latent_attention(h, p, mc, eps, shared):
    """One layer's mixer on the whole sequence h [T, W].  ``shared``: dict layer index ->
    (latent, rotated key) of the layers that own a cache; ``mc`` the layer's mixer dict."""
    T = h.shape[0]
    H, d, r, dv, rank = mc["heads"], mc["dim"], mc["rot_dim"], mc["vdim"], mc["kv_rank"]
    rot = mc.get("rot") or {"dims": r, "base": 10000.0}
    pos = torch.arange(T, dtype=F64)
    cq = norm_plain(h @ p["dq"].T, p["dq.norm"], eps)
    q = (cq @ p["uq"].T).view(T, H, d + r)
    q_plain, q_rot = q[..., :d], rotate_half(q[..., d:], pos, rot["dims"], rot["base"])
    if "kv_from" in mc:
        lat, k_rot = shared[mc["kv_from"]]
    else:
        down = h @ p["dkv"].T
        lat = norm_plain(down[:, :rank], p["dkv.norm"], eps)
        k_rot = rotate_half(down[:, rank:], pos, rot["dims"], rot["base"])
        shared[mc["index"]] = (lat, k_rot)
    k_plain = (lat @ p["uk"].T).view(T, H, d)
    v = (lat @ p["uv"].T).view(T, H, dv)
    qq = torch.cat([q_plain, q_rot], -1)
    kk = torch.cat([k_plain, k_rot[:, None, :].expand(T, H, r)], -1)
    o = sink_softmax_attention(qq, kk, v, mc["scale"], p["sink"])
    o = o * torch.sigmoid(h @ p["g"].T)[:, :, None]
    return o.reshape(T, H * dv) @ p["o"].T


def forget_gate_recurrence(q, f, v):
    """q, f [T, H, d], v [T, H, dv]: S = diag(f) S + (1 - f) v^T, o = S^T q."""
    T, H, d = q.shape
    S = torch.zeros(H, d, v.shape[-1], dtype=F64)
    out = torch.zeros(T, H, v.shape[-1], dtype=F64)
    for t in range(T):
        for h in range(H):
            S[h] = f[t, h][:, None] * S[h] + torch.outer(1.0 - f[t, h], v[t, h])
            out[t, h] = S[h].T @ q[t, h]
    return out


def hgrn2(h, p, mc, eps):
    T = h.shape[0]
    H, d, dv = mc["heads"], mc["dim"], mc["vdim"]
    q = silu(h @ p["q"].T).view(T, H, d)
    v = (h @ p["v"].T).view(T, H, dv)
    lo = p["lower"]
    f = (lo + (1.0 - lo) * torch.sigmoid(h @ p["f"].T + p["f.b"])).view(T, H, d)
    o = norm_plain(forget_gate_recurrence(q, f, v), p["norm"], eps)
    return o.reshape(T, H * dv) @ p["o"].T


def causal_conv(x, w, b=None):
    """x [T, C], w [C, taps] (last column = current token), zeros before the start."""
    T, C = x.shape
    taps = w.shape[1]
    out = torch.zeros(T, C, dtype=F64)
    for t in range(T):
        for j in range(taps):
            src = t - (taps - 1) + j
            if src >= 0:
                out[t] += w[:, j] * x[src]
    return out if b is None else out + b


def state_space_recurrence(x, B, C, dt, a_log, skip):
    """x [T, H, dv], B / C [T, H, N] (already expanded to heads), dt [T, H] (after softplus)."""
    T, H, dv = x.shape
    S = torch.zeros(H, B.shape[-1], dv, dtype=F64)
    y = torch.zeros(T, H, dv, dtype=F64)
    for t in range(T):
        for h in range(H):
            S[h] = math.exp(-math.exp(float(a_log[h])) * float(dt[t, h])) * S[h] + \
                float(dt[t, h]) * torch.outer(B[t, h], x[t, h])
            y[t, h] = S[h].T @ C[t, h] + skip[h] * x[t, h]
    return y


def mamba2(h, p, mc, eps):
    T = h.shape[0]
    H, dv, N, G = mc["heads"], mc["vdim"], mc["state"], mc.get("groups", 1)
    ng = mc.get("norm_groups", 1)
    inner, gn = H * dv, G * N
    proj = h @ p["in"].T
    z, xbc, dt = proj[:, :inner], proj[:, inner:2 * inner + 2 * gn], proj[:, 2 * inner + 2 * gn:]
    xbc = silu(causal_conv(xbc, p["conv"], p["conv.b"]))
    x = xbc[:, :inner].view(T, H, dv)
    per = H // G
    B = xbc[:, inner:inner + gn].view(T, G, N).repeat_interleave(per, 1)
    C = xbc[:, inner + gn:].view(T, G, N).repeat_interleave(per, 1)
    y = state_space_recurrence(x, B, C, softplus(dt + p["dt_bias"]), p["A_log"], p["D"])
    y = y.reshape(T, inner) * silu(z)
    y = rms(y.view(T, ng, inner // ng), eps).reshape(T, inner) * p["norm"]
    return y @ p["o"].T


def xielu(z, a):
    """a = the layer's two numbers."""
    ap, aq = softplus(a[0]), softplus(a[1])
    neg = (0.5 + aq) * (torch.exp(z.clamp_max(0)) - 1.0 - z) + 0.5 * z
    return torch.where(z > 0, ap * z * z + 0.5 * z, neg)


def feed_forward(h, p):
    return xielu(h @ p["up"].T + p["up.b"], p["act"]) @ p["down"].T + p["down.b"]


def sub(params, prefix):
    return {k[len(prefix):]: v.to(F64) for k, v in params.items() if k.startswith(prefix)}


def forward(cfg, params, tokens, return_layers=False):
    """Logits [T, vocab] of one sequence (and the residual stream after every layer)."""
    eps, mult = cfg["norm"]["eps"], cfg.get("residual_mult", 1.0)
    x = params["embed"].to(F64)[torch.tensor(tokens)] * cfg["embedding"]["scale"]
    shared, layers = {}, []
    for i, L in enumerate(cfg["layers"]):
        h = norm_scalar(x, params[f"l{i}.norm1"].to(F64), eps)
        p = sub(params, f"l{i}.mix.")
        mc = dict(L["mixer"], index=i)
        if L["type"] == "latent_attention":
            y = latent_attention(h, p, mc, eps, shared)
        elif L["type"] == "hgrn2":
            y = hgrn2(h, p, mc, eps)
        else:
            y = mamba2(h, p, mc, eps)
        x = x + mult * y
        if L.get("mlp"):
            x = x + mult * feed_forward(norm_scalar(x, params[f"l{i}.norm2"].to(F64), eps),
                                        sub(params, f"l{i}.mlp."))
        layers.append(x.clone())
    logits = norm_scalar(x, params["final.norm"].to(F64), eps) @ params["head"].to(F64).T
    return (logits, layers) if return_layers else logits
