"""Sokipel in plain float64 torch, one function per mechanism, written from the design's equations for the tests to compare the
engine against.  Nothing here is shared with the product path: every sequence is run whole, token by token where the design
is recurrent, with dense masks where it attends.

    W: checkpoint-named tensors (float64), cfg: the config.json dict, tokens: one sequence.
"""
import math

import torch

D = torch.float64


def unit(x, eps):
    """x over its root mean square along the last axis (eps inside the root)."""
    return x / torch.sqrt((x * x).mean(-1, keepdim=True) + eps)


def silu(x):
    return x * torch.sigmoid(x)


def time_conv(x, w):
    """Causal convolution over time per channel: y_t = sum_j w[:, j] x_(t - J + 1 + j), J taps, x_t = 0 for t < 0.  x [T, C], w [C, J]."""
    T, J = x.shape[0], w.shape[1]
    y = torch.zeros_like(x)
    for t in range(T):
        for j in range(J):
            s = t - J + 1 + j
            if s >= 0:
                y[t] += w[:, j] * x[s]
    return y


def frequencies(rot):
    """Rotation frequencies of the dims/2 pairs.  scaling {factor}: all divided by factor; scaling {factor, low, high, original}: by
    wavelength - short ones stay, long ones are divided, those between blend."""
    dims, base = rot["dims"], rot["base"]
    out = []
    sc = rot.get("scaling")
    for i in range(dims // 2):
        f = base ** (-2.0 * i / dims)
        if sc and "original" in sc:
            wl = 2 * math.pi / f
            if wl > sc["original"] / sc["low"]:
                f = f / sc["factor"]
            elif wl >= sc["original"] / sc["high"]:
                mix = (sc["original"] / wl - sc["low"]) / (sc["high"] - sc["low"])
                f = (1 - mix) * f / sc["factor"] + mix * f
        elif sc:
            f = f / sc["factor"]
        out.append(f)
    return torch.tensor(out, dtype=D)


def rotate(x, rot, interleaved):
    """x [T, heads, size]: the first rot.dims entries of every head are turned pair by pair by position * frequency; pairs are
    (2i, 2i+1) when interleaved, (i, i + dims/2) otherwise."""
    if not rot:
        return x
    dims = rot["dims"]
    ang = torch.arange(x.shape[0], dtype=D)[:, None, None] * frequencies(rot)
    c, s = torch.cos(ang), torch.sin(ang)
    out = x.clone()
    if interleaved:
        a, b = x[..., 0:dims:2], x[..., 1:dims:2]
        out[..., 0:dims:2], out[..., 1:dims:2] = a * c - b * s, b * c + a * s
    else:
        a, b = x[..., :dims // 2], x[..., dims // 2:dims]
        out[..., :dims // 2], out[..., dims // 2:dims] = a * c - b * s, b * c + a * s
    return out


def sink_softmax_attention(q, k, v, scale, sink, chunk):
    """q [T, H, d], k [T, G, d], v [T, G, dv]; sink [H]: a logit that only the denominator sees; chunk > 0: keys of the query's own
    block of `chunk` positions only.  Returns [T, H, dv]."""
    T, H = q.shape[0], q.shape[1]
    G = k.shape[1]
    out = torch.zeros(T, H, v.shape[2], dtype=D)
    for h in range(H):
        g = h // (H // G)
        for i in range(T):
            first = (i // chunk) * chunk if chunk else 0
            s = (k[first:i + 1, g] @ q[i, h]) * scale
            top = max(float(s.max()), float(sink[h]))
            e = torch.exp(s - top)
            out[i, h] = (e[:, None] * v[first:i + 1, g]).sum(0) / (e.sum() + math.exp(float(sink[h]) - top))
    return out


def attention(W, p, m, h, eps, beside):
    """`beside`: the variant of the parallel mixer (biases, a norm per head, halves layout, positions divided, a gate per head, every
    earlier token visible); else the chunked one (a norm over the whole projection, interleaved layout)."""
    T, H, d = h.shape[0], m["heads"], m["dim"]
    G, dv = m.get("kv_heads", H), m.get("vdim", d)
    q, k, v = h @ W[p + "q"].T, h @ W[p + "k"].T, h @ W[p + "v"].T
    if beside:
        q, k, v = q + W[p + "q.b"], k + W[p + "k.b"], v + W[p + "v.b"]
        q = unit(q.view(T, H, d), eps) * W[p + "q.norm"]
        k = unit(k.view(T, G, d), eps) * W[p + "k.norm"]
    else:
        q = (unit(q, eps) * W[p + "q.norm"]).view(T, H, d)
        k = (unit(k, eps) * W[p + "k.norm"]).view(T, G, d)
    q, k = rotate(q, m.get("rot"), not beside), rotate(k, m.get("rot"), not beside)
    chunk = (m.get("mask") or {}).get("size", 0)
    o = sink_softmax_attention(q, k, v.view(T, G, dv), m.get("scale", d ** -0.5), W[p + "sink"], chunk)
    if beside:
        o = o * torch.sigmoid(h @ W[p + "g"].T)[:, :, None]
    return o.reshape(T, H * dv) @ W[p + "o"].T


def gated_delta(W, p, m, h, eps):
    T, H, d = h.shape[0], m["heads"], m["dim"]
    G, dv = m.get("kv_heads", H), m.get("vdim", d)
    q = silu(time_conv(h @ W[p + "q"].T, W[p + "q.conv"])).view(T, G, d)
    k = silu(time_conv(h @ W[p + "k"].T, W[p + "k.conv"])).view(T, G, d)
    v = silu(time_conv(h @ W[p + "v"].T, W[p + "v.conv"])).view(T, H, dv)
    q = q / torch.sqrt((q * q).sum(-1, keepdim=True) + 1e-6) / math.sqrt(d)
    k = k / torch.sqrt((k * k).sum(-1, keepdim=True) + 1e-6)
    beta = torch.sigmoid(h @ W[p + "b"].T)
    decay = torch.exp(-torch.exp(W[p + "A_log"]) * torch.nn.functional.softplus(h @ W[p + "a"].T + W[p + "dt_bias"]))
    o = torch.zeros(T, H, dv, dtype=D)
    for n in range(H):
        g = n // (H // G)
        S = torch.zeros(d, dv, dtype=D)
        for t in range(T):
            S = decay[t, n] * S
            S = S + torch.outer(k[t, g], beta[t, n] * (v[t, n] - S.T @ k[t, g]))
            o[t, n] = S.T @ q[t, g]
    o = unit(o, eps) * W[p + "norm"]
    return (o.reshape(T, H * dv) * silu(h @ W[p + "g"].T)) @ W[p + "o"].T


def experts(W, p, mlp, x):
    """Sigmoid scores, the `top` best, each expert fed with score * x; the capped gated unit."""
    top, cap = mlp["router"]["top"], mlp["expert"]["limit"]
    score = torch.sigmoid(x @ W[p + "router"].T)
    y = torch.zeros_like(x)
    for t in range(x.shape[0]):
        for e in torch.topk(score[t], top).indices.tolist():
            inp = score[t, e] * x[t]
            a = torch.clamp(W[f"{p}e{e}.gate"] @ inp, max=cap)
            b = torch.clamp(W[f"{p}e{e}.up"] @ inp, min=-cap, max=cap)
            y[t] += W[f"{p}e{e}.down"] @ (a * torch.sigmoid(1.702 * a) * (b + 1.0))
    return y


def forward(W, cfg, tokens, collect=None):
    """fp64 logits [T, vocab]; `collect` (a list) receives the stream after every layer."""
    eps, mult = cfg["norm"]["eps"], cfg.get("residual_mult", 1.0)
    x = W["embed"][torch.tensor(tokens)] * cfg.get("embedding", {}).get("scale", 1.0)
    for i, L in enumerate(cfg["layers"]):
        p, m = f"l{i}.", L["mixer"]
        h = x + time_conv(x, W[p + "canon1"]) if cfg.get("canon") else x
        if L["type"] == "attention":
            y = attention(W, p + "mix.", m, h, eps, False)
        elif L["type"] == "delta":
            y = gated_delta(W, p + "mix.", m, h, eps)
        else:
            y = m["left_scale"] * attention(W, p + "mix.left.", m["left"], h, eps, True) + m["right_scale"] * gated_delta(W, p + "mix.right.", m["right"], h, eps)
        x = x + mult * W[p + "norm1"] * unit(y, eps)
        if L.get("mlp"):
            x = x + mult * W[p + "norm2"] * unit(experts(W, p + "mlp.", L["mlp"], x), eps)
        if collect is not None:
            collect.append(x.clone())
    z = (unit(x, eps) * W["final.norm"]) @ W["head"].T
    cap = cfg.get("logit_softcap")
    return cap * torch.tanh(z / cap) if cap else z
