"""Lakatar in plain float64 torch, one function per mechanism, written from the design's equations for the tests to compare the
engine against.  Nothing here is shared with the product path: every sequence is run whole, token by token where the design
is recurrent, with dense causal masks where it attends.

    W: checkpoint-named tensors (float64), cfg: the config.json dict, tokens: one sequence.
"""
import math

import torch

D = torch.float64


def unit(x, eps):
    """x over its root mean square (eps inside the root)."""
    return x / torch.sqrt((x * x).mean(-1, keepdim=True) + eps)


def silu(x):
    return x * torch.sigmoid(x)


def post_norm(x, branch, alpha, scale, w, eps):
    """The norm after the sum: unit(alpha x + scale * branch) (1 + w)."""
    return unit(alpha * x + scale * branch, eps) * (1.0 + w)


def frequencies(rot):
    """Rotation frequencies of the dims/2 pairs and the factor on cos / sin (YaRN when `scaling` is given)."""
    dims, base = rot["dims"], rot["base"]
    f = torch.tensor([base ** (-2.0 * i / dims) for i in range(dims // 2)], dtype=D)
    sc = rot.get("scaling")
    if not sc:
        return f, 1.0
    where = lambda turns: dims * math.log(sc["original"] / (2 * math.pi * turns)) / (2 * math.log(base))
    lo, hi = max(math.floor(where(sc["fast"])), 0), min(math.ceil(where(sc["slow"])), dims - 1)
    ramp = torch.tensor([min(max((i - lo) / max(hi - lo, 0.001), 0.0), 1.0) for i in range(dims // 2)], dtype=D)
    return f / sc["factor"] * ramp + f * (1 - ramp), 0.1 * math.log(sc["factor"]) + 1.0


def rotate(x, positions, rot, interleaved):
    """x [T, heads, size]: the first rot.dims entries of every head are turned pair by pair by position * frequency; pairs are
    (2i, 2i+1) when interleaved, (i, i + dims/2) otherwise."""
    dims = rot["dims"]
    f, mag = frequencies(rot)
    ang = positions.to(D)[:, None, None] * f
    c, s = torch.cos(ang) * mag, torch.sin(ang) * mag
    out = x.clone()
    if interleaved:
        a, b = x[..., 0:dims:2], x[..., 1:dims:2]
        out[..., 0:dims:2], out[..., 1:dims:2] = a * c - b * s, b * c + a * s
    else:
        a, b = x[..., :dims // 2], x[..., dims // 2:dims]
        out[..., :dims // 2], out[..., dims // 2:dims] = a * c - b * s, b * c + a * s
    return out


def retention(W, p, m, h, eps):
    T, H, dk, dv = h.shape[0], m["heads"], m["dim"], m.get("vdim", m["dim"])
    pos = torch.arange(T)
    q, k, v = (h @ W[p + n].T for n in "qkv")
    q, k, v = q.view(T, H, dk), k.view(T, H, dk), v.view(T, H, dv)
    if m.get("rot"):
        q, k = rotate(q, pos, m["rot"], False), rotate(k, pos, m["rot"], False)
    k = k / math.sqrt(dk)
    out = torch.zeros(T, H, dv, dtype=D)
    for i in range(H):
        S = torch.zeros(dk, dv, dtype=D)
        for t in range(T):
            S = m["decay"][i] * S + torch.outer(k[t, i], v[t, i])
            out[t, i] = S.T @ q[t, i]
    out = unit(out, eps).reshape(T, H * dv) * silu(h @ W[p + "g"].T)
    return out @ W[p + "o"].T


def wkv(W, p, m, h, eps):
    T, H, dk = h.shape[0], m["heads"], m["dim"]
    before = torch.cat([torch.zeros(1, h.shape[1], dtype=D), h[:-1]])
    blend = {n: h + (before - h) * W[p + "mu." + n] for n in "rkvgw"}
    r, k, v = ((blend[n] @ W[p + n].T).view(T, H, dk) for n in "rkv")
    gate = silu(blend["g"] @ W[p + "g"].T)
    decay = torch.exp(-torch.exp(torch.tanh(blend["w"] @ W[p + "w1"].T) @ W[p + "w2"].T + W[p + "w0"])).view(T, H, dk)
    out = torch.zeros(T, H, dk, dtype=D)
    for i in range(H):
        S = torch.zeros(dk, dk, dtype=D)
        for t in range(T):
            kv = torch.outer(k[t, i], v[t, i])
            out[t, i] = (S + W[p + "u"][i][:, None] * kv).T @ r[t, i]
            S = decay[t, i][:, None] * S + kv
    out = unit(out, eps).reshape(T, H * dk) * W[p + "norm"] * gate
    return out @ W[p + "o"].T


def latent_attention(W, p, m, h, eps, latents, index):
    T, H, dn, dr, dv, R = h.shape[0], m["heads"], m["dim"], m["rot_dim"], m.get("vdim", m["dim"]), m["kv_rank"]
    pos = torch.arange(T)
    cq = unit(h @ W[p + "dq"].T, eps) * W[p + "dq.norm"]
    q = (cq @ W[p + "uq"].T).view(T, H, dn + dr)
    q_plain, q_rot = q[..., :dn], (rotate(q[..., dn:], pos, m["rot"], True) if dr else q[..., dn:])
    if m.get("kv_from") is not None:
        c, k_rot = latents[m["kv_from"]]
    else:
        down = h @ W[p + "dkv"].T
        c = unit(down[:, :R], eps) * W[p + "dkv.norm"]
        k_rot = rotate(down[:, None, R:], pos, m["rot"], True)[:, 0] if dr else down[:, R:]
        latents[index] = (c, k_rot)
    k_plain, v = (c @ W[p + "uk"].T).view(T, H, dn), (c @ W[p + "uv"].T).view(T, H, dv)
    gate = torch.sigmoid(h @ W[p + "g"].T)
    out = torch.zeros(T, H, dv, dtype=D)
    for i in range(H):
        score = (q_plain[:, i] @ k_plain[:, i].T + q_rot[:, i] @ k_rot.T) * m["scale"]
        score = score.masked_fill(torch.ones(T, T, dtype=torch.bool).triu(1), -math.inf)
        out[:, i] = torch.softmax(score, -1) @ v[:, i] * gate[:, i:i + 1]
    return out.reshape(T, H * dv) @ W[p + "o"].T


def gated_ff(W, p, h):
    return (silu(h @ W[p + "gate"].T) * (h @ W[p + "up"].T)) @ W[p + "down"].T


def route(W, p, mlp, h):
    """(chosen expert ids [T, top], their weights [T, top], scores [T, E])."""
    r = mlp["router"]
    E, top = r["experts"], r["top"]
    s = torch.softmax(h @ W[p + "router"].T, -1)
    choice = s + W[p + "correction"]
    g = r.get("groups")
    if g and g["count"] > 1:
        per = E // g["count"]
        best = choice.view(-1, g["count"], per).max(-1).values.topk(g["keep"], -1).indices
        allowed = torch.zeros(h.shape[0], g["count"], dtype=torch.bool).scatter_(1, best, True)
        choice = choice.masked_fill(~allowed.repeat_interleave(per, 1), -math.inf)
    ids = choice.topk(top, -1).indices
    return ids, s.gather(1, ids) * r.get("scale", 1.0), s


def experts(W, p, mlp, h):
    ids, wts, _ = route(W, p, mlp, h)
    out = torch.zeros_like(h)
    for t in range(h.shape[0]):
        for e, w in zip(ids[t].tolist(), wts[t]):
            out[t] += w * gated_ff(W, f"{p}e{e}.", h[t:t + 1])[0]
    if mlp.get("shared"):
        out = out + torch.sigmoid(h @ W[p + "shared.sg"].T) * gated_ff(W, p + "shared.", h)
    return out


def forward(W, cfg, tokens, collect=None):
    """fp64 logits [T, vocab]; `collect` (a list) receives the stream after every layer."""
    eps, alpha = cfg["norm"]["eps"], cfg.get("postln_alpha", 1.0)
    x = W["embed"][torch.tensor(tokens)]
    latents = {}
    for i, L in enumerate(cfg["layers"]):
        p = f"l{i}."
        if L["type"] == "retention":
            y = retention(W, p + "mix.", L["mixer"], x, eps)
        elif L["type"] == "wkv":
            y = wkv(W, p + "mix.", L["mixer"], x, eps)
        else:
            y = latent_attention(W, p + "mix.", L["mixer"], x, eps, latents, i)
        x = post_norm(x, y, alpha, W[p + "ls1"], W[p + "norm1"], eps)
        if L.get("mlp"):
            x = post_norm(x, experts(W, p + "mlp.", L["mlp"], x), alpha, W[p + "ls2"], W[p + "norm2"], eps)
        if collect is not None:
            collect.append(x.clone())
    return (unit(x, eps) * (1.0 + W["final.norm"])) @ W["head"].T
