"""A plain, slow Saposun decoder in float64 torch on the CPU, one function per mechanism, written from
the design's equations.  It shares no code with hfee_amd: the tests compare the engine with it.

Notation.  x: the residual stream [T, width] of one sequence whose first token sits at position 0.
`w`: a dict from tensor names to tensors (linear weights [out, in], applied as W x).  `m`: the "mixer"
dict of a layer's entry in config.json.  Every function takes the whole sequence at once; the retention
walks over it token by token, so cutting a sequence can change nothing here.
"""
from __future__ import annotations

import torch
import torch.nn.functional as F


def rms(x, eps):
    return x / torch.sqrt((x * x).mean(-1, keepdim=True) + eps)


def rms_norm(x, weight, eps):
    return rms(x, eps) * weight


def angles(positions, dims, base):
    freq = torch.tensor([base ** (-2.0 * i / dims) for i in range(dims // 2)], dtype=torch.float64)
    return positions.to(torch.float64)[:, None] * freq[None, :]


def rotate_half(x, positions, dims, base):
    """x [T, heads, dim]: the first `dims` dims of each head are turned, pairs (i, i + dims/2)."""
    half = dims // 2
    a = angles(positions, dims, base)
    cos, sin = torch.cos(a).to(x.dtype)[:, None, :], torch.sin(a).to(x.dtype)[:, None, :]
    u, v = x[..., :half], x[..., half:dims]
    return torch.cat([u * cos - v * sin, v * cos + u * sin, x[..., dims:]], dim=-1)


def rotate_interleaved(x, positions, dims, base):
    """x [T, heads, dim]: the first `dims` dims of each head are turned, pairs (2i, 2i + 1)."""
    a = angles(positions, dims, base)
    cos, sin = torch.cos(a).to(x.dtype)[:, None, :], torch.sin(a).to(x.dtype)[:, None, :]
    u, v = x[..., 0:dims:2], x[..., 1:dims:2]
    turned = torch.stack([u * cos - v * sin, v * cos + u * sin], dim=-1).flatten(-2)
    return torch.cat([turned, x[..., dims:]], dim=-1)


def window_mask(T, size):
    i, j = torch.arange(T)[:, None], torch.arange(T)[None, :]
    return (i - j >= 0) & (i - j < size)


def latent_keys(h, w, pre, m, eps):
    """What a latent-attention layer leaves for itself and for the layers that read it: the normed latent
    c [T, kv_rank] and the rotated key part [T, rot_dim]."""
    T = h.shape[0]
    R, Dr = m["kv_rank"], m["rot_dim"]
    down = h @ w[pre + "dkv"].T
    c = rms_norm(down[:, :R], w[pre + "dkv.norm"], eps)
    pos = torch.arange(T)
    kr = rotate_interleaved(down[:, None, R:R + Dr], pos, m["rot"]["dims"], m["rot"]["base"])[:, 0]
    return c, kr


def latent_attention(h, w, pre, m, eps, shared=None):
    """shared: (c, rotated key part) of the layer named by `kv_from`, or None for a layer with its own."""
    T = h.shape[0]
    H, Dn, Dr, Dv = m["heads"], m["dim"], m["rot_dim"], m["vdim"]
    c, kr = latent_keys(h, w, pre, m, eps) if shared is None else shared
    cq = rms_norm(h @ w[pre + "dq"].T, w[pre + "dq.norm"], eps)
    q = (cq @ w[pre + "uq"].T).view(T, H, Dn + Dr)
    pos = torch.arange(T)
    q_plain = q[..., :Dn]
    q_rot = rotate_interleaved(q[..., Dn:], pos, m["rot"]["dims"], m["rot"]["base"])
    k_plain = (c @ w[pre + "uk"].T).view(T, H, Dn)
    v = (c @ w[pre + "uv"].T).view(T, H, Dv)
    s = torch.einsum("ihd,jhd->hij", q_plain, k_plain) + torch.einsum("ihd,jd->hij", q_rot, kr)
    s = s * m["scale"]
    s = s.masked_fill(~window_mask(T, m["mask"]["size"] if m.get("mask") else T)[None], float("-inf"))
    p = torch.softmax(s, dim=-1)
    o = torch.einsum("hij,jhd->ihd", p, v).reshape(T, H * Dv)
    return o @ w[pre + "o"].T


def retention(h, w, pre, m, eps):
    T = h.shape[0]
    H, D, V = m["heads"], m["dim"], m["vdim"]
    pos = torch.arange(T)
    q = (h @ w[pre + "q"].T).view(T, H, D)
    k = (h @ w[pre + "k"].T).view(T, H, D)
    v = (h @ w[pre + "v"].T).view(T, H, V)
    if m.get("rot"):
        q = rotate_half(q, pos, m["rot"]["dims"], m["rot"]["base"])
        k = rotate_half(k, pos, m["rot"]["dims"], m["rot"]["base"])
    k = k * D ** -0.5
    decay = torch.tensor(m["decay"], dtype=h.dtype)
    S = torch.zeros(H, D, V, dtype=h.dtype)
    out = []
    for t in range(T):
        S = decay[:, None, None] * S + k[t][:, :, None] * v[t][:, None, :]
        out.append(torch.einsum("hdv,hd->hv", S, q[t]))
    o = rms(torch.stack(out), eps).reshape(T, H * V)
    o = o * F.silu(h @ w[pre + "g"].T)
    return o @ w[pre + "o"].T


def short_conv(u, taps):
    """u [T, C], taps [C, K]: y_t = sum_j taps[:, j] * u_(t - K + 1 + j), zeros before the start."""
    T, C = u.shape
    K = taps.shape[1]
    padded = torch.cat([torch.zeros(K - 1, C, dtype=u.dtype), u], dim=0)
    return sum(padded[j:j + T] * taps[:, j][None, :] for j in range(K))


def pooled_window_attention(h, w, pre, m, eps):
    T = h.shape[0]
    H, G, D, V = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    pos = torch.arange(T)
    q, k, v = h @ w[pre + "q"].T, h @ w[pre + "k"].T, h @ w[pre + "v"].T
    if m.get("conv"):
        q, k, v = short_conv(q, w[pre + "q.conv"]), short_conv(k, w[pre + "k.conv"]), short_conv(v, w[pre + "v.conv"])
    q, k, v = q.view(T, H, D), k.view(T, G, D), v.view(T, G, V)
    if m.get("rot"):
        q = rotate_half(q, pos, m["rot"]["dims"], m["rot"]["base"])
        k = rotate_half(k, pos, m["rot"]["dims"], m["rot"]["base"])
    v = rms(v, eps)
    size = m["mask"]["size"] if m.get("mask") else T          # (without a mask: every earlier position)
    P = m["mask"].get("pool", 0) if m.get("mask") else 0
    cap = m.get("softcap")
    out = torch.zeros(T, H, V, dtype=h.dtype)
    for i in range(T):
        first = max(0, i - size + 1)
        keys, values = [k[first:i + 1]], [v[first:i + 1]]
        if P:
            for b in range(T // P):
                if b * P + P - 1 <= i - size:
                    keys.append(k[b * P:b * P + P].mean(0, keepdim=True))
                    values.append(v[b * P:b * P + P].mean(0, keepdim=True))
        kk, vv = torch.cat(keys), torch.cat(values)                 # [keys, G, D]
        for hd in range(H):
            g = hd // (H // G)
            s = (kk[:, g] @ q[i, hd]) * m["scale"]
            if cap:
                s = cap * torch.tanh(s / cap)
            out[i, hd] = torch.softmax(s, dim=0) @ vv[:, g]
    gate = torch.sigmoid(h @ w[pre + "g"].T)                        # [T, H]
    o = (out * gate[:, :, None]).reshape(T, H * V)
    return o @ w[pre + "o"].T


def router(h, w, pre, r):
    """(chosen experts [T, top], their weights [T, top], the margin between the last chosen and the best
    unchosen choice score of every token)."""
    z = h @ w[pre + "router"].T
    s = torch.softmax(z, dim=-1)
    choice = s + w[pre + "correction"]
    top = r["top"]
    order = torch.sort(choice, dim=-1, descending=True, stable=True)
    chosen = order.indices[:, :top]
    margin = (order.values[:, top - 1] - order.values[:, top]) if top < choice.shape[1] else torch.full((h.shape[0],), float("inf"))
    return chosen, torch.gather(s, 1, chosen), margin


def experts(h, w, pre, mlp, margins=None):
    chosen, weights, margin = router(h, w, pre, mlp["router"])
    if margins is not None:
        margins.append(margin)
    out = torch.zeros_like(h)
    for t in range(h.shape[0]):
        for j in range(chosen.shape[1]):
            e = int(chosen[t, j])
            p = f"{pre}e{e}."
            y = (F.silu(w[p + "gate"] @ h[t]) * (w[p + "up"] @ h[t]))
            out[t] += weights[t, j] * (w[p + "down"] @ y)
    return out


def layer(x, w, i, cfg, shared_keys, margins=None):
    entry = cfg["layers"][i]
    eps, mult = cfg["norm"]["eps"], cfg.get("residual_mult", 1.0)
    m, pre = entry["mixer"], f"l{i}.mix."
    h = rms_norm(x, w[f"l{i}.norm1"], eps)
    if entry["type"] == "latent_attention":
        if m.get("kv_from") is None:
            shared_keys[i] = latent_keys(h, w, pre, m, eps)
            y = latent_attention(h, w, pre, m, eps)
        else:
            y = latent_attention(h, w, pre, m, eps, shared=shared_keys[m["kv_from"]])
    elif entry["type"] == "retention":
        y = retention(h, w, pre, m, eps)
    elif entry["type"] == "attention":
        y = pooled_window_attention(h, w, pre, m, eps)
    else:
        raise ValueError(entry["type"])
    if entry.get("mlp") is not None:
        y = y + experts(h, w, f"l{i}.mlp.", entry["mlp"], margins)
    return x + mult * y


def forward(tokens, w, cfg, dtype=torch.float64, streams=None, margins=None):
    """Logits [T, vocab] of one sequence; `streams` (a list) gets the residual stream after every layer,
    `margins` every router's margins."""
    w = {n: (t.to(dtype) if t.is_floating_point() else t) for n, t in w.items()}
    x = w["embed"][torch.as_tensor(tokens, dtype=torch.long)]
    shared_keys = {}
    for i in range(len(cfg["layers"])):
        x = layer(x, w, i, cfg, shared_keys, margins)
        if streams is not None:
            streams.append(x)
    return rms_norm(x, w["final.norm"], cfg["norm"]["eps"]) @ w["head"].T


def greedy(tokens, w, cfg, count):
    tokens = list(tokens)
    out = []
    for _ in range(count):
        nxt = int(forward(tokens, w, cfg)[-1].argmax())
        out.append(nxt)
        tokens.append(nxt)
    return out
