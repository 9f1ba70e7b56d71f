"""A plain, slow Ronavik decoder in float64 (or float32) torch on the CPU, one function per mechanism,
written from the design's equations.  It shares no code with hfee_amd: the tests compare the engine
with it.

Notation.  x: the residual stream [T, width] of one sequence whose first token sits at position 0.
`w`: a dict from tensor names to tensors (linear weights [out, in], applied as W x).  Every function
takes the whole sequence at once; the recurrent mixers walk over it token by token, so cutting a
sequence can change nothing here.
"""
from __future__ import annotations

import math

import torch
import torch.nn.functional as F


def rms_norm(x, weight, eps):
    return x / torch.sqrt((x * x).mean(-1, keepdim=True) + eps) * weight


def gelu_tanh(z):
    return 0.5 * z * (1 + torch.tanh(math.sqrt(2 / math.pi) * (z + 0.044715 * z ** 3)))


def causal_conv(x, taps, bias):
    """x [T, C], taps [C, K] (the last column is the current token's), zeros before the start."""
    T, C = x.shape
    K = taps.shape[1]
    padded = torch.cat([torch.zeros(K - 1, C, dtype=x.dtype), x], dim=0)
    y = torch.zeros_like(x)
    for j in range(K):
        y = y + padded[j:j + T] * taps[:, j]
    return y + bias


def sigmoid_attention(h, w, pre, m, eps):
    """Grouped attention without a softmax: a visible key's weight is sigmoid(score + a number a head);
    q and k are normed per head with a weight shared by the heads; no rotation; the query grows with
    the logarithm of its position in steps of `every`."""
    T = h.shape[0]
    H, G, D, V = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    q = rms_norm((h @ w[pre + "q"].T).view(T, H, D), w[pre + "q.norm"], eps)
    k = rms_norm((h @ w[pre + "k"].T).view(T, G, D), w[pre + "k.norm"], eps)
    v = (h @ w[pre + "v"].T).view(T, G, V)
    temp = m.get("q_temp")
    if temp is not None:
        p = torch.arange(T)
        steps = torch.div(p + 1, temp["every"], rounding_mode="floor")
        q = q * (1 + temp["coef"] * torch.log(steps.to(h.dtype) + 1))[:, None, None]
    rep = H // G
    kh, vh = k.repeat_interleave(rep, dim=1), v.repeat_interleave(rep, dim=1)
    s = torch.einsum("ihd,jhd->hij", q, kh) * m["scale"] + w[pre + "pb"][:, None, None]
    seen = torch.arange(T)[None, :] <= torch.arange(T)[:, None]
    p = torch.where(seen[None], torch.sigmoid(s), torch.zeros_like(s))
    o = torch.einsum("hij,jhd->ihd", p, vh).reshape(T, H * V)
    return o @ w[pre + "o"].T


def gated_linear_recurrent_unit(h, w, pre, m):
    """Two branches of `width` channels: y through gelu; u through a short convolution, then a
    recurrence a channel whose decay and input gate come from u by block-diagonal matrices."""
    T = h.shape[0]
    W, nb = m["width"], m["blocks"]
    y = gelu_tanh(h @ w[pre + "y"].T + w[pre + "y.b"])
    u = causal_conv(h @ w[pre + "x"].T + w[pre + "x.b"], w[pre + "conv"], w[pre + "conv.b"])
    ub = u.view(T, nb, W // nb)
    r = torch.sigmoid(torch.einsum("boi,tbi->tbo", w[pre + "ra"], ub) + w[pre + "ra.b"]).reshape(T, W)
    i = torch.sigmoid(torch.einsum("boi,tbi->tbo", w[pre + "ri"], ub) + w[pre + "ri.b"]).reshape(T, W)
    log_a = -8.0 * r * F.softplus(w[pre + "lam"])
    a = torch.exp(log_a)
    inject = torch.sqrt(1 - a * a) * i * u
    S = torch.zeros(W, dtype=h.dtype)
    out = []
    for t in range(T):
        S = a[t] * S + inject[t]
        out.append(S)
    return (torch.stack(out) * y) @ w[pre + "o"].T


def side_by_side(h, w, pre, m, eps):
    left = sigmoid_attention(h, w, pre + "left.", m["left"], eps)
    right = gated_linear_recurrent_unit(h, w, pre + "right.", m["right"])
    return m.get("left_scale", 1.0) * left + m.get("right_scale", 1.0) * right


def state_space(h, w, pre, m, eps):
    """A state matrix [state, vdim] a head: S <- exp(-exp(A) dt) S + dt B x^T, y = S^T C + D x; the
    heads side by side times silu(z), then normed in equal parts."""
    T = h.shape[0]
    H, V, N, G, K = m["heads"], m["vdim"], m["state"], m["groups"], m["conv"]
    inner = H * V
    proj = h @ w[pre + "in"].T
    z, xbc, dt = proj[:, :inner], proj[:, inner:2 * inner + 2 * G * N], proj[:, 2 * inner + 2 * G * N:]
    xbc = F.silu(causal_conv(xbc, w[pre + "conv"], w[pre + "conv.b"]))
    x = xbc[:, :inner].view(T, H, V)
    B = xbc[:, inner:inner + G * N].view(T, G, N).repeat_interleave(H // G, dim=1)
    C = xbc[:, inner + G * N:].view(T, G, N).repeat_interleave(H // G, dim=1)
    dt = F.softplus(dt + w[pre + "dt_bias"])                       # [T, H]
    decay = torch.exp(-torch.exp(w[pre + "A_log"]) * dt)           # [T, H]
    S = torch.zeros(H, N, V, dtype=h.dtype)
    ys = []
    for t in range(T):
        S = decay[t][:, None, None] * S + dt[t][:, None, None] * B[t][:, :, None] * x[t][:, None, :]
        ys.append(torch.einsum("hnv,hn->hv", S, C[t]) + w[pre + "D"][:, None] * x[t])
    y = torch.stack(ys).reshape(T, inner) * F.silu(z)
    parts = m["norm_groups"]
    yg = y.view(T, parts, inner // parts)
    yg = yg / torch.sqrt((yg * yg).mean(-1, keepdim=True) + eps)
    return (yg.reshape(T, inner) * w[pre + "norm"]) @ w[pre + "o"].T


def routed_experts(h, w, pre, mlp, margins=None):
    """Scores sigmoid(W_router h); the `top` largest choose the experts; a chosen expert's score
    multiplies its input; down(relu(up(.))^2); the outputs are summed.  margins: a list that receives, a
    token, how far the last chosen expert's logit is above the best one not chosen, in units of the
    logits' spread over the experts (infinite where every expert is chosen)."""
    E, top = mlp["router"]["experts"], mlp["router"]["top"]
    z = h @ w[pre + "router"].T
    # (the largest scores are the largest logits; chosen by the logits, so that two scores that both round
    # to one cannot tie)
    idx = torch.topk(z, top, dim=-1).indices
    vals = torch.sigmoid(torch.gather(z, -1, idx))
    if margins is not None:
        if top < E:
            best = torch.topk(z, top + 1, dim=-1).values
            margins.append((best[:, top - 1] - best[:, top]) / z.std(dim=-1).clamp_min(1e-30))
        else:
            margins.append(torch.full((h.shape[0],), float("inf"), dtype=h.dtype))
    out = torch.zeros(h.shape[0], w[pre + "e0.down"].shape[0], dtype=h.dtype)
    for t in range(h.shape[0]):
        for j in range(top):
            e = int(idx[t, j])
            a = torch.relu(w[f"{pre}e{e}.up"] @ (vals[t, j] * h[t])) ** 2
            out[t] = out[t] + w[f"{pre}e{e}.down"] @ a
    return out


def forward(cfg: dict, w: dict, tokens, dtype=torch.float64, layers_out=None, margins_out=None):
    """Logits [T, vocab] of one sequence from position 0.  layers_out: a list that receives the
    residual stream after every layer; margins_out: one that receives every router's margins [T]."""
    w = {k: (v.to(dtype) if v.is_floating_point() else v) for k, v in w.items()}
    eps = cfg["norm"]["eps"]
    tok = torch.as_tensor(tokens, dtype=torch.long)
    x = w["embed"][tok] + w["pos"][:len(tok)]
    for i, layer in enumerate(cfg["layers"]):
        pre = f"l{i}."
        h = rms_norm(x, w[pre + "norm1"], eps)
        if layer["type"] == "parallel":
            y = side_by_side(h, w, pre + "mix.", layer["mixer"], eps)
        elif layer["type"] == "mamba2":
            y = state_space(h, w, pre + "mix.", layer["mixer"], eps)
        else:
            raise ValueError(layer["type"])
        y = y * torch.sigmoid(h @ w[pre + "rg1"].T + w[pre + "rg1.b"])
        x = x + rms_norm(y, w[pre + "norm1b"], eps)
        if layer.get("mlp") is not None:
            h = rms_norm(x, w[pre + "norm2"], eps)
            y = routed_experts(h, w, pre + "mlp.", layer["mlp"], margins_out)
            y = y * torch.sigmoid(h @ w[pre + "rg2"].T + w[pre + "rg2.b"])
            x = x + rms_norm(y, w[pre + "norm2b"], eps)
        if layers_out is not None:
            layers_out.append(x.clone())
    return rms_norm(x, w["final.norm"], eps) @ w["embed"].T
