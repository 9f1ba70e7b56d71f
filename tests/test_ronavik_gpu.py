"""The Ronavik decoder on the GPU against the plain implementation: the new kernels alone (attention without a
softmax with a key that stands out far back and at page borders, the norm of q and k with the temperature's
steps, the real-gated recurrent unit and the state-space recurrence in portions over slots, the gate before
the norm in parts, the gated residual, the router and the experts without a gate, learned positions), each
mechanism as a model of one layer, the whole model under four ways of cutting the same requests into steps
(whole, bulk then single tokens, portions down to two tokens, mixed batches on a small page pool with four
state slots, pages and slots used again), in 32-bit and in bfloat16, on configurations with even and with
odd sizes and on one without any attention; long decoding through graph replays; greedy generation through
the entry point and its scheduler; the trace runner and the command line as subprocesses."""
import json
import math
import os
import subprocess
import sys

import numpy as np
import pytest
import torch
import torch.nn.functional as F

import plain_ronavik as pr
import ronavik_util as ru
import trace_util as tu
from conftest import ROOT

pytestmark = pytest.mark.gpu

TOL = {"float32": 3e-5, "bfloat16": 8e-2}
DT = {"float32": torch.float32, "bfloat16": torch.bfloat16}
LENGTHS = {"A": [5, 17, 64, 1, 100, 33, 129, 49, 2], "B": [40, 3, 100, 65, 2, 31], "C": [90, 3, 41, 1, 130],
           "D": [700, 47, 313, 1, 161]}


def i32(a):
    return torch.as_tensor(np.asarray(a, dtype=np.int32)).cuda()


# ------------------------------------------------------------------ kernels alone

def _paged(lengths, page_size=16, seed=0):
    """Block tables for sequences of these lengths over shuffled pages (page 0 is never handed out, so that a
    table's unused entries, which hold 0, would show if they were read)."""
    rng = np.random.default_rng(seed)
    need = [-(-n // page_size) for n in lengths]
    pages = rng.permutation(np.arange(1, sum(need) + 1))
    tables, at = np.zeros((len(lengths), max(need)), dtype=np.int32), 0
    for s, k in enumerate(need):
        tables[s, :k] = pages[at:at + k]
        at += k
    return tables, sum(need) + 1


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("H,G,dk,dv,every", [(4, 2, 16, 32, 8), (3, 3, 20, 12, 5), (8, 2, 32, 64, 100), (2, 1, 16, 48, 0)])
def test_attention_without_a_softmax(dtype, H, G, dk, dv, every):
    """Two sequences side by side, the longer one of several hundred tokens: written in portions whose edges
    fall inside pages, read by portions and by single tokens (the long one's keys split over several waves),
    plain and, where the sizes allow, on the matrix cores.  One key far back is made to stand out for one
    query head: its weight is near one where all others are near zero, so leaving it out, or normalizing,
    shows at once."""
    from hfee_amd.kernels import ops
    dt = DT[dtype]
    g = torch.Generator().manual_seed(dk + H)
    lengths, scale, eps, coef = [613, 37], 0.25, 1e-5, 0.6
    qs = [torch.randn(n, H, dk, generator=g) for n in lengths]
    ks = [torch.randn(n, G, dk, generator=g) for n in lengths]
    vs = [torch.randn(n, G, dv, generator=g) for n in lengths]
    qw, kw = torch.rand(dk, generator=g) + 0.5, torch.rand(dk, generator=g) + 0.5
    bias = torch.randn(H, generator=g) - 6.0                 # (most keys weigh next to nothing)
    far = 3
    ks[0][far, 1 // (H // G)] = qs[0][-1, 1] * 4.0            # the last query of head 1 looks at key 3 of its key head
    ks[0][15], ks[0][16] = ks[0][15] * 2, ks[0][16] * 2       # the keys on both sides of a page border
    qs, ks, vs = ([t.to(dt).float() for t in x] for x in (qs, ks, vs))

    def definition(q, k, v):
        n = q.shape[0]
        rms = lambda x, w: x / torch.sqrt((x * x).mean(-1, keepdim=True) + eps) * w          # noqa: E731
        qn, kn = rms(q.double(), qw.double()), rms(k.double(), kw.double())
        if every:
            steps = torch.div(torch.arange(n) + 1, every, rounding_mode="floor")
            qn = qn * (1 + coef * torch.log(steps.double() + 1))[:, None, None]
        kh, vh = kn.repeat_interleave(H // G, 1), v.double().repeat_interleave(H // G, 1)
        s = torch.einsum("ihd,jhd->hij", qn, kh) * scale + bias.double()[:, None, None]
        p = torch.sigmoid(s) * (torch.arange(n)[None, :] <= torch.arange(n)[:, None])
        return torch.einsum("hij,jhd->ihd", p, vh).reshape(n, H * dv)
    want = [definition(q, k, v) for q, k, v in zip(qs, ks, vs)]

    tables, pages = _paged(lengths)
    cache = torch.zeros(pages, G, 16 * (dk + dv), dtype=dt, device="cuda")
    cache[0].fill_(float("nan"))
    bt = i32(tables)
    matrix = dtype == "bfloat16" and ops.attention_kv_sizes_fit(dk, dv)
    got = [torch.zeros(n, H * dv) for n in lengths]
    fed = [0, 0]
    for sizes in ([7, 2], [9, 0], [300, 17], [290, 16], [1, 1], [5, 1], [1, 0]):
        segs = [(s, n) for s, n in enumerate(sizes) if n]
        n_all = sum(n for _, n in segs)
        q = torch.cat([qs[s][fed[s]:fed[s] + n].reshape(n, -1) for s, n in segs]).to(dt).cuda()
        k = torch.cat([ks[s][fed[s]:fed[s] + n].reshape(n, -1) for s, n in segs]).to(dt).cuda()
        v = torch.cat([vs[s][fed[s]:fed[s] + n].reshape(n, -1) for s, n in segs]).to(dt).cuda()
        positions = i32(np.concatenate([np.arange(fed[s], fed[s] + n) for s, n in segs]))
        token_segment = i32(np.concatenate([np.full(n, i) for i, (_, n) in enumerate(segs)]))
        tab = bt[[s for s, _ in segs]].contiguous()
        ops.qk_norm_write(q, k, v, positions, token_segment, tab, cache, qw.cuda(), kw.cuda(), eps, H, G, dk, dv, 16,
                          temperature=(coef, every) if every else None)
        out = torch.zeros(n_all, H * dv, dtype=dt, device="cuda")
        ops.attention_kv_plain(out, q, cache, positions, token_segment, tab, H, G, dk, dv, 16, scale, bias.cuda(), weights="sigmoid")
        outs = [out]
        if matrix:
            rows_most = ops.attention_kv_rows(dk, dv, H // G, "sigmoid")
            portions, singles, row = [], [], 0
            for i, (s, n) in enumerate(segs):
                if n > 1:
                    portions += [(row + o, min(rows_most, n - o), fed[s] + o, i) for o in range(0, n, rows_most)]
                else:
                    singles.append((row, 1, fed[s], i))
                row += n
            out2 = torch.zeros(n_all, H * dv, dtype=dt, device="cuda")
            if portions:
                ops.attention_kv_bf16(out2, q, cache, i32(portions).reshape(-1, 4), 0, tab, H, G, dk, dv, 16, scale, bias.cuda(),
                                      weights="sigmoid")
            if singles:
                for splits in (1, 3):
                    partial = torch.zeros(ops.attention_kv_partial_words(len(singles), H, dv, splits) + 1, device="cuda")
                    ops.attention_kv_bf16(out2, q, cache, i32(singles).reshape(-1, 4), 1, tab, H, G, dk, dv, 16, scale,
                                          bias.cuda(), partial=partial if splits > 1 else None, splits=splits, weights="sigmoid")
                    if splits == 1:
                        first = out2.clone()
                    else:
                        rows_single = [r for r, _, _, _ in singles]
                        assert ru.rel(out2[rows_single].float().cpu(), first[rows_single].float().cpu()) < 2e-2
            outs.append(out2)
        row = 0
        for s, n in segs:
            for o in outs:
                w = want[s][fed[s]:fed[s] + n]
                err = (o[row:row + n].double().cpu() - w).abs().max() / w.abs().max()
                assert err < (2e-5 if dtype == "float32" else 3e-2), (sizes, s, float(err))
            got[s][fed[s]:fed[s] + n] = outs[-1][row:row + n].float().cpu()
            fed[s] += n
            row += n
    assert fed == lengths


def test_the_temperature_steps_where_it_should():
    """q at positions around multiples of `every`: the factor is 1 + coef * ln(floor((p + 1) / every) + 1)."""
    from hfee_amd.kernels import ops
    every, coef, dk = 7, 0.9, 8
    positions = [0, 5, 6, 7, 12, 13, 14, 47, 48]
    q = torch.ones(len(positions), dk).cuda()
    ops.qk_norm_write(q, None, None, i32(positions), None, None, None, torch.ones(dk).cuda(), None, 0.0, 1, 1, dk, dk, 16,
                      temperature=(coef, every))
    want = [1 + coef * math.log((p + 1) // every + 1) for p in positions]
    assert np.allclose(q[:, 0].cpu().numpy(), want, rtol=1e-6)
    assert want[1] == 1.0 and want[2] > 1.0 and want[5] > want[4] and want[8] > want[7]


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("W,blocks", [(48, 3), (40, 1), (300, 5)])
def test_recurrent_unit_in_portions(dtype, W, blocks):
    """The unit by its definition in float64 against the kernels fed the same two sequences in portions of
    unequal size (down to single tokens, and long ones that are walked in chunks, the last chunk not full,
    beside a short one) in other slots; a slot of NaNs beside them stays untouched."""
    from hfee_amd.kernels import ops
    dt = DT[dtype]
    g = torch.Generator().manual_seed(W)
    T, bs = [301, 23], W // blocks
    ra, ri = torch.randn(blocks, bs, bs, generator=g) * 0.5, torch.randn(blocks, bs, bs, generator=g) * 0.5
    rab, rib = torch.randn(blocks, bs, generator=g), torch.randn(blocks, bs, generator=g)
    lam, yb = torch.randn(W, generator=g) - 2.0, torch.randn(W, generator=g) * 0.3
    us = [torch.randn(t, W, generator=g) for t in T]
    ys = [torch.randn(t, W, generator=g).to(dt).float() for t in T]
    want, final = [], []
    for u, y in zip(us, ys):
        ub = u.double().view(-1, blocks, bs)
        r = torch.sigmoid(torch.einsum("boi,tbi->tbo", ra.double(), ub) + rab.double()).reshape(-1, W)
        i = torch.sigmoid(torch.einsum("boi,tbi->tbo", ri.double(), ub) + rib.double()).reshape(-1, W)
        a = torch.exp(-8.0 * r * F.softplus(lam.double()))
        S, out = torch.zeros(W, dtype=torch.float64), []
        for t in range(u.shape[0]):
            S = a[t] * S + torch.sqrt(1 - a[t] ** 2) * i[t] * u[t].double()
            out.append(S * pr.gelu_tanh(y[t].double() + yb.double()))
        want.append(torch.stack(out))
        final.append(S)
    w_gates = torch.cat([ra, ri], dim=1).transpose(1, 2).contiguous().cuda()
    gate_bias = torch.cat([rab, rib], dim=1).contiguous().view(-1).cuda()
    rate = (-8.0 * F.softplus(lam)).cuda()
    state = torch.zeros(5, W, device="cuda")
    state[1].fill_(float("nan"))
    slots, fed = [3, 0], [0, 0]
    got = [torch.zeros(t, W) for t in T]
    for sizes in ([7, 2], [1, 1], [150, 0], [2, 13], [141, 7]):
        segs = [(s, n) for s, n in enumerate(sizes) if n]
        u = torch.cat([us[s][fed[s]:fed[s] + n] for s, n in segs]).cuda()
        y = torch.cat([ys[s][fed[s]:fed[s] + n] for s, n in segs]).to(dt).cuda()
        rows = np.cumsum([0] + [n for _, n in segs])[:-1]
        gates = torch.zeros(u.shape[0], 2 * W, device="cuda")
        ops.head_linear(gates, u, w_gates, blocks, bs, 2 * bs)
        out = torch.zeros(u.shape[0], W, dtype=dt, device="cuda")
        words = ops.rglru_scan_scratch(max(sizes), len(segs), W)
        assert (words > 0) == (max(sizes) > 100)
        ops.rglru_scan(out, state, gates, gate_bias, u, rate, y, yb.cuda(), i32(rows), i32([n for _, n in segs]),
                       i32([slots[s] for s, _ in segs]), bs, longest=max(sizes),
                       scratch=torch.full((words,), float("nan"), device="cuda") if words else None)
        for (s, n), r in zip(segs, rows):
            got[s][fed[s]:fed[s] + n] = out[r:r + n].float().cpu()
            fed[s] += n
    for s in range(2):
        assert ru.rel(got[s], want[s]) < (2e-5 if dtype == "float32" else 6e-3)
        assert ru.rel(state[slots[s]].cpu(), final[s]) < 2e-5
    assert bool(torch.isnan(state[1]).all()) and float(state[2].abs().sum()) == 0.0


@pytest.mark.parametrize("n", [5, 33, 150])
def test_products_a_block_in_32_bit(n):
    """out[t, h] = W_h^T x[t, h] with what lies behind a head's inputs copied behind its outputs: a few tokens
    on the vector units, many on the matrix cores in float32 (tiles of 64 tokens and 128 outputs that the
    sizes do not fill, inputs that are no whole chunk); a token's result does not depend on its company."""
    from hfee_amd.kernels import ops
    g = torch.Generator().manual_seed(n)
    heads, n_in, n_out, tail = 3, 70, 150, 5
    x = torch.randn(n, heads * (n_in + tail) + 3, generator=g)
    w = torch.randn(heads, n_in, n_out, generator=g)
    out = torch.full((n, heads * (n_out + tail) + 2), float("nan"), device="cuda")
    ops.head_linear(out, x.cuda(), w.cuda(), heads, n_in, n_out, tail=tail)
    xh = x[:, :heads * (n_in + tail)].view(n, heads, n_in + tail).double()
    want = torch.cat([torch.einsum("thi,hio->tho", xh[:, :, :n_in], w.double()), xh[:, :, n_in:]], dim=2).reshape(n, -1)
    got = out.cpu()
    assert ru.rel(got[:, :want.shape[1]], want) < 2e-6
    assert bool(torch.isnan(got[:, want.shape[1]:]).all())
    if n >= 64:          # the first tokens alone, in a step of their own size: the same bits
        alone = torch.zeros(40, out.shape[1], device="cuda")
        ops.head_linear(alone, x[:40].cuda(), w.cuda(), heads, n_in, n_out, tail=tail)
        assert torch.equal(alone.cpu()[:, :want.shape[1]], got[:40, :want.shape[1]])


@pytest.mark.parametrize("H,G,N,V", [(4, 2, 16, 8), (3, 1, 10, 12), (2, 2, 33, 70), (8, 4, 64, 32)])
def test_state_space_recurrence_in_portions(H, G, N, V):
    """S <- a S + dt B x^T with one decay a head, y = S^T C, by its definition in float64 against the kernel
    in portions for two requests in other slots, the final states included."""
    from hfee_amd.kernels import ops
    g = torch.Generator().manual_seed(N)
    T = [45, 23]
    data = []
    for t in T:
        C, B = torch.randn(t, G, N, generator=g) * 0.4, torch.randn(t, G, N, generator=g) * 0.4
        x = torch.randn(t, H, V, generator=g)
        a = torch.rand(t, H, generator=g) * 0.3 + 0.7
        dtv = torch.rand(t, H, generator=g) + 0.1
        data.append((C, B, x, a, dtv))
    want, final = [], []
    for C, B, x, a, dtv in data:
        o = torch.zeros(C.shape[0], H, V, dtype=torch.float64)
        final.append([])
        for h in range(H):
            S = torch.zeros(N, V, dtype=torch.float64)
            for t in range(C.shape[0]):
                S = a[t, h].double() * S + dtv[t, h].double() * B[t, h // (H // G)].double()[:, None] * x[t, h].double()[None, :]
                o[t, h] = S.T @ C[t, h // (H // G)].double()
            final[-1].append(S)
        want.append(o.reshape(C.shape[0], -1))
    state = torch.zeros(5, H, *ops.scan_state_shape(N, V), device="cuda")
    state[1].fill_(float("nan"))
    slots, fed = [3, 0], [0, 0]
    got = [torch.zeros(t, H * V) for t in T]
    for sizes in ([7, 2], [1, 1], [20, 0], [2, 13], [15, 7]):
        segs = [(s, n) for s, n in enumerate(sizes) if n]
        parts = [tuple(x[fed[s]:fed[s] + n] for x in data[s]) for s, n in segs]
        cat = [torch.cat([p[i].reshape(p[i].shape[0], -1) for p in parts]).cuda().contiguous() for i in range(5)]
        rows = np.cumsum([0] + [n for _, n in segs])[:-1]
        out = torch.zeros(sum(n for _, n in segs), H * V, device="cuda")
        ops.linear_scan(out, state, cat[0], cat[1], cat[2], cat[3], cat[4], i32(rows), i32([n for _, n in segs]),
                        i32([slots[s] for s, _ in segs]), H, G, N, V, "scaled_add", decay_per_head=True)
        for (s, n), r in zip(segs, rows):
            got[s][fed[s]:fed[s] + n] = out[r:r + n].cpu()
            fed[s] += n
    for s in range(2):
        assert ru.rel(got[s], want[s]) < 2e-5
        assert ru.rel(ops.scan_state_matrix(state[slots[s]], N, V).cpu(), torch.stack(final[s])) < 2e-5
    assert bool(torch.isnan(state[1]).all()) and float(state[2].abs().sum()) == 0.0


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("C", [10, 24])
def test_convolution_with_biases_carries_its_inputs(dtype, C):
    """A bias on the inputs stands only where there is an input: before a sequence's start are zeros.  Portions
    shorter than the taps; the state holds the inputs with their bias."""
    from hfee_amd.kernels import ops
    dt = DT[dtype]
    g = torch.Generator().manual_seed(1)
    K, T = 4, 19
    x = torch.randn(T, C, generator=g).to(dt)
    taps, ib, ob = torch.randn(C, K, generator=g), torch.randn(C, generator=g), torch.randn(C, generator=g)
    biased = (x.float() + ib).to(dt).double()
    want = pr.causal_conv(biased, taps.double(), ob.double())
    state = torch.zeros(3, K - 1, C, dtype=dt, device="cuda")
    got, at = torch.zeros(T, C), 0
    for n in (2, 1, 1, 7, 3, 5):
        rows = x[at:at + n].cuda()
        y = torch.zeros(n, C, device="cuda")
        seg = (i32(np.zeros(n)), i32([0]), i32([2]))
        ops.short_conv_silu(y, rows, state, taps.cuda(), *seg, in_bias=ib.cuda(), out_bias=ob.cuda(), activation="none")
        ops.short_conv_keep(state, rows, i32([0]), i32([n]), i32([2]), in_bias=ib.cuda())
        got[at:at + n] = y.cpu()
        at += n
    assert ru.rel(got, want) < 2e-6
    assert torch.equal(state[2].double().cpu(), biased[T - (K - 1):])
    assert float(state[:2].abs().sum()) == 0.0


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_gate_then_norm_in_parts_and_the_gated_residual(dtype):
    from hfee_amd.kernels import ops
    dt = DT[dtype]
    g = torch.Generator().manual_seed(2)
    n, H, V, parts, eps = 5, 6, 10, 4, 1e-5
    inner = H * V
    o, x = torch.randn(n, inner, generator=g), torch.randn(n, inner, generator=g)
    z = torch.randn(n, inner, generator=g).to(dt)
    skip, w = torch.randn(H, generator=g), torch.rand(inner, generator=g) + 0.5
    out = torch.zeros(n, inner, dtype=dt, device="cuda")
    ops.gate_group_norm(out, o.cuda(), x.cuda(), skip.cuda(), z.cuda(), w.cuda(), H, parts, eps)
    y = (o.double() + skip.double().repeat_interleave(V) * x.double()) * F.silu(z.double())
    yg = y.view(n, parts, -1)
    want = (yg / torch.sqrt((yg * yg).mean(-1, keepdim=True) + eps)).reshape(n, inner) * w.double()
    assert ru.rel(out.double().cpu(), want) < (2e-6 if dtype == "float32" else 6e-3)
    # x += norm((a y + b y2) * sigmoid(gate + bias)) * w, and the norm that follows: rows that are no whole
    # groups of four or start anywhere (a loop over the row), and rows that a thread holds in registers
    # (one, two and eight groups a thread, the last ones past the row's end)
    for d, shift in ((90, 3), (64, 8), (1032, 8), (5000, 16)):
        xs, y1, y2 = (torch.randn(n, d, generator=g) for _ in range(3))
        wide = torch.randn(n, d + 2 * shift, generator=g).to(dt)
        gate, gate_gpu = wide[:, shift:shift + d], wide.cuda()[:, shift:shift + d]        # (rows inside wider rows)
        gb, w1, w2 = torch.randn(d, generator=g), torch.rand(d, generator=g) + 0.5, torch.rand(d, generator=g) + 0.5
        for second in (True, False):
            for gated in (True, False):
                xg, nxt = xs.clone().cuda(), torch.zeros(n, d, dtype=dt, device="cuda")
                ops.gated_norm_add(xg, y1.cuda(), w1.cuda(), eps, y2=y2.cuda() if second else None, scales=(0.7, -1.3),
                                   gate=gate_gpu if gated else None, gate_bias=gb.cuda() if gated else None, next_out=nxt,
                                   next_weight=w2.cuda(), next_eps=2 * eps)
                v = 0.7 * y1.double() + (-1.3 * y2.double() if second else 0)
                if gated:
                    v = v * torch.sigmoid(gate.double() + gb.double())
                want_x = xs.double() + pr.rms_norm(v, w1.double(), eps)
                assert ru.rel(xg.double().cpu(), want_x) < 2e-6
                assert ru.rel(nxt.double().cpu(), pr.rms_norm(want_x, w2.double(), 2 * eps)) < (2e-6 if dtype == "float32" else 6e-3)
    d = 90
    xs, y1, y2 = (torch.randn(n, d, generator=g) for _ in range(3))
    xa = xs.clone().cuda()
    ops.scaled_add(xa, y1.cuda(), 0.7, y2.cuda(), -1.3)
    assert ru.rel(xa.cpu(), xs + 0.7 * y1 - 1.3 * y2) < 1e-6
    table = torch.randn(9, d, generator=g).to(dt)
    xp = xs.clone().cuda()
    ops.add_table_rows(xp, table.cuda(), i32([8, 0, 3, 3, 1]))
    assert torch.equal(xp.cpu(), xs + table.float()[[8, 0, 3, 3, 1]])


@pytest.mark.parametrize("n,E,top", [(50, 5, 2), (7, 70, 3), (33, 4, 4), (9, 130, 1)])
def test_the_router_picks_the_largest_scores(n, E, top):
    from hfee_amd.kernels import ops
    g = torch.Generator().manual_seed(E)
    logits = torch.randn(n, E, generator=g) * 3
    chosen = torch.zeros(n, top, dtype=torch.int32, device="cuda")
    weights = torch.zeros(n, top, device="cuda")
    ops.router_topk(chosen, weights, logits.cuda(), top)
    vals, idx = torch.topk(logits, top, dim=-1)
    assert torch.equal(chosen.cpu().long(), idx)
    assert np.allclose(weights.cpu().numpy(), torch.sigmoid(vals).numpy(), rtol=1e-6)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_experts_without_a_gate(dtype):
    """Row by row in both dtypes and, in bfloat16, grouped on the matrix cores (experts with no token, with more
    than a tile of them); the weight stands on the input."""
    from hfee_amd.kernels import ops
    dt = DT[dtype]
    g = torch.Generator().manual_seed(6)
    n, top, E, Fd, width = 300, 2, 5, 96, 64
    h = torch.randn(n, width, generator=g).to(dt)
    wu, wd = (torch.randn(E, Fd, width, generator=g) * 0.2).to(dt), (torch.randn(E, width, Fd, generator=g) * 0.2).to(dt)
    chosen = torch.stack([torch.randperm(E - 1, generator=g)[:top] for _ in range(n)]).int()       # (expert 4 has no token)
    weights = torch.rand(n, top, generator=g) + 0.2
    want = torch.zeros(n, width, dtype=torch.float64)
    for t in range(n):
        for j in range(top):
            e = int(chosen[t, j])
            want[t] += wd[e].double() @ torch.relu(wu[e].double() @ (weights[t, j].double() * h[t].double())) ** 2
    act = torch.zeros(n * top, Fd, dtype=dt, device="cuda")
    out = torch.full((n, width), 7.0, device="cuda")
    ops.moe_up(act, h.cuda(), None, wu.cuda(), top, chosen=chosen.cuda(), in_weights=weights.cuda())
    ops.moe_down(out, act, wd.cuda(), top, weight=1.0, chosen=chosen.cuda(), accumulate=False)
    assert ru.rel(out.double().cpu(), want) < (2e-5 if dtype == "float32" else 2e-2)
    if dtype == "bfloat16":
        grouped = torch.zeros(n, width, device="cuda")
        order = torch.zeros(n * top, dtype=torch.int32, device="cuda")
        tiles = torch.zeros(3 * ops.moe_group_tiles(n, top, E) + 1, dtype=torch.int32, device="cuda")
        y = torch.zeros(n * top, width, device="cuda")
        ops.moe_grouped(grouped, h.cuda(), None, wu.cuda(), wd.cuda(), top, order, tiles, act, y, weight=1.0,
                        chosen=chosen.cuda(), in_weights=weights.cuda())
        assert ru.rel(grouped.double().cpu(), want) < 2e-2


# ------------------------------------------------------------------ the whole model

@pytest.fixture(scope="module")
def folders(tmp_path_factory):
    base = tmp_path_factory.mktemp("ronavik")
    return {(name, dtype): ru.make_folder(base / f"{name.replace(' ', '_')}_{dtype}", cj, seed=7 + ord(name[0]), dtype=dtype)
            for name, cj in list(ru.CONFIGS.items()) + list(ru.SINGLE.items()) for dtype in ("float32", "bfloat16")}


def plain_logits(folder, tokens, margins=None):
    """The plain implementation's logits; margins: a list that receives, a position, the smallest margin by
    which any of its routers chose."""
    cj, w = ru.load_plain(folder)
    each = []
    logits = pr.forward(cj, w, tokens, dtype=torch.float64, margins_out=each).numpy()
    if margins is not None:
        margins.extend(torch.stack(each).min(0).values.tolist() if each else [float("inf")] * len(tokens))
    return logits


# In bfloat16 a router reads rounded numbers: a token whose last chosen expert and the best one not chosen
# score almost alike may go to the other one.  Its sub-layer's result is normed, so that is a change as large
# as the stream itself, and the states and the cache carry it to every token behind it.  So in bfloat16 a
# request is compared up to the first position at which a router of the plain implementation chose by less
# than NEAR_TIE of its logits' spread (a few positions in a hundred), and the configurations in which every
# token uses every expert ("... every expert": nothing is chosen) are compared at every position.
NEAR_TIE = 0.05


class Rows(dict):
    """(request, position) -> logits of the plain implementation; `.margins`: -> the routers' smallest margin."""
    margins: dict


@pytest.fixture(scope="module")
def plain_rows(folders):
    cache = {}

    def get(name, dtype, lengths=None):
        key = (name, dtype, tuple(lengths or LENGTHS[name[0]]))
        if key not in cache:
            cj = (ru.CONFIGS.get(name) or ru.SINGLE[name])
            reqs = tu.make_requests(cj["vocab"], list(key[2]), seed=ord(name[0]))
            rows = Rows()
            rows.margins = {}
            for rid, toks in reqs.items():
                margins = []
                logits = plain_logits(folders[(name, dtype)], toks, margins)
                rows.update({(rid, i): logits[i] for i in range(len(toks))})
                rows.margins.update({(rid, i): margins[i] for i in range(len(toks))})
            cache[key] = (reqs, rows)
        return cache[key]
    return get


def compare(got, want, dtype, what, margins=None):
    """32-bit: every position within the tolerance.  bfloat16: every position before its request's first near
    tie (see NEAR_TIE) within twice the tolerance and all but one in two hundred of them within it (rounding
    has outliers where a row of logits is small); over all positions, also those behind a near tie, the
    median is well within it."""
    assert set(got) == set(want), f"{what}: positions differ"
    tol = TOL[dtype]
    margins = margins if margins is not None else getattr(want, "margins", {})
    errors = {key: ru.rel(got[key], want[key]) for key in want}
    keys = sorted(want)
    if dtype != "float32":
        first_tie = {}
        for rid, at in keys:
            if margins.get((rid, at), float("inf")) < NEAR_TIE:
                first_tie[rid] = min(at, first_tie.get(rid, at))
        keys = [(rid, at) for rid, at in keys if at < first_tie.get(rid, at + 1)]
    over = sorted((errors[key], key) for key in keys if not errors[key] < tol)
    allowed = 0 if dtype == "float32" else len(keys) // 200
    assert len(over) <= allowed and not any(e >= 2 * tol for e, _ in over), \
        f"{what}: {len(over)} of {len(keys)} positions beyond {tol}, the worst {over[-1]}, the first {min(k for _, k in over)}"
    assert np.median(list(errors.values())) < tol / 2, f"{what}: median relative error {np.median(list(errors.values())):.3e}"


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", sorted(ru.SINGLE))
def test_each_mechanism_as_a_model_of_one_layer(folders, plain_rows, name, dtype):
    from hfee_amd.trace_replay import Replayer
    reqs, want = plain_rows(name, dtype, [37, 2, 11])
    for what, steps in (("whole", tu.whole(reqs)), ("bulk then single tokens", tu.bulk_then_tail(reqs, 9)),
                        ("portions", tu.portions(reqs, sizes=(2, 5, 3, 2, 7)))):
        rep = Replayer(folders[(name, dtype)], dtype, 64, max_requests=2)
        compare(tu.run(rep, steps), want, dtype, f"{name} {dtype} {what}")


@pytest.mark.parametrize("name,dtype", [(n, d) for n in ("A", "B", "C", "D") for d in ("float32", "bfloat16")]
                         + [("A every expert", "bfloat16"), ("D every expert", "bfloat16")])
def test_every_way_of_cutting_gives_the_plain_logits(folders, plain_rows, name, dtype):
    from hfee_amd.trace_replay import Replayer
    reqs, want = plain_rows(name, dtype)
    longest = max(len(t) for t in reqs.values())
    one = (longest + 63) // 64 * 64
    for what, steps, room in (("whole", tu.whole(reqs), one), ("bulk then single tokens", tu.bulk_then_tail(reqs, 40), one),
                              ("portions", tu.portions(reqs), one), ("mixed", *tu.mixed(reqs, seed=len(name[0])))):
        rep = Replayer(folders[(name, dtype)], dtype, room, max_requests=4)
        got = tu.run(rep, steps)
        compare(got, want, dtype, f"{name} {dtype} {what}")
        rep.engine.cache.check()
        assert not rep.engine.cache.requests


def test_cuts_agree_closely_in_32_bit(folders, plain_rows):
    """Whole prompts against portions and single tokens: rounding apart, the same logits."""
    from hfee_amd.trace_replay import Replayer
    reqs, _ = plain_rows("A", "float32")
    runs = []
    for steps in (tu.whole(reqs), tu.portions(reqs, sizes=(2, 3, 16, 1, 15, 17, 2)), tu.bulk_then_tail(reqs, 20)):
        runs.append(tu.run(Replayer(folders[("A", "float32")], "float32", 192, max_requests=4), steps))
    for other in runs[1:]:
        for key in runs[0]:
            assert ru.rel(other[key], runs[0][key]) < 3e-6


@pytest.mark.parametrize("name", ["A", "C"])
def test_a_slot_that_is_used_again_starts_from_nothing(folders, plain_rows, name):
    """One state slot and a pool of one request's pages: every request inherits the slot and the pages of
    the one before, whose states and convolution inputs must be gone."""
    from hfee_amd.trace_replay import Replayer
    reqs, want = plain_rows(name, "float32")
    longest = max(len(t) for t in reqs.values())
    rep = Replayer(folders[(name, "float32")], "float32", (longest + 63) // 64 * 64, max_requests=1)
    got = tu.run(rep, tu.portions(reqs, sizes=(9, 2, 30)))
    compare(got, want, "float32", f"{name}: one slot for all")


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_long_decoding(folders, dtype):
    """300 single tokens after a short prompt: decode steps replayed from captured graphs, across page
    borders and several steps of the temperature, the states carried through every replay."""
    from hfee_amd.trace_replay import Replayer
    rng = np.random.default_rng(9)
    toks = rng.integers(0, 500, size=330).tolist()
    name = "D" if dtype == "float32" else "D every expert"      # (in bfloat16 no near tie of a router on the way)
    rep = Replayer(folders[(name, dtype)], dtype, 384, max_requests=4)
    steps = [{"entries": [("a", toks[:30], [29])], "end": []}]
    steps += [{"entries": [("a", toks[i:i + 1], [0])], "end": ["a"] if i == 329 else []} for i in range(30, 330)]
    got = tu.run(rep, steps)
    assert rep.engine.graph_replays > 250
    margins = []
    want = plain_logits(folders[(name, dtype)], toks, margins)
    compare(got, {("a", i): want[i] for i in range(29, 330)}, dtype, f"long decoding {dtype}",
            {("a", i): m for i, m in enumerate(margins)})


def test_a_far_token_shows_through_attention_alone(folders):
    """Two sequences that differ in their first token only: 100 tokens later the engine's logits differ by what
    the plain implementation says, in a model whose only path back is the attention (the unit's scale is 0)."""
    from hfee_amd.trace_replay import Replayer
    folder = folders[("sigmoid attention", "float32")]
    toks = tu.make_requests(50, [101], seed=3)["r0"]
    other = [(toks[0] + 7) % 50] + toks[1:]
    rep = Replayer(folder, "float32", 256, max_requests=2)
    got = tu.run(rep, [{"entries": [("a", toks[:60], []), ("b", other[:60], [])], "end": []},
                       {"entries": [("b", other[60:], [40]), ("a", toks[60:], [40])], "end": ["a", "b"]}])
    want = plain_logits(folder, toks)[100] - plain_logits(folder, other)[100]
    assert np.abs(want).max() > 1e-6
    assert ru.rel(got[("a", 100)] - got[("b", 100)], want) < 1e-2


def greedy(folder, prompt, count):
    seq = list(prompt)
    for _ in range(count):
        seq.append(int(np.argmax(plain_logits(folder, seq)[-1])))
    return seq[len(prompt):]


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_greedy_generation_through_the_entry_point(folders, dtype):
    from hfee_amd import LLM, SamplingParams
    folder = folders[("A" if dtype == "float32" else "A every expert", dtype)]      # (no router's near tie in bfloat16)
    llm = LLM(folder, dtype=dtype, num_ctx=128, num_parallel=3, max_batch_tokens=24)
    g = np.random.default_rng(5)
    prompts = [g.integers(0, 131, size=n).tolist() for n in (5, 40, 1, 17, 33)]
    outs = llm.generate(prompts, SamplingParams.greedy(num_predict=8))
    for p, o in zip(prompts, outs):
        want = greedy(folder, p, 8)
        if dtype == "float32":
            assert o.token_ids == want
        else:
            logits = plain_logits(folder, p + want)
            margins = []
            for i in range(8):
                row = np.sort(logits[len(p) - 1 + i])
                margins.append(float((row[-1] - row[-2]) / np.abs(row).max()))
            tu.agree_until_a_near_tie(o.token_ids, want, margins, f"greedy {dtype}")


def test_trace_runner_as_a_subprocess(folders, tmp_path):
    folder = folders[("B", "float32")]
    toks = list(range(1, 40))
    lines = [{"step": 0, "entries": [{"id": "x", "tokens": toks[:21], "want": [0, 20]}], "end": []},
             {"step": 1, "entries": [{"id": "x", "tokens": toks[21:22], "want": []}], "end": []},
             {"step": 2, "entries": [{"id": "x", "tokens": toks[22:], "want": [16]}, {"id": "y", "tokens": toks[:2], "want": [1]}],
              "end": ["x", "y"]}]
    out = tmp_path / "out"
    p = subprocess.run([sys.executable, os.path.join(ROOT, "bin", "trace_run"), "--model", folder, "--dtype", "float32",
                        "--out", str(out), "--max-tokens", "128"], input="\n".join(json.dumps(l) for l in lines) + "\n",
                       capture_output=True, text=True, timeout=600)
    assert p.returncode == 0, p.stderr[-2000:]
    assert [l for l in p.stdout.splitlines() if l.startswith("done")] == ["done 0", "done 1", "done 2"]
    want = plain_logits(folder, toks)
    a = np.fromfile(out / "0.f32", dtype="<f4").reshape(2, -1)
    c = np.fromfile(out / "2.f32", dtype="<f4").reshape(2, -1)
    assert not (out / "1.f32").exists()
    assert ru.rel(a[0], want[0]) < 3e-5 and ru.rel(a[1], want[20]) < 3e-5
    assert ru.rel(c[0], want[38]) < 3e-5 and ru.rel(c[1], want[1]) < 3e-5


def test_the_command_line_runs_the_design(folders):
    """`hfee run <folder> --tokens ...`: the greedy continuation's ids."""
    folder = folders[("B", "float32")]
    prompt = tu.make_requests(97, [11], seed=8)["r0"]
    want = greedy(folder, prompt, 7)
    p = subprocess.run([sys.executable, os.path.join(ROOT, "bin", "hfee"), "run", folder, "--tokens",
                        ",".join(map(str, prompt)), "--dtype", "float32", "--temperature", "0", "--repeat-penalty", "1",
                        "--num-predict", "7", "--num-ctx", "128", "--verbose"],
                       capture_output=True, text=True, timeout=300, stdin=subprocess.DEVNULL)
    assert p.returncode == 0, p.stderr[-2000:]
    assert [int(t) for t in p.stdout.strip().splitlines()[0].split()] == want
