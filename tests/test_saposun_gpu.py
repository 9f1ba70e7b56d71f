"""The Saposun decoder on the GPU against the plain implementation: the new kernels alone (attention over a
window with pooled blocks, a cap and a gate, with keys that stand out just inside and just outside the window,
inside a block that is seen and one that is not yet, far back and at page borders, in prompts and token by
token; the rotation and value norm on the way into the cache; the pooled means; the rotation in float32; the
retention in portions over slots; the router with a softmax and a correction; gated routed experts), each
mechanism as a model of one layer, the whole model under four ways of cutting the same requests into steps
(whole, bulk then single tokens, portions down to two tokens, mixed batches on a small page pool with four state
slots, pages and slots used again), in 32-bit and in bfloat16, on configurations with even and with odd sizes and
on one without any attention; long decoding through graph replays; greedy generation through the entry point and
its scheduler; the trace runner and the command line as subprocesses."""
import json
import os
import subprocess
import sys

import numpy as np
import pytest
import torch

import plain_saposun as ps
import saposun_util as su
import trace_util as tu
from conftest import ROOT

pytestmark = pytest.mark.gpu

TOL = {"float32": 3e-5, "bfloat16": 8e-2}
DT = {"float32": torch.float32, "bfloat16": torch.bfloat16}
LENGTHS = {"A": [5, 17, 64, 1, 100, 33, 129, 49, 2], "B": [40, 3, 100, 65, 2, 31], "C": [90, 3, 41, 1, 130],
           "D": [700, 47, 313, 1, 161]}


def i32(a):
    return torch.as_tensor(np.asarray(a, dtype=np.int32)).cuda()


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


# ------------------------------------------------------------------ kernels alone

def windowed_definition(q, k, v, gate, scale, window, pool, cap):
    """q [n, H, dk], k [n, G, dk], v [n, G, dv] (as the cache holds them), gate [n, H] or None, float64."""
    n, H, _ = q.shape
    G = k.shape[1]
    out = torch.zeros(n, H, v.shape[2], dtype=torch.float64)
    for i in range(n):
        first = max(0, i - window + 1) if window else 0
        keys, values = [k[first:i + 1]], [v[first:i + 1]]
        if pool and window:
            for b in range(n // pool):
                if b * pool + pool - 1 <= i - window:
                    keys.append(k[b * pool:(b + 1) * pool].mean(0, keepdim=True))
                    values.append(v[b * pool:(b + 1) * pool].mean(0, keepdim=True))
        kk, vv = torch.cat(keys), torch.cat(values)
        for h in range(H):
            s = (kk[:, h // (H // G)] @ q[i, h]) * scale
            if cap:
                s = cap * torch.tanh(s / cap)
            out[i, h] = torch.softmax(s, 0) @ vv[:, h // (H // G)]
    if gate is not None:
        out = out * torch.sigmoid(gate)[:, :, None]
    return out.reshape(n, -1)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("H,G,dk,dv,window,pool,cap,gated", [
    (4, 2, 32, 16, 19, 5, 4.0, True), (3, 3, 10, 12, 7, 1, 0.0, False), (8, 2, 64, 64, 100, 7, 20.0, True),
    (2, 1, 16, 48, 5, 11, 0.0, True), (6, 2, 80, 64, 45, 9, 25.0, True), (4, 4, 32, 32, 33, 0, 0.0, False),
    (4, 1, 96, 64, 0, 0, 0.0, False), (8, 2, 32, 32, 50, 0, 0.0, False), (16, 1, 48, 32, 21, 0, 0.0, False)])
def test_attention_over_a_window_with_pooled_blocks(dtype, H, G, dk, dv, window, pool, cap, gated):
    """Two sequences side by side, written in portions whose edges fall inside pages, windows and blocks, read
    by portions and by single tokens (plain, and where the sizes allow on the matrix cores, the single tokens'
    keys whole and split).  Keys are made to stand out for the last query of the long sequence's head 1: the
    first key of its window, the key just before it (which nobody may see as a token), a key in the newest
    block that is seen and one in the first block that is not yet, a key far back, and the keys on both sides of
    a page border; every position's result is compared with the definition, so a window or a block that is one
    token off shows at its edge."""
    from hfee_amd.kernels import ops
    dt = DT[dtype]
    g = torch.Generator().manual_seed(dk + H + window)
    lengths, scale = [333, 37], 0.25
    qs = [torch.randn(n, H, dk, generator=g) for n in lengths]
    ks = [torch.randn(n, G, dk, generator=g) for n in lengths]
    vs = [torch.randn(n, G, dv, generator=g) for n in lengths]
    gates = [torch.randn(n, H, generator=g) for n in lengths] if gated else [None, None]
    last, kv1 = lengths[0] - 1, 1 // (H // G)
    standouts = [3, 15, 16]
    if window:
        standouts += [last - window + 1, last - window]
        if pool:
            seen = (last - window + 1) // pool             # blocks 0 .. seen - 1 are seen by the last query
            standouts += [seen * pool - 1, seen * pool + (1 if pool > 1 else 0)]
    # every one of them in turn is what some query near the end looks at hardest
    for n_back, j in enumerate(standouts):
        if 0 <= j < lengths[0]:
            ks[0][j, kv1] = qs[0][last - n_back % 3, 1] * 3.0
    qs, ks, vs = ([t.to(dt).float() for t in x] for x in (qs, ks, vs))
    gates = [None if t is None else t.to(dt).float() for t in gates]
    pooling = bool(pool and window)
    tables, pages = _paged(lengths)
    cache = torch.zeros(pages, G, 16 * (dk + dv), dtype=dt, device="cuda")
    cache[0].fill_(float("nan"))
    bt = i32(tables)
    matrix = dtype == "bfloat16" and ops.attention_kv_sizes_fit(dk, dv)
    sight = dict(window=window, pool=pool if window else 0, softcap=cap)
    if pooling:        # the pooled blocks: a cache layer of their own that grows by an entry every `pool` tokens
        pool_tables, pool_pages = _paged([-(-n // pool) for n in lengths], seed=1)
        pooled = torch.zeros(pool_pages, G, 16 * (dk + dv), dtype=dt, device="cuda")
        pooled[0].fill_(float("nan"))
        pbt = i32(pool_tables)
    # the values as the cache holds them: normed a head, rounded
    eps = 1e-5
    vn = [(v.double() / torch.sqrt((v.double() ** 2).mean(-1, keepdim=True) + eps)).to(dt).double() for v in vs]
    want = [windowed_definition(q.double(), k.double(), v, None if gt is None else gt.double(), scale, window, pool, cap)
            for q, k, v, gt in zip(qs, ks, vn, gates)]
    fed = [0, 0]
    for sizes in ([7, 2], [9, 0], [150, 17], [140, 16], [1, 1], [5, 1], [1, 0], [20, 0]):
        segs = [(s, n) for s, n in enumerate(sizes) if n]
        n_all = sum(n for _, n in segs)
        cat = lambda xs: torch.cat([xs[s][fed[s]:fed[s] + n].reshape(n, -1) for s, n in segs])      # noqa: E731
        q32, k32, v32 = cat(qs).cuda(), cat(ks).cuda(), cat(vs).cuda()
        gate = cat(gates).to(dt).cuda() if gated else None
        positions = i32(np.concatenate([np.arange(fed[s], fed[s] + n) for s, n in segs]))
        token_segment = i32(np.concatenate([np.full(n, i) for i, (_, n) in enumerate(segs)]))
        tab = bt[[s for s, _ in segs]].contiguous()
        q = torch.zeros(n_all, H * dk, dtype=dt, device="cuda")
        ops.rotate_norm_write(q, q32, k32, v32, positions, token_segment, tab, None, None, cache, H, G, dk, dv, 16,
                              int(positions.max()), value_eps=eps)
        if pooling:
            sight.update(pooled=pooled, pool_tables=pbt[[s for s, _ in segs]].contiguous())
            ops.kv_pool_write(cache, pooled, pool, positions, token_segment, tab, sight["pool_tables"], G, dk, dv, 16)
        out = torch.zeros(n_all, H * dv, dtype=dt, device="cuda")
        ops.attention_kv_plain(out, q, cache, positions, token_segment, tab, H, G, dk, dv, 16, scale, gate=gate, **sight)
        outs = [out]
        if matrix:
            rows_most = ops.attention_kv_rows(dk, dv, H // G, "softmax")
            portions, singles, row = [], [], 0
            for i, (s, n) in enumerate(segs):
                if n > 1:
                    portions += [(row + o, min(rows_most, n - o), fed[s] + o, i) for o in range(0, n, rows_most)]
                else:
                    singles.append((row, 1, fed[s], i))
                row += n
            out2 = torch.zeros(n_all, H * dv, dtype=dt, device="cuda")
            if portions:
                ops.attention_kv_bf16(out2, q, cache, i32(portions).reshape(-1, 4), 0, tab, H, G, dk, dv, 16, scale, gate=gate, **sight)
            if singles:
                for splits in (1, 3):
                    partial = torch.zeros(ops.attention_kv_partial_words(len(singles), H, dv, splits) + 1, device="cuda")
                    ops.attention_kv_bf16(out2, q, cache, i32(singles).reshape(-1, 4), 1, tab, H, G, dk, dv, 16, scale,
                                          partial=partial if splits > 1 else None, splits=splits, gate=gate, **sight)
                    if splits == 1:
                        first = out2.clone()
                    else:
                        rows_single = [r for r, _, _, _ in singles]
                        assert su.rel(out2[rows_single].float().cpu(), first[rows_single].float().cpu()) < 2e-2
            outs.append(out2)
        row = 0
        for s, n in segs:
            for o in outs:
                w = want[s][fed[s]:fed[s] + n]
                err = (o[row:row + n].double().cpu() - w).abs().max() / w.abs().max()
                assert err < (2e-5 if dtype == "float32" else 3e-2), (sizes, s, float(err))
            fed[s] += n
            row += n
    assert fed == lengths
    assert torch.isnan(cache[0].float()).all() and (not pooling or torch.isnan(pooled[0].float()).all())


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_rotation_and_value_norm_on_the_way_into_the_cache(dtype):
    from hfee_amd.kernels import ops
    dt = DT[dtype]
    H, G, dk, dv, rot, n = 4, 2, 12, 10, 8, 21
    g = torch.Generator().manual_seed(2)
    q, k, v = torch.randn(n, H * dk, generator=g), torch.randn(n, G * dk, generator=g), torch.randn(n, G * dv, generator=g)
    start = 5
    pos = torch.arange(start, start + n)
    a = ps.angles(pos, rot, 300.0)
    cos, sin = torch.cos(a).float().cuda(), torch.sin(a).float().cuda()
    table_cos = torch.zeros(start + n, rot // 2, device="cuda")
    table_sin = torch.zeros(start + n, rot // 2, device="cuda")
    table_cos[start:], table_sin[start:] = cos, sin
    tables, pages = _paged([start + n])
    cache = torch.zeros(pages, G, 16 * (dk + dv), dtype=dt, device="cuda")
    q_out = torch.zeros(n, H * dk, dtype=dt, device="cuda")
    ops.rotate_norm_write(q_out, q.cuda(), k.cuda(), v.cuda(), i32(pos), i32(np.zeros(n)), i32(tables), table_cos, table_sin,
                          cache, H, G, dk, dv, 16, start + n - 1, value_eps=1e-3)
    want_q = ps.rotate_half(q.double().view(n, H, dk), pos, rot, 300.0).reshape(n, -1)
    want_k = ps.rotate_half(k.double().view(n, G, dk), pos, rot, 300.0)
    want_v = ps.rms(v.double().view(n, G, dv), 1e-3)
    tol = 1e-6 if dtype == "float32" else 1e-2
    assert su.rel(q_out.double().cpu(), want_q) < tol
    pages_of = cache.double().cpu()
    for t in range(n):
        p = start + t
        page, slot = tables[0, p // 16], p % 16
        keys = pages_of[page, :, :16 * dk].view(G, 16, dk)[:, slot]
        values = pages_of[page, :, 16 * dk:].view(G, dv, 16)[:, :, slot]
        assert su.rel(keys, want_k[t]) < tol and su.rel(values, want_v[t]) < tol


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_rotation_in_32_bit_on_the_way_into_a_recurrence(dtype):
    from hfee_amd.kernels import ops
    dt = DT[dtype]
    H, D, rot, n = 3, 10, 6, 40
    g = torch.Generator().manual_seed(3)
    x = torch.randn(n, 2 * H * D, generator=g).to(dt)
    pos = torch.arange(100, 100 + n)
    a = ps.angles(torch.arange(100 + n), rot, 1000.0)
    out = torch.zeros(n, 2 * H * D, device="cuda")
    ops.rotate_rows(out, x.cuda(), i32(pos), torch.cos(a).float().cuda(), torch.sin(a).float().cuda(), 2 * H, D, 100 + n - 1,
                    scaled_from=H, factor=D ** -0.5)
    want = ps.rotate_half(x.double().view(n, 2 * H, D), pos, rot, 1000.0)
    want[:, H:] *= D ** -0.5
    assert su.rel(out.double().cpu(), want.reshape(n, -1)) < 2e-6
    plain = torch.zeros(n, 2 * H * D, device="cuda")
    ops.rotate_rows(plain, x.cuda(), i32(pos), None, None, 2 * H, D, 0)
    assert torch.equal(plain.cpu(), x.float())


@pytest.mark.parametrize("H,D,V", [(2, 16, 32), (3, 12, 20), (4, 32, 64), (1, 4, 4)])
def test_retention_in_portions(H, D, V):
    """Two requests in other slots, in portions of unequal size, against the closed form
    o_t = sum_j decay^(t - j) (q_t . k_j) v_j; a slot of NaNs beside them stays untouched."""
    from hfee_amd.kernels import ops
    g = torch.Generator().manual_seed(H + D)
    lengths, slots = [70, 23], [2, 0]
    decay = torch.tensor([1.0, 0.9, 0.5, 0.99][:H])
    qs = [torch.randn(n, H, D, generator=g) for n in lengths]
    ks = [torch.randn(n, H, D, generator=g) * D ** -0.5 for n in lengths]
    vs = [torch.randn(n, H, V, generator=g) for n in lengths]
    want = []
    for q, k, v in zip(qs, ks, vs):
        n = q.shape[0]
        t = torch.arange(n)
        power = (t[:, None] - t[None, :]).clamp(min=0).double()
        w = torch.einsum("ihd,jhd->hij", q.double(), k.double()) * decay.double()[:, None, None] ** power[None]
        w = w * (t[None, :] <= t[:, None])
        want.append(torch.einsum("hij,jhv->ihv", w, v.double()).reshape(n, -1))
    state = torch.zeros(4, H, *ops.scan_state_shape(D, V), device="cuda")
    state[1].fill_(float("nan"))
    fed = [0, 0]
    for sizes in ([5, 2], [1, 1], [40, 0], [2, 17], [22, 3]):
        segs = [(s, n) for s, n in enumerate(sizes) if n]
        cat = lambda xs: torch.cat([xs[s][fed[s]:fed[s] + n].reshape(n, -1) for s, n in segs]).cuda()      # noqa: E731
        q, k, v = cat(qs), cat(ks), cat(vs)
        rows = np.cumsum([0] + [n for _, n in segs])[:-1]
        out = torch.zeros(q.shape[0], H * V, device="cuda")
        ops.linear_scan(out, state, q, k, v, decay.cuda(), None, i32(rows), i32([n for _, n in segs]), i32([slots[s] for s, _ in segs]),
                        H, H, D, V, "decay_add", decay_per_head=True)
        row = 0
        for s, n in segs:
            assert su.rel(out[row:row + n].double().cpu(), want[s][fed[s]:fed[s] + n]) < 2e-5, (sizes, s)
            fed[s] += n
            row += n
    assert fed == lengths and torch.isnan(state[1]).all() and torch.isfinite(state[[0, 2, 3]]).all()


@pytest.mark.parametrize("n,E,top", [(50, 5, 2), (7, 70, 3), (33, 4, 4), (9, 130, 1), (20, 16, 3)])
def test_the_router_adds_its_correction_to_the_choice_only(n, E, top):
    from hfee_amd.kernels import ops
    g = torch.Generator().manual_seed(n + E)
    logits = torch.randn(n, E, generator=g)
    correction = torch.randn(E, generator=g) * 0.1
    scores = torch.softmax(logits.double(), -1)
    for corr in (correction, None):
        chosen = torch.zeros(n, top, dtype=torch.int32, device="cuda")
        weights = torch.zeros(n, top, device="cuda")
        ops.router_topk(chosen, weights, logits.cuda(), top, score="softmax", correction=None if corr is None else corr.cuda())
        choice = scores + (0 if corr is None else corr.double())
        want = torch.sort(choice, dim=-1, descending=True, stable=True).indices[:, :top]
        assert torch.equal(chosen.cpu().long(), want)
        assert su.rel(weights.double().cpu(), torch.gather(scores, 1, want)) < 1e-6
    # a correction large enough to turn a choice round, and the weight of the expert it brings in
    big = torch.zeros(E)
    big[E - 1] = 10.0
    chosen = torch.zeros(n, top, dtype=torch.int32, device="cuda")
    weights = torch.zeros(n, top, device="cuda")
    ops.router_topk(chosen, weights, logits.cuda(), top, score="softmax", correction=big.cuda())
    assert (chosen[:, 0] == E - 1).all()
    assert su.rel(weights[:, 0].double().cpu(), scores[:, E - 1]) < 1e-6


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("n,width", [(8, 4096), (100, 72), (3, 5000), (70, 1024), (1, 58)])
def test_the_scaled_sum_with_the_next_norm(dtype, n, width):
    from hfee_amd.kernels import ops
    g = torch.Generator().manual_seed(n + width)
    x, y, w = torch.randn(n, width, generator=g), torch.randn(n, width, generator=g), torch.rand(width, generator=g) + 0.5
    got_x, nxt = x.clone().cuda(), torch.zeros(n, width, dtype=DT[dtype], device="cuda")
    ops.scaled_add_norm(got_x, y.cuda(), 0.3, nxt, w.cuda(), 1e-5)
    want_x = x.double() + 0.3 * y.double()
    assert su.rel(got_x.double().cpu(), want_x) < 1e-6
    assert su.rel(nxt.double().cpu(), ps.rms_norm(want_x, w.double(), 1e-5)) < (2e-6 if dtype == "float32" else 1e-2)


# ------------------------------------------------------------------ the whole model

@pytest.fixture(scope="module")
def folders(tmp_path_factory):
    base = tmp_path_factory.mktemp("saposun")
    return {(name, dtype): su.make_folder(base / f"{name.replace(' ', '_')}_{dtype}", cj, seed=7 + ord(name[0]), dtype=dtype)
            for name, cj in list(su.CONFIGS.items()) + list(su.SINGLE.items()) for dtype in ("float32", "bfloat16")}


def plain_logits(folder, tokens, margins=None):
    """The plain implementation's logits; margins: a list that receives, a position, the smallest margin by
    which any of its routers chose."""
    cj, w = su.load_plain(folder)
    each = []
    logits = ps.forward(tokens, w, cj, margins=each).numpy()
    if margins is not None:
        margins.extend(torch.stack(each).min(0).values.tolist() if each else [float("inf")] * len(tokens))
    return logits


# In bfloat16 a router reads rounded numbers: a token whose last chosen expert and the best one not chosen score
# almost alike may go to the other one, and the states and the cache carry the difference to every token behind
# it.  So in bfloat16 a request is compared up to the first position at which a router of the plain
# implementation chose by less than NEAR_TIE, and the configurations in which every token uses every expert
# ("... every expert": nothing is chosen) are compared at every position.
NEAR_TIE = 0.02


class Rows(dict):
    """(request, position) -> logits of the plain implementation; `.margins`: -> the routers' smallest margin."""
    margins: dict


@pytest.fixture(scope="module")
def plain_rows(folders):
    cache = {}

    def get(name, dtype, lengths=None):
        key = (name, dtype, tuple(lengths or LENGTHS[name[0]]))
        if key not in cache:
            cj = (su.CONFIGS.get(name) or su.SINGLE[name])
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
    tie (see NEAR_TIE) within twice the tolerance and all but one in a hundred of them (or one) within it: a head of
    the retention whose sum is small is divided by a small root mean square, which makes rounding show; over all
    positions the median is well within it."""
    assert set(got) == set(want), f"{what}: positions differ"
    tol = TOL[dtype]
    margins = margins if margins is not None else getattr(want, "margins", {})
    errors = {key: su.rel(got[key], want[key]) for key in want}
    keys = sorted(want)
    if dtype != "float32":
        first_tie = {}
        for rid, at in keys:
            if margins.get((rid, at), float("inf")) < NEAR_TIE:
                first_tie[rid] = min(at, first_tie.get(rid, at))
        keys = [(rid, at) for rid, at in keys if at < first_tie.get(rid, at + 1)]
    over = sorted((errors[key], key) for key in keys if not errors[key] < tol)
    allowed = 0 if dtype == "float32" else max(1, len(keys) // 100)
    assert len(over) <= allowed and not any(e >= 2 * tol for e, _ in over), \
        f"{what}: {len(over)} of {len(keys)} positions beyond {tol}, the worst {over[-1]}, the first {min(k for _, k in over)}"
    assert np.median(list(errors.values())) < tol / 2, f"{what}: median relative error {np.median(list(errors.values())):.3e}"


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", sorted(su.SINGLE))
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
    """Whole prompts against portions and single tokens: rounding apart, the same logits (the per-head products of
    the latent layers add in another order from 32 rows on, and the recurrence's heads are divided by their root
    mean square, which a small sum makes small)."""
    from hfee_amd.trace_replay import Replayer
    reqs, _ = plain_rows("A", "float32")
    runs = []
    for steps in (tu.whole(reqs), tu.portions(reqs, sizes=(2, 3, 16, 1, 15, 17, 2)), tu.bulk_then_tail(reqs, 20)):
        runs.append(tu.run(Replayer(folders[("A", "float32")], "float32", 192, max_requests=4), steps))
    for other in runs[1:]:
        for key in runs[0]:
            assert su.rel(other[key], runs[0][key]) < 1e-5


@pytest.mark.parametrize("name", ["A", "C"])
def test_a_slot_that_is_used_again_starts_from_nothing(folders, plain_rows, name):
    """One state slot and a pool of one request's pages: every request inherits the slot and the pages of the
    one before, whose states, convolution inputs and pooled blocks must be gone."""
    from hfee_amd.trace_replay import Replayer
    reqs, want = plain_rows(name, "float32")
    longest = max(len(t) for t in reqs.values())
    rep = Replayer(folders[(name, "float32")], "float32", (longest + 63) // 64 * 64, max_requests=1)
    got = tu.run(rep, tu.portions(reqs, sizes=(9, 2, 30)))
    compare(got, want, "float32", f"{name}: one slot for all")


def test_the_pooled_blocks_take_a_page_every_so_many_tokens(folders, plain_rows):
    """The attention layer's pooled blocks are a cache group that grows by an entry every `pool` tokens: a request
    of 150 tokens with blocks of 3 holds 50 entries of it, four pages; its tokens are a window group that keeps the
    window's pages only."""
    from hfee_amd.trace_replay import Replayer
    reqs, want = plain_rows("attention", "float32", [150])
    rep = Replayer(folders[("attention", "float32")], "float32", 192, max_requests=2)
    groups = rep.engine.cache.groups
    assert sorted((g.every, g.kind, g.window, g.cache_layers) for g in groups) == [(1, "window", 10, (0,)), (3, "full", 0, ((0, 1),))]
    rows = rep.step([("r0", reqs["r0"], list(range(150)))])
    held = {groups[g].every: sum(p >= 0 for p in t) for g, t in enumerate(rep.engine.cache.get("r0").tables)}
    assert held == {1: 2, 3: 4}            # (the next query reads the positions from 141 on: the ninth and tenth page)
    compare({("r0", i): rows[i] for i in range(150)}, want, "float32", "a group that grows every third token")
    rep.engine.release("r0")
    rep.engine.cache.check()


def test_a_window_gives_back_the_pages_it_has_passed(folders, plain_rows):
    """The latent layers' cache is a window group of the manager: a request of 150 tokens holds the pages of its
    widest window and no more, whether it came in portions or token by token, and its logits are the plain ones."""
    from hfee_amd.trace_replay import Replayer
    reqs, want = plain_rows("latent", "float32", [150])
    toks = reqs["r0"]
    rep = Replayer(folders[("latent", "float32")], "float32", 192, max_requests=2)
    groups = rep.engine.cache.groups
    assert [g.kind for g in groups] == ["window"] and groups[0].window == 6
    got, fed = {}, 0
    for n in [40, 3, 2, 50] + [1] * 55:
        rows = rep.step([("r0", toks[fed:fed + n], list(range(n)))])
        got.update({("r0", fed + i): rows[i] for i in range(n)})
        fed += n
        held = [p for p in rep.engine.cache.get("r0").tables[0] if p >= 0]
        assert len(held) <= 2, (fed, held)          # a window of 6 positions touches two pages of 16 at most
        rep.engine.cache.check()
    compare(got, want, "float32", "a window group")
    rep.engine.release("r0")
    assert not rep.engine.cache.requests


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_long_decoding(folders, dtype):
    """300 single tokens after a short prompt: decode steps replayed from captured graphs, across page borders,
    while windows move on and pooled blocks are made and come into sight, the states carried through every replay."""
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


def test_a_far_token_shows_through_the_retention_alone(folders):
    """Two sequences that differ in their first token only: 100 tokens later the engine's logits differ by what
    the plain implementation says, in a model whose only path back is the retention's state (one head does not decay)."""
    from hfee_amd.trace_replay import Replayer
    folder = folders[("retention", "float32")]
    toks = tu.make_requests(50, [101], seed=3)["r0"]
    other = [(toks[0] + 7) % 50] + toks[1:]
    rep = Replayer(folder, "float32", 256, max_requests=2)
    got = tu.run(rep, [{"entries": [("a", toks[:60], []), ("b", other[:60], [])], "end": []},
                       {"entries": [("b", other[60:], [40]), ("a", toks[60:], [40])], "end": ["a", "b"]}])
    want = plain_logits(folder, toks)[100] - plain_logits(folder, other)[100]
    assert np.abs(want).max() > 1e-6
    assert su.rel(got[("a", 100)] - got[("b", 100)], want) < 1e-2


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
    assert su.rel(a[0], want[0]) < 3e-5 and su.rel(a[1], want[20]) < 3e-5
    assert su.rel(c[0], want[38]) < 3e-5 and su.rel(c[1], want[1]) < 3e-5


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
