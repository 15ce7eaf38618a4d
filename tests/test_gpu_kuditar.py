"""Kuditar on the GPU against the plain implementation: each kernel alone, each mixer alone with its own cache (whole,
token by token, in portions, in unequal batches, with pages and slots used again), the residual stream after every
layer, whole models replayed in the four ways of cutting, long decoding, and greedy generation through the session, its
scheduler and the command line.

Where random weights would hide a fault, the inputs are made so that it shows: head norms bound every score of the
model's own attention, so the attention kernel is also driven directly, with one cached key made to point along the
query (far back, on a page's first and last row, just inside and just outside a window, a run and the kept first
positions); a state that hardly fades is given one key and, hundreds of tokens later, the query that meets it.
"""
import math
import random

import numpy as np
import pytest
import torch

import plain_kuditar as P
import replay as R
from tiny import random_ids
from tiny_kuditar import CONFIGS, STD, write_folder, write_tiny

pytestmark = pytest.mark.gpu

DEV = "cuda:0"
DTYPES = [torch.float32, torch.bfloat16]


def gen(seed):
    return torch.Generator().manual_seed(seed)


def tol(dtype, ref, f32=2e-5, bf16=1e-2):
    return (f32 if dtype == torch.float32 else bf16) * max(1.0, float(ref.abs().max()))


def i32(values):
    return torch.tensor(values, dtype=torch.int32, device=DEV)


@pytest.fixture(scope="module")
def ops():
    from gesso_amd.kernels import ops
    ops.lib()
    return ops


@pytest.fixture(scope="module")
def folders(tmp_path_factory):
    return str(tmp_path_factory.mktemp("kuditar"))


def starts_of(lens):
    q_start = [0]
    for n in lens:
        q_start.append(q_start[-1] + n)
    return q_start


# ------------------------------------------------------------------ kernels alone

@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("H", [96, 100, 1024, 7, 1030, 4096])
def test_layer_norm_adds_what_is_pending_first(ops, dtype, H):
    res = torch.randn(7, H, generator=gen(0)) * 3 + 5.0          # a mean far from zero: a norm without it shows
    delta = (torch.randn(7, H, generator=gen(1)) * 2).to(dtype)
    w, b = 1 + 0.2 * torch.randn(H, generator=gen(2)), torch.randn(H, generator=gen(3))
    for d in (delta, None):
        r = res.clone().to(DEV)
        got = ops.add_layernorm(r, None if d is None else d.to(DEV), w.to(DEV), b.to(DEV), 1e-5, dtype)
        x = res.double() + (0 if d is None else d.double())
        assert float((r.cpu().double() - x).abs().max()) <= 1e-6 * float(x.abs().max())
        want = P.layer_norm(x, w.double(), b.double(), 1e-5)
        assert float((got.cpu().double() - want).abs().max()) <= tol(dtype, want)
    # some rows only, in another order: the stream stays as it was
    r = res.clone().to(DEV)
    got = ops.add_layernorm(r, delta.to(DEV), w.to(DEV), b.to(DEV), 1e-5, dtype, rows=i32([5, 0, 6, 5]))
    want = P.layer_norm(res.double() + delta.double(), w.double(), b.double(), 1e-5)[[5, 0, 6, 5]]
    assert float((got.cpu().double() - want).abs().max()) <= tol(dtype, want)
    assert torch.equal(r.cpu(), res)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("W", [96, 100, 2048])
def test_sum_of_two_normed_branches_and_the_gate_on_rows(ops, dtype, W):
    a, b = torch.randn(5, W, generator=gen(4)) * 7, torch.randn(5, W, generator=gen(5)) * 0.1
    wa, wb = 1 + 0.3 * torch.randn(W, generator=gen(6)), 1 + 0.3 * torch.randn(W, generator=gen(7))
    got = ops.normed_pair_sum(a.to(DEV), wa.to(DEV), 0.5, b.to(DEV), wb.to(DEV), 0.5, 1e-6, dtype)
    want = 0.5 * (P.rms(a.double(), 1e-6) * wa.double() + P.rms(b.double(), 1e-6) * wb.double())
    assert float((got.cpu().double() - want).abs().max()) <= tol(dtype, want)
    o = torch.randn(5, W, generator=gen(8)).to(dtype)
    rows = torch.randn(5, W + 24, generator=gen(9)).to(dtype)
    for gate, f in (("sigmoid", torch.sigmoid), ("silu", P.silu)):
        got = ops.gated_rows(o.to(DEV), rows.to(DEV), 24, gate)
        want = o.double() * f(rows[:, 24:].double())
        assert float((got.cpu().double() - want).abs().max()) <= tol(dtype, want)


class Pages:
    """A key and a value pool with the block tables of some sequences drawn from shuffled pages."""

    def __init__(self, dtype, nkv, d, vd, page_size, lens, seed=0, spare=3):
        g = gen(seed)
        blocks = [-(-n // page_size) for n in lens]
        total = sum(blocks) + spare
        order = torch.randperm(total, generator=g).tolist()
        self.table = torch.full((len(lens), max(blocks)), total, dtype=torch.int32)
        at = 0
        for s, nb in enumerate(blocks):
            self.table[s, :nb] = torch.tensor(order[at:at + nb], dtype=torch.int32)
            at += nb
        self.k = torch.full((total + 1, nkv, page_size, d), float("nan"), dtype=dtype, device=DEV)
        self.v = torch.full((total + 1, nkv, page_size, vd), float("nan"), dtype=dtype, device=DEV)
        self.table = self.table.to(DEV)
        self.ps = page_size


def tiles_of(sizes, rows):
    """int32 ``(3, ntiles)``: sequence, first row and row count of tiles of at most ``rows`` queries of one sequence."""
    seq, row, cnt, at = [], [], [], 0
    for i, n in enumerate(sizes):
        for a in range(0, n, rows):
            seq.append(i)
            row.append(at + a)
            cnt.append(min(rows, n - a))
        at += n
    return i32([seq, row, cnt])


def attention_case(ops, dtype, nh, nkv, d, vd, lens, cuts, ps=8, window=None, keep_first=0, chunk=None, cap=None, sinks=None,
                   scale=0.3, seed=0, plant=None, tiled=0):
    """Sequences of ``lens`` tokens fed in the pieces ``cuts[s]``: raw q | k | v rows go through the cache write (no norm,
    no turn) and the general attention kernel.  ``plant``: ``(sequence, key position, query position, size)``: that key is
    made to point along that query's first head, ``size`` times as long.  ``tiled``: 16 or 32: the kernel on the matrix
    cores with tiles of that many queries instead.  Returns the kernel's rows and the plain attention's, per sequence."""
    g = gen(seed)
    rows = [torch.randn(n, (nh + nkv) * d + nkv * vd, generator=g) for n in lens]
    if plant is not None:
        s, kp, qp, size = plant
        qv = rows[s][qp, :d]
        rows[s][kp, nh * d:nh * d + d] = qv / qv.norm() * size
    rows = [r.to(dtype) for r in rows]
    pg = Pages(dtype, nkv, d, vd, ps, lens, seed)
    sk = None if sinks is None else sinks.to(DEV)
    done = [0] * len(lens)
    got = [[] for _ in lens]
    for step in range(max(len(c) for c in cuts)):
        live = [s for s in range(len(lens)) if step < len(cuts[s])]
        sizes = [cuts[s][step] for s in live]
        x = torch.cat([rows[s][done[s]:done[s] + n] for s, n in zip(live, sizes)]).to(DEV)
        pos = [done[s] + i for s, n in zip(live, sizes) for i in range(n)]
        seq_of = [i for i, n in enumerate(sizes) for _ in range(n)]
        table = pg.table[live].contiguous()
        ops.qknorm_rope_kv(x, None, None, 1.0, None, None, 0, i32(pos), i32(seq_of), table, ps, pg.k, pg.v, nh, nkv, d, vd=vd)
        if tiled and all(n == 1 for n in sizes):
            # steps of single tokens: the kernel for single queries, its keys split over two blocks where it may
            y = ops.attention_decode(x, x.shape[1], pg.k, pg.v, i32(pos), table, ps, window, scale, nh, nkv, d, len(pos),
                                     2 if max(pos) >= 128 else 1, chunk=chunk, softcap=cap, keep_first=keep_first, sinks=sk)
        elif tiled:
            y = ops.attention_prefill(x, x.shape[1], pg.k, pg.v, i32(pos), tiles_of(sizes, tiled), table, ps, window, scale,
                                      nh, nkv, d, len(pos), tile_rows=tiled, chunk=chunk, softcap=cap, keep_first=keep_first,
                                      sinks=sk)
        else:
            y = ops.attention_generic(x, x.shape[1], pg.k, pg.v, i32(pos), i32(seq_of), table, ps, window, scale, nh, nkv, d,
                                      len(pos), vd=vd, chunk=chunk, softcap=cap, keep_first=keep_first, sinks=sk)
        at = 0
        for s, n in zip(live, sizes):
            got[s].append(y[at:at + n].double().cpu())
            at += n
            done[s] += n
    assert done == list(lens)
    want = []
    for s, n in enumerate(lens):
        r = rows[s].double()
        q, k, v = r[:, :nh * d].reshape(n, nh, d), r[:, nh * d:(nh + nkv) * d].reshape(n, nkv, d), r[:, (nh + nkv) * d:].reshape(n, nkv, vd)
        want.append(P.softmax_attention(q, k, v, list(range(n)), scale, cap=cap, window=window, keep_first=keep_first,
                                        chunk=chunk, sink=None if sinks is None else sinks.double()).reshape(n, nh * vd))
    return [torch.cat(g_) for g_ in got], want


RULES = [dict(), dict(cap=2.0), dict(window=7, keep_first=3), dict(window=1, keep_first=0), dict(window=17, keep_first=20),
         dict(window=24, keep_first=9, cap=5.0, sink=True), dict(window=9, sink=True), dict(chunk=7), dict(chunk=1),
         dict(chunk=16, cap=3.0), dict(window=40, keep_first=2, sink=True), dict(sink=True, cap=30.0)]


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("rule", RULES)
def test_attention_with_caps_windows_kept_positions_runs_and_sinks(ops, dtype, rule):
    rule = dict(rule)
    for nh, nkv, d, vd, ps in ((4, 2, 24, 16, 8), (3, 3, 10, 22, 4), (2, 1, 64, 64, 16)):
        sinks = torch.linspace(-2.0, 3.0, nh) if rule.get("sink") else None
        kw = {k: v for k, v in rule.items() if k != "sink"}
        lens = [70, 1, 33, 9]
        cuts = [[30, 1, 1, 20, 2, 16], [1], [33], [2, 2, 1, 1, 3]]
        got, want = attention_case(ops, dtype, nh, nkv, d, vd, lens, cuts, ps=ps, sinks=sinks, seed=nh + d, **kw)
        for s in range(len(lens)):
            assert float((got[s] - want[s]).abs().max()) <= tol(dtype, want[s], 2e-5, 2e-2), (s, nh, rule)


@pytest.mark.parametrize("rule", [r for r in RULES if not r.get("chunk")] + [dict(window=100, keep_first=70, cap=4.0, sink=True),
                                                                               dict(window=64, keep_first=64), dict(chunk=64, cap=3.0)])
@pytest.mark.parametrize("rows", [16, 32])
def test_tiled_prompt_attention_with_caps_windows_kept_positions_and_sinks(ops, rule, rows):
    """The prompt kernel on the matrix cores: sequences long enough for several steps of 64 keys, fed whole, in long
    portions and in short ones beside single tokens."""
    rule = dict(rule)
    for nh, nkv, d, ps in ((4, 2, 64, 16), (2, 2, 32, 8), (8, 2, 128, 16), (6, 1, 64, 4)):
        if rows == 32 and nh // nkv > 4:
            continue
        sinks = torch.linspace(-2.0, 3.0, nh) if rule.get("sink") else None
        kw = {k: v for k, v in rule.items() if k != "sink"}
        lens = [230, 1, 97, 40]
        cuts = [[100, 64, 1, 33, 30, 1, 1], [1], [97], [2, 17, 1, 1, 17, 1, 1]]
        got, want = attention_case(ops, torch.bfloat16, nh, nkv, d, d, lens, cuts, ps=ps, sinks=sinks, seed=nh + d, tiled=rows, **kw)
        for s in range(len(lens)):
            assert float((got[s] - want[s]).abs().max()) <= tol(torch.bfloat16, want[s], 2e-5, 2e-2), (s, nh, d, rule)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("ps", [8, 16])
def test_a_key_that_stands_out_is_seen_or_not_at_every_edge(ops, dtype, ps):
    """One key points along the last query: the head's weight goes there if and only if the rule lets the query see it.
    Far back, on a page's last and first row, just inside and just outside the window, the kept first positions and the
    query's run; whole and with the query fed alone."""
    T, nh, nkv, d, vd = 340, 2, 1, 16, 8
    query = T - 1
    window, keep, run = 50, 11, 64
    first_in_window = query - window + 1
    places = {"window": [first_in_window, first_in_window - 1, first_in_window + 1, keep - 1, keep, 0, query - 300 + 300 % ps,
                         (query // ps) * ps, (query // ps) * ps - 1, query - 1],
              "run": [query - query % run, query - query % run - 1, query - 1, 0, query - 300],
              "all": [query - 300, 0, ps - 1, ps, (query // ps) * ps - 1]}
    for kind, rule in (("window", dict(window=window, keep_first=keep, cap=20.0)), ("run", dict(chunk=run)), ("all", dict(cap=25.0))):
        for place in places[kind]:
            for cuts in ([[T]], [[query, 1]], [[query - 60] + [1] * 61]):
                got, want = attention_case(ops, dtype, nh, nkv, d, vd, [T], cuts, ps=ps, scale=1.0, seed=3,
                                           plant=(0, place, query, 12.0), **rule)
                assert float((got[0] - want[0]).abs().max()) <= tol(dtype, want[0], 2e-5, 2e-2), (kind, place, cuts[0][:2])
            seen = P.visible(query, place, rule.get("window"), rule.get("keep_first", 0), rule.get("chunk"))
            quiet, _ = attention_case(ops, dtype, nh, nkv, d, vd, [T], [[T]], ps=ps, scale=1.0, seed=3, **rule)
            moved = float((got[0][query, :vd] - quiet[0][query, :vd]).abs().max())
            assert (moved > 0.05) == seen, (kind, place, moved)
            if dtype == torch.bfloat16:
                # the same through the prompt kernel on the matrix cores (heads of 32), whole and in two portions
                for cuts in ([[T]], [[query - 70, 71]], [[query, 1]], [[query - 80] + [1] * 81]):
                    tg, tw = attention_case(ops, dtype, nh, nkv, 32, 32, [T], cuts, ps=ps, scale=1.0, seed=3, tiled=16,
                                            plant=(0, place, query, 12.0), **rule)
                    assert float((tg[0] - tw[0]).abs().max()) <= tol(dtype, tw[0], 2e-5, 2e-2), ("tiled", kind, place)
                tq, _ = attention_case(ops, dtype, nh, nkv, 32, 32, [T], [[T]], ps=ps, scale=1.0, seed=3, tiled=16, **rule)
                assert (float((tg[0][query, :32] - tq[0][query, :32]).abs().max()) > 0.05) == seen, ("tiled", kind, place)


@pytest.mark.parametrize("dtype", DTYPES)
def test_cache_write_with_a_plain_norm_a_partial_turn_wider_rows_and_blended_values(ops, dtype):
    from gesso_amd.parts.rope import rope_tables
    nh, nkv, d, vd, rd, ps, T = 3, 2, 12, 10, 8, 4, 23
    width = (nh + nkv) * d + nkv * vd
    x = (torch.randn(T, width + 30, generator=gen(20)) * 2).to(dtype)      # thirty columns of something else behind q | k | v
    first = torch.randn(T, nkv * vd + 5, generator=gen(21)).to(dtype)
    mix = torch.tensor([0.3])
    cos, sin = rope_tables(rd, 1e4, 64, divisor=2.5)
    pos = [17 + i for i in range(T)]
    pg = Pages(dtype, nkv, d, vd, ps, [17 + T], seed=1)
    xd = x.clone().to(DEV)
    ops.qknorm_rope_kv(xd, None, None, 1e-6, cos.to(DEV), sin.to(DEV), rd, i32(pos), i32([0] * T), pg.table, ps, pg.k, pg.v,
                       nh, nkv, d, vd=vd, plain_norm=True, v_first=first.to(DEV)[:, 5:], mix=mix.to(DEV))
    f = P.frequencies(rd, 1e4, 2.5)
    r = x.double()
    q = P.rms(P.rotate_half(r[:, :nh * d].reshape(T, nh, d), pos, f), 1e-6)
    k = P.rms(P.rotate_half(r[:, nh * d:(nh + nkv) * d].reshape(T, nkv, d), pos, f), 1e-6)
    v = 0.7 * r[:, (nh + nkv) * d:width].reshape(T, nkv, vd) + 0.3 * first[:, 5:].double().reshape(T, nkv, vd)
    out = xd.cpu().double()
    assert float((out[:, :nh * d].reshape(T, nh, d) - q).abs().max()) <= tol(dtype, q)
    assert torch.equal(out[:, nh * d:], r[:, nh * d:])                      # only q is rewritten in place
    table = pg.table[0].cpu().tolist()
    for t, p in enumerate(pos):
        page, row = table[p // ps], p % ps
        assert float((pg.k[page, :, row].double().cpu() - k[t]).abs().max()) <= tol(dtype, k)
        assert float((pg.v[page, :, row].double().cpu() - v[t]).abs().max()) <= tol(dtype, v)


def scan_case(ops, dtype, H, G, n, m, lens, cuts, per_channel, delta, seed=0, slow=False, meet=None, segment=0):
    """The recurrence over sequences of ``lens`` tokens fed in the pieces ``cuts[s]``, states in shuffled slots.  Returns
    the kernel's rows and the plain recurrence's, per sequence, and the states left."""
    g = gen(seed)
    junk = 5
    xs, decs, betas = [], [], []
    for L in lens:
        x = torch.randn(L, junk + 2 * G * n + H * m, generator=g)
        dec = torch.rand(L, 3 + (H * n if per_channel else H), generator=g) * (0.02 if slow else 0.6) + (0.98 if slow else 0.4)
        if meet is not None and L > meet[1]:
            x[:, junk:junk + 2 * G * n] *= 0.05
            x[meet[0], junk + G * n:junk + G * n + n] = 0.0
            x[meet[0], junk + G * n + 1] = 6.0                      # one key along channel 1 ...
            x[meet[1], junk:junk + n] = 0.0
            x[meet[1], junk + 1] = 6.0                              # ... and, later, the query along the same channel
        if delta:             # the delta rule is a contraction for keys no longer than one; longer keys make it grow without bound
            kk = x[:, junk + G * n:junk + 2 * G * n].reshape(L, G, n)
            x[:, junk + G * n:junk + 2 * G * n] = (kk / kk.norm(dim=-1, keepdim=True).clamp_min(1.0)).reshape(L, G * n)
        xs.append(x.to(dtype))
        decs.append(dec)
        betas.append(torch.rand(L, 2 + H, generator=g))
    slots = torch.randperm(len(lens) + 2, generator=g)[:len(lens)].tolist()
    state = torch.full((len(lens) + 3, H, n, m), float("nan"))
    for sl in slots:
        state[sl] = 0.0
    st = state.to(DEV)
    done = [0] * len(lens)
    got = [[] for _ in lens]
    for step in range(max(len(c) for c in cuts)):
        live = [s for s in range(len(lens)) if step < len(cuts[s])]
        sizes = [cuts[s][step] for s in live]
        cat = lambda parts: torch.cat([parts[s][done[s]:done[s] + k] for s, k in zip(live, sizes)]).to(DEV)
        if segment:       # the portions' segments side by side
            y = ops.gated_state_scan_segments(cat(xs), junk, junk + G * n, junk + 2 * G * n, H, G, n, m, cat(decs), 3,
                                              per_channel, st, sizes, i32([slots[s] for s in live]), segment, q_scale=0.5,
                                              beta=cat(betas) if delta else None, ob=2)
        else:
            y = ops.gated_state_scan(cat(xs), junk, junk + G * n, junk + 2 * G * n, H, G, n, m, cat(decs), 3, per_channel, st,
                                     i32(starts_of(sizes)), i32([slots[s] for s in live]), len(live), q_scale=0.5,
                                     beta=cat(betas) if delta else None, ob=2)
        at = 0
        for s, k in zip(live, sizes):
            got[s].append(y[at:at + k].double().cpu())
            at += k
            done[s] += k
    assert done == list(lens)
    want = []
    for s, L in enumerate(lens):
        x = xs[s].double()
        q = x[:, junk:junk + G * n].reshape(L, G, n) * 0.5
        k = x[:, junk + G * n:junk + 2 * G * n].reshape(L, G, n)
        v = x[:, junk + 2 * G * n:].reshape(L, H, m)
        heads = []
        for h in range(H):
            j = h // (H // G)
            if per_channel:
                alpha = decs[s][:, 3 + h * n:3 + (h + 1) * n].double()
                heads.append(P.gated_linear(q[:, j], k[:, j], v[:, h], alpha) if not delta else None)
            else:
                a = decs[s][:, 3 + h].double()
                b = betas[s][:, 2 + h].double() if delta else None
                heads.append(P.delta_rule(q[:, j], k[:, j], v[:, h], b, a) if delta
                             else P.gated_linear(q[:, j], k[:, j], v[:, h], a[:, None].expand(L, n)))
        want.append(torch.stack(heads, 1).reshape(L, H * m))
    untouched = [s for s in range(state.shape[0]) if s not in slots]
    assert all(torch.isnan(st[s]).all() for s in untouched)
    return [torch.cat(g_) for g_ in got], want, st.cpu(), slots


SCANS = [(4, 2, 16, 24), (3, 3, 8, 12), (6, 1, 32, 64), (2, 2, 64, 64), (2, 1, 128, 128), (5, 5, 6, 14), (2, 2, 14, 70), (1, 1, 200, 40)]


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("H,G,n,m", SCANS)
@pytest.mark.parametrize("per_channel,delta", [(False, True), (True, False), (False, False)])
def test_recurrences_over_unequal_sequences_and_any_cut(ops, dtype, H, G, n, m, per_channel, delta):
    if per_channel:
        G = H
    lens = [1, 23, 2, 41]
    whole = [[1], [23], [2], [41]]
    pieces = [[1], [5, 1, 1, 2, 7, 3, 1, 3], [1, 1], [12, 9, 1, 17, 2]]
    a, want, sa, slots_a = scan_case(ops, dtype, H, G, n, m, lens, whole, per_channel, delta, seed=n + m)
    b, _, sb, slots_b = scan_case(ops, dtype, H, G, n, m, lens, pieces, per_channel, delta, seed=n + m)
    for s in range(len(lens)):
        assert float((a[s] - want[s]).abs().max()) <= tol(torch.float32, want[s], 3e-5), s
        assert torch.equal(a[s], b[s]), s                        # one order of sums whatever the cut
        assert torch.equal(sa[slots_a[s]], sb[slots_b[s]])


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("H,G,n,m,seg", [(4, 2, 16, 24, 32), (2, 2, 64, 64, 64), (2, 1, 128, 128, 128), (5, 5, 6, 14, 16), (3, 1, 40, 70, 50)])
@pytest.mark.parametrize("per_channel,delta", [(False, True), (True, False)])
def test_recurrences_in_segments_side_by_side(ops, dtype, H, G, n, m, seg, per_channel, delta):
    """Portions of several segments beside short ones and single tokens; portions that start from states which earlier
    steps left; the states left behind against the walk in one piece."""
    if per_channel:
        G = H
    lens = [5 * seg + 3, 1, 2 * seg, seg + 9]
    pieces = [[3 * seg + 1, 1, 2 * seg + 1], [1], [seg - 1, seg + 1], [seg + 9]]
    whole = [[L] for L in lens]
    a, want, sa, slots_a = scan_case(ops, dtype, H, G, n, m, lens, whole, per_channel, delta, seed=n + m)
    b, _, sb, slots_b = scan_case(ops, dtype, H, G, n, m, lens, pieces, per_channel, delta, seed=n + m, segment=seg)
    for s in range(len(lens)):
        assert float((b[s] - want[s]).abs().max()) <= tol(torch.float32, want[s], 5e-5), s
        assert float((sb[slots_b[s]] - sa[slots_a[s]]).abs().max()) <= tol(torch.float32, sa[slots_a[s]], 5e-5), s


@pytest.mark.parametrize("cuts,seg", [([[420]], 0), ([[330] + [1] * 90], 0), ([[7] * 60], 0), ([[420]], 64), ([[290, 130]], 32)])
def test_a_state_keeps_what_it_was_given_hundreds_of_tokens_before(ops, cuts, seg):
    for per_channel, delta in ((False, True), (True, False)):
        got, want, _, _ = scan_case(ops, torch.float32, 2, 2, 8, 6, [420], cuts, per_channel, delta, seed=5, slow=True, meet=(20, 400),
                                    segment=seg)
        assert float(want[0][400].abs().max()) > 10 * float(want[0][399].abs().max())      # the meeting shows
        assert float((got[0] - want[0]).abs().max()) <= tol(torch.float32, want[0], 3e-5)


@pytest.mark.parametrize("dtype", DTYPES)
def test_what_the_delta_rule_computes_before_its_recurrence_and_the_channel_decays(ops, dtype):
    T, G, n, H = 9, 2, 12, 6
    c = torch.randn(T, 2 * G * n + 7, generator=gen(30)) * 3
    c[4, :n] = 0.0                                                 # a zero vector stays zero (eps under the root)
    rows = (torch.randn(T, 40, generator=gen(31)) * 4).to(dtype)
    a_log, dt_bias = torch.linspace(-6, 1, H), torch.linspace(-3, 1, H)
    cd = c.clone().to(DEV)
    gates = ops.delta_rule_prep(cd, G, n, n ** -0.5, 1e-6, rows.to(DEV), 11, 3, a_log.to(DEV), dt_bias.to(DEV), H).cpu().double()
    cc = c.double()
    q = P.unit(cc[:, :G * n].reshape(T, G, n)) * n ** -0.5
    k = P.unit(cc[:, G * n:2 * G * n].reshape(T, G, n))
    out = cd.cpu().double()
    assert float((out[:, :G * n].reshape(T, G, n) - q).abs().max()) <= 1e-6 and float((out[:, G * n:2 * G * n].reshape(T, G, n) - k).abs().max()) <= 1e-6
    assert torch.equal(out[:, 2 * G * n:], cc[:, 2 * G * n:])
    r = rows.double()
    g = torch.exp(-torch.exp(a_log.double()) * P.softplus(r[:, 11:11 + H] + dt_bias.double()))
    assert float((gates[:, :H] - g).abs().max()) <= 1e-6 and float((gates[:, H:] - torch.sigmoid(r[:, 3:3 + H])).abs().max()) <= 1e-6
    z = torch.randn(5, 33, generator=gen(32)) * 6
    for tau in (1.0, 16.0, 0.5):
        got = ops.channel_decay(z.clone().to(DEV), tau).cpu().double()
        assert float((got - torch.sigmoid(z.double()) ** (1 / tau)).abs().max()) <= 1e-6


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("E,top,H", [(6, 2, 96), (3, 1, 64), (4, 4, 100), (24, 2, 288), (70, 5, 40)])
def test_router_with_sigmoid_scores_chooses_by_corrected_scores_and_weighs_by_plain_ones(ops, dtype, E, top, H):
    x = torch.randn(11, H, generator=gen(33)).to(dtype)
    router = (torch.randn(E, H, generator=gen(34)) * 0.3).to(dtype)
    corr = torch.randn(E, generator=gen(35)) * 0.5
    choice, weight = ops.moe_router(x.to(DEV), router.to(DEV), corr.to(DEV), top, score="sigmoid", renormalize=False, scale=2.5)
    W = {"r.router": router.double(), "r.correction": corr.double()}
    chosen, weights = P.route(x.double(), W, "r.", top, 2.5)
    s = torch.sigmoid(x.double() @ router.double().T) + corr.double()
    for t in range(11):
        mine, theirs = choice[t].cpu().tolist(), chosen[t].tolist()
        if mine != theirs:        # a close call between two corrected scores may fall either way in float32
            gap = float(s[t][theirs].min() - s[t][[e for e in range(E) if e not in theirs]].max()) if top < E else 1.0
            assert sorted(mine) == sorted(theirs) or gap < 1e-5, t
        if sorted(mine) == sorted(theirs):
            ref = {e: float(w) for e, w in zip(theirs, weights[t])}
            assert all(abs(float(w) - ref[e]) <= 1e-5 for e, w in zip(mine, weight[t].cpu()))


# ------------------------------------------------------------------ mixers alone, each with its own cache

def _harness(spec, dtype, seed, page_size, num_pages, sharp):
    """A mixer with its own cache; the tensors ``sharp`` names are set to the given values (rounded to the tensors' type,
    as a file of that type would hold them) and the part is bound anew."""
    from test_gpu_parts import Harness
    from gesso_amd.parts import part_class
    from gesso_amd.weights.loader import held_dtype
    h = Harness("mixer", spec, dtype, seed=seed, page_size=page_size, num_pages=num_pages, std=0.25)
    if sharp:
        table = part_class("mixer", spec).tensor_specs(spec)
        for name, value in sharp.items():
            h.tensors[name] = value.to(dtype).double().reshape(h.tensors[name].shape)
        h.part.bind({k: v.to(dtype).to(DEV, held_dtype(dtype, table[k].role, dtype)) for k, v in h.tensors.items()})
    return h


ATT = {"q_proj.weight": "q", "k_proj.weight": "k", "v_proj.weight": "v", "gate_proj.weight": "g", "out_proj.weight": "o",
       "q_proj.bias": "q.b", "k_proj.bias": "k.b", "v_proj.bias": "v.b", "q_norm.weight": "q.norm", "k_norm.weight": "k.norm",
       "sinks": "sink", "value_mix": "vmix"}
DELTA = {"q_proj.weight": "q", "k_proj.weight": "k", "v_proj.weight": "v", "gate_proj.weight": "g", "beta_proj.weight": "b",
         "decay_proj.weight": "a", "q_conv.weight": "q.conv", "k_conv.weight": "k.conv", "v_conv.weight": "v.conv",
         "A_log": "A_log", "dt_bias": "dt_bias", "out_norm.weight": "norm", "out_proj.weight": "o"}
DECAY = {"q_proj.weight": "q", "k_proj.weight": "k", "v_proj.weight": "v", "gate_proj.weight": "g", "decay_down.weight": "a1",
         "decay_up.weight": "a2", "decay_up.bias": "a2.b", "out_norm.weight": "norm", "out_proj.weight": "o"}


def renamed(tensors, names, prefix, under=""):
    return {prefix + stored: tensors[under + local] for local, stored in names.items() if under + local in tensors}


def mixer_harness(kind, dtype, W=96, page_size=8, num_pages=64, seed=11, **kw):
    """A mixer of the design with its cache and the plain function of the same tensors."""
    from gesso_amd.config import AttentionSpec, GatedDeltaSpec, GatedLinearSpec, MixerPairSpec, NoPositionSpec, RMSNormSpec, RopeSpec
    eps = 1e-6
    g = gen(seed)

    def left_spec(H, G, d, vd, windowed, window=None, keep=0, run=None, cap=None, rd=0):
        pos = RopeSpec(head_dim=d, rotary_dim=rd, theta=1e4, max_position=1024) if rd else NoPositionSpec()
        return AttentionSpec(hidden=W, n_heads=H, n_kv_heads=G, head_dim=d, position=pos, qk_norm=RMSNormSpec(d, eps), bias=True,
                             out_bias=False, scale=0.3, value_dim=vd, softcap=cap, window=window, keep_first=keep,
                             head_sinks=windowed, chunk=run)

    def left_m(H, G, d, vd, window=None, keep=0, run=None, cap=None, rd=0):
        m = {"heads": H, "kv_heads": G, "dim": d, "vdim": vd, "scale": 0.3, "softcap": cap,
             "rot": {"base": 1e4, "dims": rd} if rd else None}
        m["mask"] = {"size": window, "keep_first": keep} if window else ({"size": run} if run else None)
        return m

    if kind == "gated":
        H, G, d, vd, rd, cap, factor = kw.get("H", 4), kw.get("G", 2), kw.get("d", 24), kw.get("vd", 16), kw.get("rd", 8), kw.get("cap", 6.0), kw.get("factor", 4.0)
        pos = RopeSpec(head_dim=d, rotary_dim=rd, theta=2e4, max_position=1024, frequency_divisor=factor) if rd else NoPositionSpec()
        spec = AttentionSpec(hidden=W, n_heads=H, n_kv_heads=G, head_dim=d, position=pos, qk_norm=RMSNormSpec(d, eps),
                             qk_norm_weight=False, scale=0.3, value_dim=vd, softcap=cap, out_gate="sigmoid", value_mix=True)
        h = _harness(spec, dtype, seed, page_size, num_pages, {})
        w = renamed(h.tensors, ATT, "m.")
        m = {"heads": H, "kv_heads": G, "dim": d, "vdim": vd, "scale": 0.3, "softcap": cap,
             "rot": {"base": 2e4, "dims": rd, "scaling": {"factor": factor}} if rd else None}
        return h, lambda x: P.gated_attention(x.double(), w, "m.", m, list(range(x.shape[0])), eps)[0]
    if kind in ("windowed", "runs"):
        H, G, d, vd = kw.get("H", 4), kw.get("G", 2), kw.get("d", 24), kw.get("vd", 16)
        rule = dict(window=kw.get("window", 21), keep=kw.get("keep", 5), cap=kw.get("cap", 6.0), rd=kw.get("rd", 24)) \
            if kind == "windowed" else dict(run=kw.get("run", 19))
        spec = left_spec(H, G, d, vd, kind == "windowed", **rule)
        sharp = {"sinks": torch.linspace(-2.0, 3.0, H)} if kind == "windowed" else {}
        h = _harness(spec, dtype, seed, page_size, num_pages, sharp)
        w = renamed(h.tensors, ATT, "m.")
        m = left_m(H, G, d, vd, **rule)
        f = P.windowed_branch if kind == "windowed" else P.chunked_branch
        return h, lambda x: f(x.double(), w, "m.", m, list(range(x.shape[0])), eps)
    if kind == "delta":
        H, G, n, m_, K = kw.get("H", 4), kw.get("G", 2), kw.get("n", 16), kw.get("m", 24), kw.get("taps", 4)
        spec = GatedDeltaSpec(hidden=W, n_heads=H, qk_heads=G, key_dim=n, value_dim=m_, conv_taps=K, eps=eps)
        sharp = {"A_log": torch.linspace(-6.0, 1.0, H), "dt_bias": torch.linspace(-3.0, 1.0, H)}
        h = _harness(spec, dtype, seed, page_size, num_pages, sharp)
        for k_ in ("q_conv.weight", "k_conv.weight", "v_conv.weight"):
            sharp[k_] = h.tensors[k_] * 4.0
        h = _harness(spec, dtype, seed, page_size, num_pages, sharp)
        w = renamed(h.tensors, DELTA, "m.")
        m = {"heads": H, "kv_heads": G, "dim": n, "vdim": m_, "conv": K}
        return h, lambda x: P.delta_branch(x.double(), w, "m.", m, eps)
    if kind == "decay":
        H, n, m_, r, tau = kw.get("H", 3), kw.get("n", 16), kw.get("m", 24), kw.get("r", 8), kw.get("tau", 8.0)
        spec = GatedLinearSpec(hidden=W, n_heads=H, key_dim=n, value_dim=m_, decay_rank=r, tau=tau, eps=eps)
        sharp = {"decay_up.bias": torch.rand(H * n, generator=g) * 6.0}
        h = _harness(spec, dtype, seed, page_size, num_pages, sharp)
        w = renamed(h.tensors, DECAY, "m.")
        m = {"heads": H, "dim": n, "vdim": m_, "tau": tau}
        return h, lambda x: P.gated_linear_branch(x.double(), w, "m.", m, eps)
    if kind == "pair":
        left = left_spec(4, 2, 24, 16, True, window=21, keep=5, cap=6.0, rd=24)
        right = GatedDeltaSpec(hidden=W, n_heads=4, qk_heads=2, key_dim=16, value_dim=24, conv_taps=4, eps=eps)
        spec = MixerPairSpec(left=left, right=right, left_scale=0.5, right_scale=0.5, branch_norm_eps=eps, hidden=W)
        sharp = {"left.sinks": torch.linspace(-2.0, 3.0, 4), "right.A_log": torch.linspace(-6.0, 1.0, 4),
                 "right.dt_bias": torch.linspace(-3.0, 1.0, 4)}
        h = _harness(spec, dtype, seed, page_size, num_pages, sharp)
        w = renamed(h.tensors, ATT, "m.left.", "left.")
        w.update(renamed(h.tensors, DELTA, "m.right.", "right."))
        w.update({"m.left.out": h.tensors["left_norm.weight"], "m.right.out": h.tensors["right_norm.weight"]})
        lm = left_m(4, 2, 24, 16, window=21, keep=5, cap=6.0, rd=24)
        rm = {"heads": 4, "kv_heads": 2, "dim": 16, "vdim": 24, "conv": 4}

        def plain(x):
            pos = list(range(x.shape[0]))
            return P.pair(P.windowed_branch(x.double(), w, "m.left.", lm, pos, eps), P.delta_branch(x.double(), w, "m.right.", rm, eps),
                          w, "m.", eps)
        return h, plain
    raise ValueError(kind)


CASES = [("gated", dict()), ("gated", dict(W=64, H=3, G=3, d=10, vd=22, rd=0, cap=None)), ("gated", dict(W=128, H=4, G=1, d=64, vd=64, rd=64, factor=1.0, page_size=16)),
         ("windowed", dict()), ("windowed", dict(W=64, H=2, G=1, d=12, vd=8, window=1, keep=0, rd=6, cap=None)),
         ("windowed", dict(W=64, H=3, G=3, d=10, vd=14, window=7, keep=11, rd=0)), ("windowed", dict(W=128, H=4, G=2, d=64, vd=64, window=32, keep=16, rd=64, page_size=16)),
         ("runs", dict()), ("runs", dict(W=64, H=2, G=2, d=8, vd=40, run=1)), ("runs", dict(W=128, H=4, G=1, d=64, vd=64, run=32, page_size=16)),
         ("delta", dict()), ("delta", dict(W=64, H=6, G=1, n=8, m=12, taps=1)), ("delta", dict(W=64, H=2, G=2, n=12, m=20, taps=5)),
         ("delta", dict(W=128, H=2, G=2, n=64, m=64, taps=4)), ("delta", dict(W=100, H=5, G=5, n=10, m=6, taps=2)),
         ("decay", dict()), ("decay", dict(W=64, H=2, n=24, m=8, r=3, tau=1.0)), ("decay", dict(W=128, H=2, n=128, m=128, r=16, tau=16.0)),
         ("decay", dict(W=100, H=5, n=6, m=14, r=7, tau=2.0)), ("pair", dict())]


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("kind,kw", CASES)
def test_mixers_whole_token_by_token_in_portions_and_in_batches(dtype, kind, kw):
    h, plain = mixer_harness(kind, dtype, **kw)
    W = kw.get("W", 96)
    T = 90
    x = torch.randn(T, W, generator=gen(40)).to(dtype)
    want = plain(x)
    bound = tol(dtype, want, 5e-5, 3e-2)
    whole = h.mixer(x, [("whole", T)])
    assert float((whole - want).abs().max()) <= bound
    # most of it at once, the rest token by token (across the window's, the kept positions' and a run's edges)
    head = 40
    got = [h.mixer(x[:head], [("tail", head)])] + [h.mixer(x[i:i + 1], [("tail", 1)]) for i in range(head, T)]
    assert float((torch.cat(got) - want).abs().max()) <= bound
    # the first tokens one by one from an empty cache and a zero state
    got = [h.mixer(x[i:i + 1], [("first", 1)]) for i in range(6)]
    assert float((torch.cat(got) - want[:6]).abs().max()) <= bound
    # portions of several sizes, down to two tokens
    at, got = 0, []
    for size in (2, 7, 2, 13, 3, 16, 5, 2, 31, 9):
        size = min(size, T - at)
        if size:
            got.append(h.mixer(x[at:at + size], [("cut", size)]))
            at += size
    assert at == T and float((torch.cat(got) - want).abs().max()) <= bound
    for rid in ("whole", "tail", "first", "cut"):
        h.manager.release(rid)
    # unequal requests side by side: a single token of one, a portion of another, a whole short one
    y = torch.randn(30, W, generator=gen(41)).to(dtype)
    u = torch.randn(5, W, generator=gen(42)).to(dtype)
    h.mixer(y[:29], [("b", 29)])
    h.mixer(x[:50], [("a", 50)])
    out = h.mixer(torch.cat([y[29:30], x[50:70], u]), [("b", 1), ("a", 20), ("c", 5)])
    assert float((out[0] - plain(y)[29]).abs().max()) <= bound
    assert float((out[1:21] - want[50:70]).abs().max()) <= bound
    assert float((out[21:] - plain(u)).abs().max()) <= bound


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("kind,kw", [("delta", dict()), ("delta", dict(W=128, H=2, G=2, n=64, m=64, taps=4)), ("decay", dict()),
                                     ("decay", dict(W=128, H=2, n=128, m=128, r=16, tau=16.0)), ("pair", dict())])
def test_recurrent_mixers_with_portions_long_enough_for_segments(dtype, kind, kw):
    """A prompt of several segments whole; the same in two long portions and single tokens; a long portion of one request
    beside a single token of another."""
    h, plain = mixer_harness(kind, dtype, num_pages=128, **kw)
    W = kw.get("W", 96)
    T = 700
    x = torch.randn(T, W, generator=gen(43)).to(dtype)
    want = plain(x)
    bound = tol(dtype, want, 5e-5, 3e-2)
    assert float((h.mixer(x, [("whole", T)]) - want).abs().max()) <= bound
    got = [h.mixer(x[:300], [("cut", 300)]), h.mixer(x[300:301], [("cut", 1)]), h.mixer(x[301:690], [("cut", 389)])]
    got += [h.mixer(x[i:i + 1], [("cut", 1)]) for i in range(690, T)]
    assert float((torch.cat(got) - want).abs().max()) <= bound
    h.manager.release("whole")
    h.manager.release("cut")
    y = torch.randn(30, W, generator=gen(44)).to(dtype)
    h.mixer(y[:29], [("b", 29)])
    h.mixer(x[:130], [("a", 130)])
    out = h.mixer(torch.cat([y[29:30], x[130:500]]), [("b", 1), ("a", 370)])
    assert float((out[0] - plain(y)[29]).abs().max()) <= bound
    assert float((out[1:] - want[130:500]).abs().max()) <= bound


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("kind", ["windowed", "runs", "delta", "decay", "pair", "gated"])
def test_mixers_with_pages_and_slots_freed_and_used_again(dtype, kind):
    """A pool that holds little more than one request's rows, and four slots: requests come and go, every later one
    writes pages and a slot that an earlier one gave back (filled with NaN in between)."""
    h, plain = mixer_harness(kind, dtype, page_size=8, num_pages=9)
    for i, T in enumerate((60, 35, 64, 9, 50, 20)):
        x = torch.randn(T, 96, generator=gen(50 + i)).to(dtype)
        want = plain(x)
        at, got = 0, []
        while at < T:
            size = min((11, 2, 1, 16)[(at + i) % 4], T - at)
            got.append(h.mixer(x[at:at + size], [(i, size)]))
            at += size
        assert float((torch.cat(got) - want).abs().max()) <= tol(dtype, want, 5e-5, 3e-2), i
        h.manager.release(i)
        for pool in h.storage.keys + h.storage.values:
            pool[:, :-1].fill_(float("nan"))
        for pool, _ in h.storage.state_pools:
            pool[:, :-1].fill_(float("nan"))


@pytest.mark.parametrize("dtype", DTYPES)
def test_a_window_that_has_given_pages_back_still_reads_the_kept_first_positions(dtype):
    """Two hundred tokens through a window of 21 with 5 kept positions, pages of 4, a pool of 12 pages: the pages between
    the kept ones and the window are given back on the way and poisoned; the result does not change."""
    h, plain = mixer_harness("windowed", dtype, page_size=4, num_pages=12)
    T = 200
    x = torch.randn(T, 96, generator=gen(60)).to(dtype)
    want = plain(x)
    at, got = 0, []
    while at < T:
        size = min((9, 2, 1, 16, 3)[at % 5], T - at)
        got.append(h.mixer(x[at:at + size], [("r", size)]))
        at += size
        released = h.manager.get("r").tables[0]
        free = [p for p in range(12) if p not in released]
        for pool in h.storage.keys + h.storage.values:
            pool[:, free].fill_(float("nan"))
    assert float((torch.cat(got) - want).abs().max()) <= tol(dtype, want, 5e-5, 3e-2)
    assert sum(1 for p in h.manager.get("r").tables[0] if p >= 0) <= 2 + 7


# ------------------------------------------------------------------ whole models

LENGTHS = {"A": (1, 23, 70, 130), "B": (2, 40, 77), "C": (5, 64, 150, 260), "D": (3, 52, 110)}


def sequences(name):
    cfg, seed = CONFIGS[name]
    return {f"s{i}": random_ids(n, cfg.vocab, 100 * seed + i) for i, n in enumerate(LENGTHS[name])}


def four_ways(seqs, seed, tail=48):
    ways = {"whole": R.trace_whole, "tail": lambda s: R.trace_tail(s, tail=tail), "portions": R.trace_portions,
            "mixed": lambda s: R.trace_mixed(s, seed=seed)}
    big = R.Trace()
    for way, make in ways.items():
        t = make({f"{way}.{k}": v for k, v in seqs.items()})
        for rec, rows in zip(t.steps, t.rows):
            big.steps.append(dict(rec, step=len(big.steps)))
            big.rows.append(rows)
        big.max_tokens = max(big.max_tokens, t.max_tokens)
    return ways, big


def check_rows(plain, got, dtype, label):
    """float32: every row against the plain model.  bfloat16, for models and sequences that nobody has looked through
    for close calls of a router (the engine and the rounded plain model may then choose differently, and that row stands
    far off whatever the engine does): nine rows in ten within the factor that ``noise.py`` gives a row, half of them
    within half of it."""
    if dtype == "float32":
        return plain.check(got, label)
    ratios = []
    for name, rows in got.items():
        for pos, row in rows.items():
            ref = plain.ref[name][pos].astype(np.float64)
            d, e = np.asarray(row, dtype=np.float64) - ref, plain.rounded[name][pos].astype(np.float64) - ref
            assert np.isfinite(d).all(), (label, name, pos)
            ratios.append(float(np.sqrt((d * d).mean()) / max(np.sqrt((e * e).mean()), 1e-30)))
    ratios = np.sort(np.array(ratios))
    from noise import ROW
    print(f"{label} bfloat16: {len(ratios)} rows, a row's rms over the rounded model's: median {np.median(ratios):.2f}, "
          f"nine in ten below {ratios[int(0.9 * (len(ratios) - 1))]:.2f}, largest {ratios[-1]:.2f}")
    assert len(ratios) >= 40 and np.median(ratios) <= ROW / 2 and ratios[int(0.9 * (len(ratios) - 1))] <= ROW, label


@pytest.mark.parametrize("name", ["A", "B", "D"])
def test_the_residual_stream_after_every_layer(name, folders):
    from gesso_amd.engine.batch import StepEntry
    from gesso_amd.engine.engine import Engine
    cfg, seed = CONFIGS[name]
    model_dir = write_tiny(folders, name, torch.float32)
    ids = random_ids(47, cfg.vocab, 5 * seed)
    want = []
    P.forward(P.read_config(model_dir), P.read_weights(model_dir), ids, layers_out=want)
    eng = Engine.from_folder(model_dir, dtype="float32", device=DEV, page_size=16, max_tokens=256, num_slots=4)
    got = []
    for b in eng.model.blocks:
        def wrapped(stream, ctx, cache, orig=b.forward):
            orig(stream, ctx, cache)
            x = stream.res.double().cpu()
            pend = stream.pending if isinstance(stream.pending, tuple) else (stream.pending,)
            got.append(x + sum(d.double().cpu() for d in pend if d is not None))
        b.forward = wrapped
    eng.add_request("r")
    eng.step([StepEntry("r", ids[:29], [])])
    first = list(got)
    got.clear()
    eng.step([StepEntry("r", ids[29:], [])])
    assert len(first) == len(got) == len(want) == len(cfg.layers)
    for i, w in enumerate(want):
        mine = torch.cat([first[i], got[i]])
        assert float((mine - w).abs().max()) <= 3e-5 * max(1.0, float(w.abs().max())), f"layer {i}"


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", ["A", "B", "C", "D"])
def test_replay_four_ways(name, dtype, folders, tmp_path):
    cfg, _ = CONFIGS[name]
    model_dir = write_tiny(folders, name, torch.float32 if dtype == "float32" else torch.bfloat16)
    seqs = sequences(name)
    plain = R.Plain(model_dir, seqs, dtype)
    ways, big = four_ways(seqs, 5)
    got, rc = R.run_trace(model_dir, dtype, str(tmp_path / "out"), big, cfg.vocab)
    assert rc == 0
    for way in ways:
        mine = {k.split(".", 1)[1]: v for k, v in got.items() if k.startswith(way + ".")}
        assert {k: len(v) for k, v in mine.items()} == {k: len(v) for k, v in seqs.items()}, way
        check_rows(plain, mine, dtype, f"Kuditar {name} {way}")


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", ["A", "D"])
def test_long_decoding_token_by_token(name, dtype, folders, tmp_path):
    """A short prompt, then three hundred tokens one by one: states carried, histories moved on, windows and runs
    passed and pages begun and given back many times over."""
    cfg, seed = CONFIGS[name]
    model_dir = write_tiny(folders, name, torch.float32 if dtype == "float32" else torch.bfloat16)
    seqs = {"long": random_ids(330, cfg.vocab, 7000 + seed), "other": random_ids(301, cfg.vocab, 7100 + seed)}
    plain = R.Plain(model_dir, seqs, dtype)
    got, rc = R.run_trace(model_dir, dtype, str(tmp_path / "out"), R.trace_tail(seqs, tail=300), cfg.vocab)
    assert rc == 0 and {k: len(v) for k, v in got.items()} == {"long": 330, "other": 301}
    check_rows(plain, got, dtype, f"Kuditar {name}, 300 tokens one by one")


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", ["A", "B"])
def test_replay_with_pages_of_eight_given_back_poisoned(name, dtype, folders, tmp_path):
    cfg, _ = CONFIGS[name]
    model_dir = write_tiny(folders, name, torch.float32 if dtype == "float32" else torch.bfloat16)
    seqs = sequences(name)
    plain = R.Plain(model_dir, seqs, dtype)
    for way, make in (("portions", lambda s: R.trace_portions(s, sizes=(13, 2, 8, 3))), ("mixed", lambda s: R.trace_mixed(s, seed=9))):
        got, rc = R.run_trace(model_dir, dtype, str(tmp_path / way), make(seqs), cfg.vocab, page_size=8, extra=["--poison"])
        assert rc == 0
        check_rows(plain, got, dtype, f"Kuditar {name}, pages of 8, poisoned, {way}")


@pytest.mark.parametrize("name", ["A", "B"])
def test_greedy_generation_through_the_session(name, folders):
    """Prompts of unequal length generated together through the scheduler (prefill in portions, then the decode loop);
    float32 must give the plain model's tokens."""
    from gesso_amd import Session
    cfg, _ = CONFIGS[name]
    model_dir = write_tiny(folders, name, torch.float32)
    pc, pw = P.read_config(model_dir), P.read_weights(model_dir)
    prompts = [random_ids(n, cfg.vocab, 900 + n) for n in (3, 41, 18)]
    new = 40
    want = [P.greedy(pc, pw, p, new) for p in prompts]
    session = Session(model_dir, dtype="float32", device=DEV, context_length=256, chunk_size=16)
    try:
        assert session.generate(prompts, max_new_tokens=new) == want
        assert session.generate([prompts[1]], max_new_tokens=new)[0] == want[1]
    finally:
        session.close()
    session = Session(write_tiny(folders, name, torch.bfloat16), dtype="bfloat16", device=DEV, context_length=256)
    try:
        got = session.generate(prompts, max_new_tokens=new)
        assert [len(g) for g in got] == [len(w) for w in want]
        # every token bfloat16 chose is one the plain model ranks close to its best at that place
        from noise import supported
        pw16 = P.read_weights(write_tiny(folders, name, torch.bfloat16))
        for g_, p in zip(got, prompts):
            lg = P.forward(pc, pw16, g_).numpy()
            assert all(supported(lg[i - 1], g_[i], 0.5) for i in range(len(p), len(g_)))
    finally:
        session.close()


def test_the_command_line_serves_a_kuditar_folder(folders):
    import json
    import os
    import subprocess
    import sys
    cfg, _ = CONFIGS["D"]
    model_dir = write_tiny(folders, "D", torch.float32)
    prompt = random_ids(19, cfg.vocab, 77)
    want = P.greedy(P.read_config(model_dir), P.read_weights(model_dir), prompt, 24)
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    r = subprocess.run([sys.executable, "-m", "gesso_amd", "--model", model_dir, "--dtype", "float32", "--prompt-ids",
                        ",".join(str(t) for t in prompt), "--max-new-tokens", "24", "--n-ctx", "128"],
                       capture_output=True, text=True, cwd=root, timeout=240, env=dict(os.environ, PYTHONPATH=root))
    assert r.returncode == 0, r.stderr[-2000:]
    assert json.loads(r.stdout.strip().splitlines()[-1])["ids"] == [want]


def test_forty_requests_at_once_decode_together(folders):
    from gesso_amd import Session
    from noise import supported
    cfg, _ = CONFIGS["A"]
    model_dir = write_tiny(folders, "A", torch.bfloat16)
    pc, pw = P.read_config(model_dir), P.read_weights(model_dir)
    prompts = [random_ids(3 + (7 * i) % 40, cfg.vocab, 2000 + i) for i in range(40)]
    session = Session(model_dir, dtype="bfloat16", device=DEV, context_length=128, max_num_seqs=64)
    try:
        got = session.generate(prompts, max_new_tokens=10)
        alone = session.generate([prompts[0]], max_new_tokens=10)[0]
    finally:
        session.close()
    assert [len(g_) for g_ in got] == [len(p) + 10 for p in prompts]
    for i in (0, 17, 39):
        lg = P.forward(pc, pw, got[i]).numpy()
        assert all(supported(lg[j - 1], got[i][j], 0.5) for j in range(len(prompts[i]), len(got[i]))), i
    lg = P.forward(pc, pw, alone).numpy()
    assert all(supported(lg[j - 1], alone[j], 0.5) for j in range(len(prompts[0]), len(alone)))


def random_kuditar(seed: int):
    """A configuration drawn from a seed: two to five layers of the three kinds in any order, sizes with and without whole
    tiles, with and without caps, turns, kept positions, windows, runs, feed-forwards of either kind or none."""
    from gesso_amd.config import (ChannelDecayConfig, DeltaRuleConfig, DenseFFConfig, GatedAttentionConfig, KuditarConfig,
                                  KuditarLayer, PairConfig, RunAttentionConfig, SigmoidMoEConfig, Turn, WindowedAttentionConfig)
    rng = random.Random(seed)
    width = rng.choice([64, 72, 96, 128, 160])

    def mlp():
        r = rng.random()
        if r < 0.15:
            return None
        if r < 0.45:
            return DenseFFConfig(rng.choice([8, 24, 40, 64, 200]), rng.choice([0.5, 1.5, 7.0]))
        E = rng.choice([1, 2, 3, 5, 8, 12])
        return SigmoidMoEConfig(E, rng.randint(1, min(4, E)), rng.choice([1.0, 2.5, 0.5]), rng.choice([8, 12, 24, 40, 64]),
                                rng.choice([0.5, 1.0, 2.0, 7.0]))

    def heads():
        G = rng.choice([1, 2, 3])
        return G * rng.choice([1, 2, 3]), G

    def turn(d):
        if rng.random() < 0.2:
            return None
        dims = rng.choice([x for x in (2, 6, 8, 16, 32, 64) if x <= d])
        return Turn(rng.choice([1e2, 1e4, 2.5e5]), dims, rng.choice([1.0, 1.0, 2.0, 8.0]))

    shared = (rng.choice([1, 2]), rng.choice([6, 16, 32]))
    layers = []
    for _ in range(rng.randint(2, 5)):
        kind = rng.choice(["attention", "parallel", "parallel_2"])
        d, vd = rng.choice([6, 8, 16, 24, 48, 64, 128]), rng.choice([4, 6, 16, 32, 64])
        cap = rng.choice([None, 5.0, 30.0])
        scale = rng.choice([0.1, 0.2, 0.35])
        if kind == "attention":
            mix = rng.random() < 0.6
            H, G = heads()
            if mix:
                G, vd = shared
                H = G * rng.choice([1, 2, 4])
            layers.append(KuditarLayer(kind, GatedAttentionConfig(H, G, d, vd, scale, cap, turn(d), mix), mlp()))
        elif kind == "parallel":
            H, G = heads()
            window = rng.choice([None, 1, 5, 16, 33, 64, 100])
            keep = rng.choice([0, 1, 4, 20]) if window else 0
            RH, RG = heads()
            left = WindowedAttentionConfig(H, G, d, vd, scale, cap, turn(d), window, keep)
            right = DeltaRuleConfig(RH, RG, rng.choice([4, 8, 16, 32, 64]), rng.choice([4, 8, 24, 64]), rng.choice([1, 2, 3, 4, 5]))
            layers.append(KuditarLayer(kind, PairConfig(left, right), mlp()))
        else:
            H, G = heads()
            left = RunAttentionConfig(H, G, d, vd, scale, None, None, rng.choice([None, 1, 7, 16, 40, 64]))
            right = ChannelDecayConfig(rng.choice([1, 2, 3, 6]), rng.choice([4, 8, 16, 32, 64]), rng.choice([4, 8, 24, 64]),
                                       rng.choice([1.0, 4.0, 16.0]), rng.choice([1, 3, 8, 16]))
            layers.append(KuditarLayer(kind, PairConfig(left, right), mlp()))
    return KuditarConfig(vocab=rng.choice([97, 200, 333, 512]), width=width, norm_eps=rng.choice([1e-5, 1e-6, 1e-4]),
                         embedding_scale=rng.choice([1.0, 3.0, math.sqrt(width)]), max_position=512, layers=tuple(layers))


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("seed", [91, 92, 93, 94, 95, 96, 97, 98])
def test_replay_of_configurations_drawn_at_random(seed, dtype, tmp_path):
    cfg = random_kuditar(seed)
    rng = random.Random(seed)
    model_dir = write_folder(str(tmp_path / "m"), cfg, seed, torch.float32 if dtype == "float32" else torch.bfloat16)
    lens = [rng.randint(1, 4), rng.randint(20, 60), rng.randint(70, 120), rng.randint(130, 180)]
    seqs = {f"s{i}": random_ids(n, cfg.vocab, seed * 10 + i) for i, n in enumerate(lens)}
    plain = R.Plain(model_dir, seqs, dtype)
    ways, big = four_ways(seqs, seed, tail=40)
    got, rc = R.run_trace(model_dir, dtype, str(tmp_path / "out"), big, cfg.vocab, extra=["--poison"])
    assert rc == 0
    for way in ways:
        mine = {k.split(".", 1)[1]: v for k, v in got.items() if k.startswith(way + ".")}
        assert {k: len(v) for k, v in mine.items()} == {k: len(v) for k, v in seqs.items()}, way
        check_rows(plain, mine, dtype, f"Kuditar drawn from {seed}, {way}")
