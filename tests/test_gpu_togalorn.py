"""Togalorn on the GPU against the plain implementation: each kernel alone, each mixer and the feed-forward alone (the
mixers with their own caches: whole, token by token, in portions, in unequal batches, with pages and slots used again),
the residual stream after every layer run, whole models replayed in the four ways of cutting, long decoding, and greedy
generation through the session, its scheduler and the command line.

Where random weights would hide a fault, the inputs are made so that it shows: a state-space head that hardly decays is
given one B row and, hundreds of tokens later, one C row that meet; the rotated key part of one token (the only part of
a cached row that no norm rescales) is scaled up until that token takes a query's weight, far back and on a page's first
and last row; the router's correction is made large enough to change the choice while the weights must not see it.
"""
import math

import numpy as np
import pytest
import torch

import plain_togalorn as P
import replay as R
from tiny import random_ids
from tiny_togalorn import CONFIGS, STD, write_folder, write_tiny

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
    return str(tmp_path_factory.mktemp("togalorn"))


def starts_of(lens):
    q_start = [0]
    for n in lens:
        q_start.append(q_start[-1] + n)
    return q_start


# ------------------------------------------------------------------ kernels alone

@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("H,groups", [(96, 3), (100, 5), (1024, 1), (384, 2), (66, 66), (1030, 2)])
def test_norm_in_parts_adds_what_is_pending_first(ops, dtype, H, groups):
    res = torch.randn(7, H, generator=gen(0)) * 3
    res[:, :H // groups] *= 20                          # one part much larger than the others: a norm over the whole row shows
    d1, d2 = torch.randn(7, H, generator=gen(1)).to(dtype), (torch.randn(7, H, generator=gen(2)) * 2).to(dtype)
    w = 1 + 0.2 * torch.randn(H, generator=gen(3))
    for deltas in ((d1, d2), (d1, None), (None, None)):
        r = res.clone().to(DEV)
        got = ops.add_group_rmsnorm(r, *(None if d is None else d.to(DEV) for d in deltas), w.to(DEV), 1e-5, groups, dtype)
        x = res.double() + sum(d.double() for d in deltas if d is not None)
        assert float((r.cpu().double() - x).abs().max()) <= 1e-6 * float(x.abs().max())
        want = P.group_norm(x, w.double(), 1e-5, groups)
        assert float((got.cpu().double() - want).abs().max()) <= tol(dtype, want)
    # some rows only, in another order: the stream stays as it was
    r = res.clone().to(DEV)
    got = ops.add_group_rmsnorm(r, d1.to(DEV), None, w.to(DEV), 1e-5, groups, dtype, rows=i32([5, 0, 6]))
    want = P.group_norm(res.double() + d1.double(), w.double(), 1e-5, groups)[[5, 0, 6]]
    assert float((got.cpu().double() - want).abs().max()) <= tol(dtype, want)
    assert torch.equal(r.cpu(), res)


def conv_case(ops, dtype, C, K, lens, pieces, act=None, residual=False, bias=True, seed=0, out_dtype=None):
    """Sequences of ``lens`` tokens, each fed in the pieces ``pieces[s]`` (steps hold piece i of every sequence that has
    one), histories in shuffled slots.  Returns the kernel's rows and the plain convolution's, per sequence."""
    g = gen(seed)
    junk = 8 if C % 16 == 0 else 3          # (rows whose stride and start allow 16-byte accesses, and rows that do not)
    xs = [(torch.randn(n, C + junk, generator=g) * 1.5).to(dtype) for n in lens]
    taps = torch.randn(C, K, generator=g) * 0.5
    b = torch.randn(C, generator=g) if bias else None
    slots = torch.randperm(len(lens) + 2, generator=g)[:len(lens)].tolist()
    state = torch.full((len(lens) + 3, max(K - 1, 1), C), float("nan"))
    for sl in slots:
        state[sl] = 0.0
    st = state.to(DEV)
    done = [0] * len(lens)
    got = [[] for _ in lens]
    for step in range(max(len(p) for p in pieces)):
        live = [s for s in range(len(lens)) if step < len(pieces[s])]
        sizes = [pieces[s][step] for s in live]
        rows = torch.cat([xs[s][done[s]:done[s] + n] for s, n in zip(live, sizes)]).to(DEV)
        seq_of = [i for i, n in enumerate(sizes) for _ in range(n)]
        y = ops.channel_conv(rows[:, junk:], taps.to(DEV), None if b is None else b.to(DEV), st, i32(seq_of),
                             i32(starts_of(sizes)), i32([slots[s] for s in live]), len(live), all(n == 1 for n in sizes),
                             out_dtype or dtype, activation=act, residual=residual)
        at = 0
        for s, n in zip(live, sizes):
            got[s].append(y[at:at + n].double().cpu())
            at += n
            done[s] += n
    assert done == list(lens)
    want = []
    for s in range(len(lens)):
        x = xs[s][:, junk:].double()
        y = P.causal_conv(x, taps.double(), None if b is None else b.double())
        if act == "silu":
            y = P.silu(y)
        want.append(y + x if residual else y)
    untouched = [s for s in range(state.shape[0]) if s not in slots]
    assert all(torch.isnan(st[s]).all() for s in untouched)
    return [torch.cat(g_) for g_ in got], want, st.cpu(), slots, xs, junk


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("C,K", [(40, 4), (33, 3), (130, 2), (17, 5), (24, 1), (520, 4), (48, 4), (64, 1), (528, 3), (16, 5)])
def test_convolution_over_time_in_pieces_with_a_history_per_request(ops, dtype, C, K):
    lens = [1, 23, 2, 12, 9]
    pieces = [[1], [5, 1, 1, 2, 7, 3, 1, 3], [1, 1], [12], [2, 2, 1, 1, 3]]
    for act, residual, bias in (("silu", False, True), (None, True, False)):
        got, want, state, slots, xs, junk = conv_case(ops, dtype, C, K, lens, pieces, act, residual, bias, seed=C + K,
                                                      out_dtype=torch.float32 if act else None)
        for s in range(len(lens)):
            assert float((got[s] - want[s]).abs().max()) <= tol(torch.float32 if act else dtype, want[s]), (s, act)
            if K > 1:
                # the history left behind: the last K - 1 inputs in their order in time, zeros before the start
                x = torch.cat([torch.zeros(K - 1, C, dtype=torch.float64), xs[s][:, junk:].double()])[-(K - 1):]
                assert torch.equal(state[slots[s]].double(), x.float().double()), s


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("H,groups", [(64, 2), (96, 3), (90, 1), (256, 4), (60, 6), (2048, 1), (4096, 8), (48, 3), (64, 16)])
def test_gate_then_norm_in_parts(ops, dtype, H, groups):
    y = torch.randn(9, H, generator=gen(4)) * 2
    y[:, :H // groups] *= 30
    # the gate: a column range of wider rows (with and without a start and a stride that allow 16-byte accesses)
    at, extra = (8, 16) if H % 16 == 0 else (4, 11)
    wide = torch.randn(9, H + extra, generator=gen(5)).to(dtype)
    w = 1 + 0.3 * torch.randn(H, generator=gen(6))
    got = ops.gated_group_norm(y.to(DEV), wide.to(DEV)[:, at:at + H], w.to(DEV), 1e-6, groups, dtype).double().cpu()
    want = P.group_norm(y.double() * P.silu(wide[:, at:at + H].double()), w.double(), 1e-6, groups)
    assert float((got - want).abs().max()) <= tol(dtype, want)
    # the other order (norm, then gate) is another function: the inputs tell them apart
    other = P.group_norm(y.double(), w.double(), 1e-6, groups) * P.silu(wide[:, at:at + H].double())
    assert float((other - want).abs().max()) > 10 * tol(dtype, want)


def segment_table(sizes, seg_len):
    """Where each sequence's segments begin, then (sequence, first token within the portion, tokens, 1 at the last)."""
    first, rows = [0], []
    for i, n in enumerate(sizes):
        for a in range(0, n, seg_len):
            rows += [i, a, min(seg_len, n - a), 1 if a + seg_len >= n else 0]
        first.append(len(rows) // 4)
    return i32(first + rows), len(rows) // 4


def scan_case(ops, dtype, H, P_, N, G, lens, pieces=None, seed=0, a_log=None, meet=None, seg_len=None):
    """Rows of x | B | C (float32, as the convolution leaves them) and of step sizes inside wider rows of ``dtype``, for
    sequences of ``lens`` tokens fed in ``pieces`` (default: whole), states in shuffled slots.  ``seg_len``: a step that
    brings a portion of twice that many tokens is walked in segments of that many, side by side.  ``meet``: ``(sequence,
    far token, near token, head)``: the far token's B row and the near one's C row are made to meet, and the far
    token's x row and step size are made large."""
    g = gen(seed)
    pieces = pieces or [[n] for n in lens]
    inner = H * P_
    xbc = [torch.randn(n, inner + 2 * G * N, generator=g) * 0.6 for n in lens]
    odt = 5
    drows = [(torch.randn(n, odt + H + 2, generator=g) * 1.5).to(dtype) for n in lens]
    a_log = torch.tensor(a_log, dtype=torch.float32) if a_log is not None else torch.linspace(-6.0, 0.7, H)
    dt_bias, d_skip = torch.rand(H, generator=g) * 3 - 2, 1 + 0.3 * torch.randn(H, generator=g)
    if meet is not None:
        s, far, near, hd = meet
        grp = hd // (H // G)
        b_at, c_at = inner + grp * N, inner + G * N + grp * N
        direction = torch.randn(N, generator=g)
        direction /= direction.norm()
        xbc[s][far, b_at:b_at + N] = 6.0 * direction
        xbc[s][near, c_at:c_at + N] = 6.0 * direction
        xbc[s][far, hd * P_:(hd + 1) * P_] = 8.0 * torch.sign(torch.randn(P_, generator=g))
        drows[s][far, odt + hd] = 3.0
    slots = torch.randperm(len(lens) + 2, generator=g)[:len(lens)].tolist()
    state = torch.full((len(lens) + 3, H, N, P_), float("nan"))
    for sl in slots:
        state[sl] = 0.0
    st = state.to(DEV)
    done = [0] * len(lens)
    got = [[] for _ in lens]
    for step in range(max(len(p) for p in pieces)):
        live = [s for s in range(len(lens)) if step < len(pieces[s])]
        sizes = [pieces[s][step] for s in live]
        rows = torch.cat([xbc[s][done[s]:done[s] + n] for s, n in zip(live, sizes)]).to(DEV)
        dr = torch.cat([drows[s][done[s]:done[s] + n] for s, n in zip(live, sizes)]).to(DEV)
        y = ops.ssd_scan(rows, dr, odt, dt_bias.to(DEV), a_log.to(DEV), d_skip.to(DEV), st, i32(starts_of(sizes)),
                         i32([slots[s] for s in live]), len(live), H, P_, N, G,
                         segments=segment_table(sizes, seg_len) if seg_len and max(sizes) >= 2 * seg_len else None)
        at = 0
        for s, n in zip(live, sizes):
            got[s].append(y[at:at + n].cpu())
            at += n
            done[s] += n
    want = []
    for s, n in enumerate(lens):
        x = xbc[s].double()
        dt = torch.nn.functional.softplus(drows[s][:, odt:odt + H].double() + dt_bias.double(), threshold=1e9)
        want.append(P.state_space(x[:, :inner].reshape(n, H, P_), x[:, inner:inner + G * N].reshape(n, G, N),
                                  x[:, inner + G * N:].reshape(n, G, N), dt, a_log.double(), d_skip.double(), H // G).reshape(n, inner))
    untouched = [s for s in range(state.shape[0]) if s not in slots]
    assert all(torch.isnan(st[s]).all() for s in untouched)
    scan_case.states = [st[sl].cpu() for sl in slots]
    return [torch.cat(g_) for g_ in got], want, xbc, d_skip


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("H,P_,N,G", [(4, 16, 24, 2), (3, 24, 16, 1), (6, 8, 12, 3), (2, 64, 64, 1), (2, 128, 128, 2), (5, 10, 7, 5),
                                      (1, 40, 200, 1), (8, 32, 40, 4)])
def test_state_recurrence_over_unequal_sequences_and_any_cut(ops, dtype, H, P_, N, G):
    lens = [1, 37, 2, 20]
    got, want, _, _ = scan_case(ops, dtype, H, P_, N, G, lens, seed=H + N)
    for s in range(len(lens)):
        assert float((got[s].double() - want[s]).abs().max()) <= 5e-5 * max(1.0, float(want[s].abs().max())), s
    # the same sequences in pieces, some of one token, beside one another: the same bits
    pieces = [[1], [5, 1, 1, 9, 2, 16, 3], [1, 1], [2, 2, 8, 1, 7]]
    cut, _, _, _ = scan_case(ops, dtype, H, P_, N, G, lens, pieces, seed=H + N)
    for s in range(len(lens)):
        assert torch.equal(cut[s], got[s]), s


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("H,P_,N,G,seg", [(4, 16, 24, 2, 32), (2, 64, 64, 1, 64), (2, 128, 128, 2, 128), (5, 10, 7, 5, 16), (8, 32, 40, 4, 50)])
def test_state_recurrence_in_segments_side_by_side(ops, dtype, H, P_, N, G, seg):
    """Long portions beside short ones and single tokens; a portion that ends on a segment's edge, one a token past it;
    states that go on from earlier steps, in segments again and token by token."""
    lens = [1, 2 * seg, 40, 4 * seg + 1, 2, 3 * seg + seg // 2 + 7]
    whole, want, _, _ = scan_case(ops, dtype, H, P_, N, G, lens, seed=H + N)
    states = scan_case.states
    for pieces in (None, [[1], [2 * seg], [20, 1, 19], [2 * seg + 3, 1, 1, 2 * seg - 4], [1, 1], [seg + 7, 2 * seg + seg // 2]]):
        got, _, _, _ = scan_case(ops, dtype, H, P_, N, G, lens, pieces, seed=H + N, seg_len=seg)
        for s in range(len(lens)):
            bound = 5e-5 * max(1.0, float(want[s].abs().max()))
            assert float((got[s].double() - want[s]).abs().max()) <= bound, s
            assert float((got[s] - whole[s]).abs().max()) <= bound, s
            assert float((scan_case.states[s] - states[s]).abs().max()) <= 5e-5 * max(1.0, float(states[s].abs().max())), s


@pytest.mark.parametrize("pieces,seg", [(None, None), ([[300] + [1] * 60], None), ([[7] * 51 + [3]], None), (None, 64), ([[290, 70]], 32)])
def test_a_state_keeps_what_it_was_given_hundreds_of_tokens_before(ops, pieces, seg):
    """Head 0 hardly decays (exp(A_log) = e^-9), head 1 forgets within a few tokens: the far token's B row meets the
    near token's C row in head 0 and stands out of everything in between; in head 1 nothing of it is left."""
    H, P_, N, G = 2, 16, 32, 1
    far, near = 11, 350
    for hd, kept in ((0, True), (1, False)):
        got, want, xbc, d_skip = scan_case(ops, torch.float32, H, P_, N, G, [360], pieces, seed=3, a_log=[-9.0, 1.5],
                                           meet=(0, far, near, hd), seg_len=seg)
        assert float((got[0].double() - want[0]).abs().max()) <= 5e-5 * max(1.0, float(want[0].abs().max()))
        # what the far token alone would put out at the near one, undecayed: dt (B . C) x, dt = softplus(3 + bias) > 1
        y = want[0][near, hd * P_:(hd + 1) * P_] - d_skip[hd].double() * xbc[0][near, hd * P_:(hd + 1) * P_].double()
        assert (float(y.abs().min()) > 100.0) == kept, hd                  # (what the tokens in between add stays below 30)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("EA,top,H", [(6, 2, 96), (3, 1, 64), (4, 4, 100), (24, 2, 288), (70, 5, 40), (2, 2, 8)])
def test_router_chooses_by_corrected_scores_and_weighs_by_plain_ones(ops, dtype, EA, top, H):
    g = gen(EA + top)
    x = torch.randn(50, H, generator=g).to(dtype)
    router = (torch.randn(EA, H, generator=g) * 0.3).to(dtype)
    correction = 0.5 * torch.randn(EA, generator=g)
    choice, weight = ops.moe_router(x.to(DEV), router.to(DEV), correction.to(DEV), top)
    want_c, want_w, s = P.route(x.double(), router.double(), correction.double(), top)
    plain_c, _, _ = P.route(x.double(), router.double(), torch.zeros(EA, dtype=torch.float64), top)
    if top < EA:
        assert not torch.equal(want_c, plain_c)                           # the correction matters here
    # a choice may differ only where two corrected scores are closer than float32 tells apart
    margin = torch.sort(s + correction.double(), descending=True).values[:, :top + 1]
    clear = (margin[:, :-1] - margin[:, 1:]).min(1).values > 1e-5
    assert int(clear.sum()) >= 45
    assert torch.equal(choice.cpu().long()[clear], want_c[clear])
    assert float((weight.cpu().double()[clear] - want_w[clear]).abs().max()) <= 2e-5
    assert float((weight.sum(1) - 1).abs().max()) <= 1e-5
    # equal scores (a router of zeros): the lowest indices, equal weights
    zc, zw = ops.moe_router(x.to(DEV), torch.zeros_like(router).to(DEV), None, top)
    assert torch.equal(zc.cpu(), torch.arange(top, dtype=torch.int32).expand(50, top))
    assert float((zw.cpu() - 1.0 / top).abs().max()) <= 1e-6


class NoContext:
    """A feed-forward reads nothing of a step's context."""


def moe_harness(dtype, H, E, top, F, limit, identity, shared, seed):
    from gesso_amd.config import RoutedMoESpec
    from test_gpu_parts import Harness
    spec = RoutedMoESpec(hidden=H, n_experts=E, top=top, expert_ff=F, limit=limit, n_identity=identity,
                         shared_ff=None if shared is None else shared[0], shared_limit=None if shared is None else shared[1])
    h = Harness("ffn", spec, dtype, seed=seed, std=0.3)
    t = h.tensors
    w = {"m.router": t["router.weight"], "m.correction": t["router.correction"]}
    for e in range(E):
        for k in ("gate", "up", "down"):
            w[f"m.e{e}.{k}"] = t[f"experts.{e}.{k}.weight"]
    if shared is not None:
        for k in ("gate", "up", "down"):
            w[f"m.shared.{k}"] = t[f"shared.{k}.weight"]
    mlp = {"router": {"experts": E, "top": top, "identity": identity}, "expert": {"ff": F, "limit": limit},
           "shared": None if shared is None else {"ff": shared[0], "limit": shared[1]}}
    return h, (lambda x: P.moe(x.double(), w, "m", mlp)), w, mlp


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("H,E,top,F,limit,identity,shared", [(96, 6, 2, 40, 1.0, 2, (48, 2.0)), (64, 3, 1, 16, 0.7, 0, None),
                                                             (64, 4, 4, 24, 3.0, 0, (16, 0.5)), (64, 2, 3, 8, 1.0, 2, (40, 4.0)),
                                                             (100, 7, 3, 12, 0.5, 3, (36, 2.5)), (256, 12, 2, 48, 1.5, 3, (80, 2.0)),
                                                             (128, 8, 2, 64, 1.0, 2, (64, 2.0))])
def test_routed_experts_alone_with_identity_experts_and_a_shared_one(dtype, H, E, top, F, limit, identity, shared):
    h, plain, w, mlp = moe_harness(dtype, H, E, top, F, limit, identity, shared, seed=40 + E)
    for T in (1, 7, 70, 200):                                    # token by token, and sorted by expert
        x = (torch.randn(T, H, generator=gen(T)) * 2).to(dtype)
        got = h.part.forward(x.to(DEV), NoContext()).double().cpu()
        want = plain(x)
        # tokens whose choice is a close call are left out (float32 against float64 may choose otherwise)
        s = torch.softmax(P.linear(x.double(), w["m.router"]), -1) + w["m.correction"]
        m = torch.sort(s, descending=True).values
        clear = (m[:, top - 1] - m[:, top]) > 1e-4 if top < s.shape[1] else torch.ones(T, dtype=torch.bool)
        assert int(clear.sum()) >= (T + 1) // 2
        assert float((got[clear] - want[clear]).abs().max()) <= tol(dtype, want, 3e-5, 3e-2), T
        # a token's row does not depend on its neighbours in the batch
        alone = h.part.forward(x[T // 2:T // 2 + 1].to(DEV), NoContext()).double().cpu()
        assert float((alone[0] - got[T // 2]).abs().max()) <= tol(dtype, want, 2e-6, 1.6e-2)
    # the clamps bite: inputs this large push gates and ups past the limit
    x = (torch.randn(9, H, generator=gen(99)) * 2).double()
    g = P.linear(x, w["m.e0.gate"])
    assert float(g.max()) > limit and float(P.linear(x, w["m.e0.up"]).min()) < -limit


@pytest.mark.parametrize("dtype", DTYPES)
def test_identity_experts_give_back_the_input(ops, dtype):
    """Every token is sent to the two identity experts (their corrections are huge): the output is the input, whatever
    the experts' weights hold; with one identity expert and one real one it is their weighted sum."""
    H, E, F = 64, 3, 16
    h, plain, w, mlp = moe_harness(dtype, H, E, 2, F, 1.0, 2, None, seed=7)
    x = torch.randn(80, H, generator=gen(8)).to(dtype)
    for corr in ([0, 0, 0, 50.0, 60.0], [0, 70.0, 0, 0, 60.0]):
        h.part.correction = torch.tensor(corr, dtype=torch.float32, device=DEV)
        w["m.correction"] = torch.tensor(corr, dtype=torch.float64)
        for T in (3, 80):
            got = h.part.forward(x[:T].to(DEV), NoContext()).double().cpu()
            want = plain(x[:T])
            assert float((got - want).abs().max()) <= tol(dtype, want, 3e-5, 2e-2)
            if corr[1] == 0:
                assert float((got - x[:T].double()).abs().max()) <= tol(dtype, want, 1e-5, 1e-2)


# ------------------------------------------------------------------ the mixers alone, with their own caches

def state_harness(dtype, W=96, H=4, P_=16, N=24, G=2, norm_groups=2, taps=4, page_size=8, num_pages=16, seed=5):
    from gesso_amd.config import StateSpaceSpec
    from test_gpu_parts import Harness
    spec = StateSpaceSpec(hidden=W, n_heads=H, head_dim=P_, state=N, groups=G, norm_groups=norm_groups, conv_taps=taps, eps=1e-6)
    h = Harness("mixer", spec, dtype, seed=seed, page_size=page_size, num_pages=num_pages, std=0.25)
    # decays from almost none to fast, step-size biases and skips that matter
    sharp = {"A_log": torch.linspace(-7.0, 0.5, H), "dt_bias": torch.linspace(-3.0, 1.0, H), "D": torch.linspace(0.6, 1.4, H)}
    for k, v in sharp.items():
        h.tensors[k] = v.double()
    h.part.a_log, h.part.dt_bias, h.part.d_skip = (sharp[k].to(DEV) for k in ("A_log", "dt_bias", "D"))
    t = h.tensors
    w = {"m.in": t["in_proj.weight"], "m.conv": t["conv.weight"], "m.conv.b": t["conv.bias"], "m.dt_bias": t["dt_bias"],
         "m.A_log": t["A_log"], "m.D": t["D"], "m.norm": t["norm.weight"], "m.o": t["out_proj.weight"]}
    mx = {"heads": H, "vdim": P_, "state": N, "groups": G, "norm_groups": norm_groups, "conv": taps}
    return h, lambda x: P.mamba2(x.double(), w, "m", mx, 1e-6)


def latent_harness(dtype, W=96, H=3, n=24, r=8, dv=16, qr=40, c=48, base=1e4, page_size=8, num_pages=96, seed=6):
    from gesso_amd.config import LatentAttentionSpec, NoPositionSpec, RopeSpec
    from test_gpu_parts import Harness
    pos = RopeSpec(head_dim=r, rotary_dim=r, theta=base, max_position=512, layout="interleaved") if r else NoPositionSpec()
    spec = LatentAttentionSpec(hidden=W, n_heads=H, plain_dim=n, rot_dim=r, value_dim=dv, q_rank=qr, kv_rank=c, scale=0.2,
                               eps=1e-6, position=pos, window=None, gated=True, gate_each=True)
    h = Harness("mixer", spec, dtype, seed=seed, page_size=page_size, num_pages=num_pages, std=0.25)
    t = h.tensors
    w = {"m.dq": t["q_down.weight"], "m.dq.norm": t["q_norm.weight"], "m.uq": t["q_up.weight"], "m.dkv": t["kv_down.weight"],
         "m.dkv.norm": t["kv_norm.weight"], "m.uk": t["k_up.weight"], "m.uv": t["v_up.weight"], "m.g": t["gate.weight"],
         "m.o": t["out.weight"]}
    mx = {"heads": H, "dim": n, "rot_dim": r, "vdim": dv, "kv_rank": c, "scale": 0.2, "rot": {"base": base, "dims": r}}
    return h, lambda x: P.latent_attention(x.double(), w, "m", mx, 1e-6, list(range(x.shape[0])))


def harness(kind, dtype, **kw):
    return state_harness(dtype, **kw) if kind == "state" else latent_harness(dtype, **kw)


CASES = [("state", dict()), ("state", dict(W=64, H=3, P_=24, N=16, G=1, norm_groups=3, taps=3)),
         ("state", dict(W=64, H=6, P_=8, N=12, G=3, norm_groups=6, taps=2)), ("state", dict(W=128, H=2, P_=64, N=64, G=1, norm_groups=1, taps=4)),
         ("state", dict(W=100, H=5, P_=10, N=7, G=5, norm_groups=2, taps=1)), ("state", dict(W=128, H=2, P_=128, N=128, G=2, norm_groups=1, taps=5)),
         ("state", dict(W=128, H=8, P_=32, N=40, G=4, norm_groups=2, taps=4)),
         ("latent", dict()), ("latent", dict(W=64, H=2, n=8, r=16, dv=24, qr=24, c=32)),
         ("latent", dict(W=64, H=1, n=24, r=8, dv=16, qr=16, c=36, base=100.0)), ("latent", dict(W=100, H=5, n=0, r=6, dv=14, qr=18, c=22, base=3e4)),
         ("latent", dict(W=100, H=2, n=18, r=2, dv=6, qr=10, c=30)), ("latent", dict(W=128, H=4, n=64, r=64, dv=64, qr=64, c=128, base=5e5, page_size=16)),
         ("latent", dict(W=160, H=6, n=32, r=32, dv=64, qr=72, c=128, base=1e5, page_size=16)), ("latent", dict(W=64, H=2, n=16, r=0, dv=8, qr=16, c=32))]


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("kind,kw", CASES)
def test_mixers_whole_token_by_token_in_portions_and_in_batches(dtype, kind, kw):
    h, plain = harness(kind, dtype, **kw)
    W = kw.get("W", 96)
    T = 90
    x = torch.randn(T, W, generator=gen(40)).to(dtype)
    want = plain(x)
    bound = tol(dtype, want, 5e-5, 3e-2)
    whole = h.mixer(x, [("whole", T)])
    assert float((whole - want).abs().max()) <= bound
    # most of it at once, the rest token by token
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
@pytest.mark.parametrize("kw", [dict(), dict(W=128, H=2, P_=64, N=64, G=1, norm_groups=1, taps=4)])
def test_state_mixer_with_portions_long_enough_for_segments(dtype, kw):
    """A prompt of several segments whole; the same in two long portions and single tokens; a long portion of one request
    beside a single token of another."""
    h, plain = state_harness(dtype, **kw)
    W = kw.get("W", 96)
    T = 700
    x = torch.randn(T, W, generator=gen(43)).to(dtype)
    want = plain(x)
    bound = tol(dtype, want, 5e-5, 3e-2)
    assert float((h.mixer(x, [("whole", T)]) - want).abs().max()) <= bound
    got = [h.mixer(x[:300], [("cut", 300)]), h.mixer(x[300:301], [("cut", 1)]), h.mixer(x[301:690], [("cut", 389)])]
    got += [h.mixer(x[i:i + 1], [("cut", 1)]) for i in range(690, T)]
    assert float((torch.cat(got) - want).abs().max()) <= bound
    y = torch.randn(30, W, generator=gen(44)).to(dtype)
    h.mixer(y[:29], [("b", 29)])
    h.mixer(x[:130], [("a", 130)])
    out = h.mixer(torch.cat([y[29:30], x[130:500]]), [("b", 1), ("a", 370)])
    assert float((out[0] - plain(y)[29]).abs().max()) <= bound
    assert float((out[1:] - want[130:500]).abs().max()) <= bound


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("kind", ["state", "latent"])
def test_mixers_with_pages_and_slots_freed_and_used_again(dtype, kind):
    """A pool that holds little more than one request's rows, and four slots: requests come and go, every later one
    writes pages and a slot that an earlier one gave back (filled with NaN in between)."""
    h, plain = harness(kind, dtype, page_size=8, num_pages=9)
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
@pytest.mark.parametrize("ps", [8, 16])
def test_a_token_that_stands_out_is_attended_far_back_and_at_page_borders(dtype, ps):
    """The shared rotated key part is the one part of a cached row that no norm rescales: the input row of one token is
    scaled up (its latent keeps its size, its rotated part grows), with the sign that makes the last query's heads look
    at it.  The plain mixer's output at the query must then depend on that token, and the mixer must agree with it:
    300 tokens back, on a page's last and first row, at the very first token, whole and with the query fed alone."""
    T = 340
    query = T - 1
    # a large base: most pairs hardly turn over 340 tokens, so the scaled part's score keeps its size at any distance
    h, plain = latent_harness(dtype, W=64, H=2, n=8, r=16, dv=16, qr=24, c=32, base=1e9, page_size=ps, num_pages=2 * (T // ps + 2))
    base_x = torch.randn(T, 64, generator=gen(70)).to(dtype)
    quiet = plain(base_x)
    seen = 0
    for place in (query - 300, (query // ps) * ps, (query // ps) * ps - 1, 0, ps - 1, ps, query - 1):
        for sign in ((40.0, -40.0) if dtype == torch.float32 else (8.0, -8.0)):     # (sixteen-bit scores of 80 say little)
            x = base_x.clone()
            x[place] = (x[place].double() * sign).to(dtype)
            want = plain(x)
            moved = float((want[query] - quiet[query]).abs().max())
            whole = h.mixer(x, [("w", T)])
            h.manager.release("w")
            h.mixer(x[:query], [("t", query)])
            alone = h.mixer(x[query:], [("t", 1)])
            h.manager.release("t")
            bound = tol(dtype, want, 5e-5, 6e-2)
            assert float((whole - want).abs().max()) <= bound, (place, sign)
            assert float((alone[0] - want[query]).abs().max()) <= bound, (place, sign)
            seen += moved > (5 if dtype == torch.float32 else 2) * bound
    assert seen >= (7 if dtype == torch.float32 else 4)       # for every place one of the signs draws the query's weight


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
    for close calls of a router (a token at which the last chosen output leads the best one left out by less than
    sixteen-bit activations resolve; the engine and the rounded plain model may then choose differently, that row
    stands far off, and what the token leaves in states and caches reaches later rows faintly): most rows must stand as
    near to the plain model as the rounded model does, by the measure of ``noise.py``: nine in ten within its factor
    for a row, and half of them within half of it."""
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
def test_the_residual_stream_after_every_layer_run(name, folders):
    """float32: the stream as every layer run leaves it (a looped layer counts each time), the two results a block
    leaves beside the stream added, against the plain model's."""
    from gesso_amd.engine.batch import StepEntry
    from gesso_amd.engine.engine import Engine
    cfg, seed = CONFIGS[name]
    model_dir = write_tiny(folders, name, torch.float32)
    ids = random_ids(29, cfg.vocab, 5 * seed)
    want = []
    P.forward(P.read_config(model_dir), P.read_weights(model_dir), ids, layers_out=want)
    eng = Engine.from_folder(model_dir, dtype="float32", device=DEV, page_size=16, max_tokens=256, num_slots=4)
    got = []
    for b in set(eng.model.blocks):
        def wrapped(stream, ctx, cache, orig=b.forward):
            orig(stream, ctx, cache)
            x = stream.res.double().cpu()
            pend = stream.pending if isinstance(stream.pending, tuple) else (stream.pending,)
            got.append(x + sum(d.double().cpu() for d in pend if d is not None))
        b.forward = wrapped
    eng.add_request("r")
    eng.step([StepEntry("r", ids[:17], [])])
    first = list(got)
    got.clear()
    eng.step([StepEntry("r", ids[17:], [])])
    assert len(first) == len(got) == len(want) == len(P.run_order(P.read_config(model_dir)))
    for i, w in enumerate(want):
        mine = torch.cat([first[i], got[i]])
        assert float((mine - w).abs().max()) <= 3e-5 * max(1.0, float(w.abs().max())), f"layer run {i}"


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
        plain.check(mine, f"Togalorn {name} {way}")


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", ["A", "D"])
def test_long_decoding_token_by_token(name, dtype, folders, tmp_path):
    """A short prompt, then three hundred tokens one by one: states carried, histories moved on and pages begun many
    times over."""
    cfg, seed = CONFIGS[name]
    model_dir = write_tiny(folders, name, torch.float32 if dtype == "float32" else torch.bfloat16)
    seqs = {"long": random_ids(330, cfg.vocab, 7000 + seed), "other": random_ids(301, cfg.vocab, 7100 + seed)}
    plain = R.Plain(model_dir, seqs, dtype)
    got, rc = R.run_trace(model_dir, dtype, str(tmp_path / "out"), R.trace_tail(seqs, tail=300), cfg.vocab)
    assert rc == 0 and {k: len(v) for k, v in got.items()} == {"long": 330, "other": 301}
    check_rows(plain, got, dtype, f"Togalorn {name}, 300 tokens one by one")


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
        plain.check(got, f"Togalorn {name}, pages of 8, poisoned, {way}")


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
        for g, p in zip(got, prompts):
            lg = P.forward(pc, pw16, g).numpy()
            assert all(supported(lg[i - 1], g[i], 0.5) for i in range(len(p), len(g)))
    finally:
        session.close()


def test_the_command_line_serves_a_togalorn_folder(folders):
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
    """More requests than the engine has had slots for in the tests above: forty states, histories and block tables side
    by side.  Every token chosen is one the plain model ranks near its best at that place, and so is every token the
    first request gets when it runs alone."""
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
    assert [len(g) for g in got] == [len(p) + 10 for p in prompts]
    for i in (0, 17, 39):
        lg = P.forward(pc, pw, got[i]).numpy()
        assert all(supported(lg[j - 1], got[i][j], 0.5) for j in range(len(prompts[i]), len(got[i]))), i
    lg = P.forward(pc, pw, alone).numpy()
    assert all(supported(lg[j - 1], alone[j], 0.5) for j in range(len(prompts[0]), len(alone)))


def random_togalorn(seed: int):
    """A configuration drawn from a seed: two to four layers of either kind in any order, a loop anywhere or none, sizes
    with and without whole tiles, one to five taps or no input convolution, layers without a feed-forward, with and
    without identity and shared experts."""
    import random
    from gesso_amd.config import (ExpertConfig, LatentMixerConfig, LoopConfig, Mamba2MixerConfig, MoEConfig, TogalornConfig,
                                  TogalornLayer)
    rng = random.Random(seed)
    width = rng.choice([64, 72, 96, 128, 160])

    def mlp():
        if rng.random() < 0.15:
            return None
        E, identity = rng.choice([1, 2, 3, 5, 8]), rng.choice([0, 0, 1, 2, 4])
        top = rng.randint(1, min(4, E + identity))
        shared = None if rng.random() < 0.3 else ExpertConfig(rng.choice([8, 20, 32, 64]), rng.choice([0.5, 1.0, 2.0, 7.0]))
        return MoEConfig(E, top, identity, ExpertConfig(rng.choice([8, 12, 24, 40, 64]), rng.choice([0.5, 1.0, 1.5, 7.0])), shared)

    layers = []
    for _ in range(rng.randint(2, 4)):
        if rng.random() < 0.5:
            G = rng.choice([1, 2, 3])
            H = G * rng.choice([1, 2, 3])
            P_ = rng.choice([4, 8, 10, 16, 32, 64])
            ng = rng.choice([g for g in (1, 2, 3, 4, H) if (H * P_) % g == 0])
            layers.append(TogalornLayer("mamba2", Mamba2MixerConfig(H, P_, rng.choice([4, 7, 16, 24, 48, 64, 100]), G, ng,
                                                                    rng.choice([1, 2, 3, 4, 5])), mlp()))
        else:
            r = rng.choice([0, 2, 6, 8, 16, 32, 64])
            n = rng.choice([0, 4, 8, 18, 32, 64]) if r else rng.choice([4, 8, 18, 32, 64])
            layers.append(TogalornLayer("latent_attention", LatentMixerConfig(
                rng.choice([1, 2, 3, 5, 6]), n, r, rng.choice([4, 6, 16, 24, 32, 64]), rng.choice([10, 16, 24, 40, 80]),
                rng.choice([22, 32, 48, 64, 128]), rng.choice([0.08, 0.125, 0.2, 0.3]), rng.choice([1e2, 1e4, 5e5])), mlp()))
    n = len(layers)
    loop = None
    if rng.random() < 0.75:
        a = rng.randint(0, n - 1)
        loop = LoopConfig(a, rng.randint(a + 1, n), rng.choice([1, 2, 3]))
    groups = rng.choice([g for g in (1, 2, 3, 4, 8) if width % g == 0])
    return TogalornConfig(vocab=rng.choice([97, 200, 333, 512]), width=width, norm_eps=rng.choice([1e-5, 1e-6, 1e-4]),
                          norm_groups=groups, embedding_scale=rng.choice([1.0, 3.0, math.sqrt(width)]),
                          canon_taps=rng.choice([None, 1, 2, 3, 4, 5]), loop=loop, max_position=512, layers=tuple(layers))


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("seed", [71, 72, 73, 74, 75, 76, 77, 78])
def test_replay_of_configurations_drawn_at_random(seed, dtype, tmp_path):
    import random
    cfg = random_togalorn(seed)
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
        check_rows(plain, mine, dtype, f"Togalorn drawn from {seed}, {way}")
