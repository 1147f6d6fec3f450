"""Vumalix on the device: each mechanism's kernels against the plain implementation, then whole models under every
way of cutting requests into steps, and generation through the entry points."""
from __future__ import annotations

import json
import math
import os
import subprocess
import sys
from types import SimpleNamespace

import numpy as np
import pytest
import torch

import helpers
from plain import vumalix as pv
from vumalix_cases import CASES, folder_of, rounded

pytestmark = pytest.mark.gpu
F64 = torch.float64
DEV = "cuda:0"


def _dev(t, dtype=torch.float32):
    return t.to(dtype).to(DEV).contiguous()


def _i32(values):
    return torch.tensor(list(values), dtype=torch.int32, device=DEV)


def _step_ctx(rows, slots):
    """The tables of a step whose requests bring ``rows`` = [(request, first position, end position)], in that order."""
    lens = [b - a for _, a, b in rows]
    starts = np.cumsum([0] + lens)[:-1]
    tok_seq = [s for s, n in enumerate(lens) for _ in range(n)]
    return SimpleNamespace(q_start=_i32(starts), q_len=_i32(lens), pos0=_i32(a for _, a, _ in rows), tok_seq=_i32(tok_seq),
                           state_slots=_i32(slots[r] for r, _, _ in rows), num_seqs=len(rows), host={"max_q_len": max(lens)})


# ------------------------------------------------------------------------------------------ the convolution of the residual
@pytest.mark.parametrize("d, taps, dtype", [(64, 4, torch.float32), (50, 2, torch.bfloat16), (24, 8, torch.float32), (16, 1, torch.float32),
                                            (40, 0, torch.bfloat16), (96, 5, torch.bfloat16), (7, 3, torch.float32)])
def test_the_convolution_of_the_residual_in_portions(d, taps, dtype):
    """Three requests whose tokens come in four steps of unequal portions (single tokens, portions shorter than the
    convolution, long ones; the first and third steps bring single tokens only, so the kernel moves the slots on itself)
    into slots that hold garbage: x + conv(x) against the plain function, and the slots after every step."""
    from glassbox_amd import ops
    torch.manual_seed(d + taps)
    lens = {0: 23, 1: 3, 2: 9}
    cuts = {0: (1, 20, 1, 1), 1: (1, 1, 0, 1), 2: (1, 2, 1, 5)}
    slots = {0: 2, 1: 0, 2: 3}
    w = torch.randn(d, taps).float() if taps else None
    state = torch.full((5, max(taps - 1, 1), d), 55.0, device=DEV) if taps > 1 else None
    data = {r: torch.randn(T, d).float().to(F64) for r, T in lens.items()}
    want = {r: pv.mixer_input(x, w.to(F64) if taps else None) for r, x in data.items()}
    tol = 1e-5 if dtype == torch.float32 else 1e-2
    done = {r: 0 for r in lens}
    for step in range(4):
        rows = [(r, done[r], done[r] + cuts[r][step]) for r in lens if cuts[r][step]]
        rows.sort(key=lambda x: x[2] - x[1] > 1)
        ctx = _step_ctx(rows, slots)
        n = sum(b - a for _, a, b in rows)
        x = _dev(torch.cat([data[r][a:b] for r, a, b in rows], 0))
        out = torch.full((n, d + 3), 9.0, dtype=dtype, device=DEV)[:, :d]   # rows wider than the residual
        ops.time_conv(x, _dev(w.t()) if taps else None, state, ctx, out)
        got, at = out.cpu().to(F64), 0
        for r, a, b in rows:
            assert (got[at:at + b - a] - want[r][a:b]).abs().max() < tol * max(1.0, float(want[r].abs().max())), (step, r)
            at += b - a
            done[r] = b
            if state is not None:
                kept = state[slots[r]].cpu().to(F64)
                assert all(torch.equal(kept[i], data[r][b - (taps - 1) + i]) for i in range(taps - 1) if b - (taps - 1) + i >= 0)
    if state is not None:
        assert torch.all(state[1] == 55.0) and torch.all(state[4] == 55.0)   # nobody else's slot was touched


@pytest.mark.parametrize("d, taps, dtype", [(64, 4, torch.bfloat16), (40, 8, torch.float32), (128, 2, torch.float32), (8, 1, torch.bfloat16)])
def test_the_convolution_in_long_portions(d, taps, dtype):
    """Steps of several hundred rows (the kernel that takes four tokens a thread): three requests whose portions begin and
    end at any token of a group of four, a second step that reads what the first left in the slots, and a request that
    joins with a portion shorter than the convolution."""
    from glassbox_amd import ops
    torch.manual_seed(3 * d + taps)
    lens = {0: 571, 1: 333, 2: 263}
    cuts = {0: (301, 270), 1: (2, 331), 2: (0, 263)}
    slots = {0: 1, 1: 4, 2: 0}
    w = torch.randn(d, taps).float()
    state = torch.full((5, max(taps - 1, 1), d), 55.0, device=DEV) if taps > 1 else None
    data = {r: torch.randn(T, d).float().to(F64) for r, T in lens.items()}
    want = {r: pv.mixer_input(x, w.to(F64)) for r, x in data.items()}
    tol = 1e-5 if dtype == torch.float32 else 1e-2
    done = {r: 0 for r in lens}
    for step in range(2):
        rows = [(r, done[r], done[r] + cuts[r][step]) for r in lens if cuts[r][step]]
        ctx = _step_ctx(rows, slots)
        x = _dev(torch.cat([data[r][a:b] for r, a, b in rows], 0))
        out = torch.full((x.shape[0], d + 4), 9.0, dtype=dtype, device=DEV)[:, :d]
        ops.time_conv(x, _dev(w.t()), state, ctx, out)
        got, at = out.cpu().to(F64), 0
        for r, a, b in rows:
            assert (got[at:at + b - a] - want[r][a:b]).abs().max() < tol * max(1.0, float(want[r].abs().max())), (step, r)
            at += b - a
            done[r] = b
            if state is not None:
                kept = state[slots[r]].cpu().to(F64)
                assert all(torch.equal(kept[i], data[r][b - (taps - 1) + i]) for i in range(taps - 1) if b - (taps - 1) + i >= 0)
    if state is not None:
        assert torch.all(state[2] == 55.0) and torch.all(state[3] == 55.0)


# ------------------------------------------------------------------------------------------ norms and the polynomial
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_norms_of_slices_the_polynomial_the_gate_and_the_normed_add(dtype):
    from glassbox_amd import ops
    torch.manual_seed(9)
    f = lambda t: t.to(dtype).to(F64)
    tol = 2e-5 if dtype == torch.float32 else 2e-2
    for n, a, b, rest in ((5, 24, 40, 9), (70, 7, 13, 0), (3, 300, 520, 64)):
        rows = f(torch.randn(n, a + b + rest, dtype=F64) * 2)
        ga, gb = torch.rand(a).to(F64) + 0.5, torch.rand(b).to(F64) + 0.5
        oa, ob = torch.empty(n, a, dtype=dtype, device=DEV), torch.empty(n, b + 2, dtype=dtype, device=DEV)[:, :b]
        ops.norm_slices(_dev(rows, dtype), 1e-5, (0, _dev(ga), oa), (a, _dev(gb), ob))
        assert (oa.cpu().to(F64) - pv.unit_rms(rows[:, :a], 1e-5) * ga).abs().max() < tol * 3
        assert (ob.cpu().to(F64) - pv.unit_rms(rows[:, a:a + b], 1e-5) * gb).abs().max() < tol * 3
        one = torch.empty(n, b, dtype=dtype, device=DEV)
        ops.norm_slices(_dev(rows, dtype), 1e-5, (a, _dev(gb), one))
        assert torch.equal(one, ob)
    for n, ff in ((4, 96), (33, 30), (2, 5000)):
        z = f(torch.randn(n, ff, dtype=F64) * 1.5)
        coef = torch.tensor([0.6, -0.3, 0.2, 0.1]).to(F64)
        out = torch.empty(n, ff, dtype=dtype, device=DEV)
        ops.poly_norm(_dev(z, dtype), _dev(coef), 1e-5, out)
        want = pv.poly_norm(z, coef, 1e-5)
        assert (out.cpu().to(F64) - want).abs().max() < tol * float(want.abs().max())
    for n, H, hc, V in ((6, 4, 32, 16), (65, 3, 48, 48), (2, 2, 136, 40)):
        att, gate = f(torch.randn(n, H, hc, dtype=F64)), f(torch.randn(n, H * V + 8, dtype=F64) * 3)
        out = torch.empty(n, H * V, dtype=dtype, device=DEV)
        ops.gate_heads(_dev(att.reshape(n, -1), dtype), hc, _dev(gate, dtype)[:, 3:3 + H * V], out, H, V)
        want = att[:, :, :V] * torch.sigmoid(gate[:, 3:3 + H * V]).view(n, H, V)
        assert (out.cpu().to(F64).view(n, H, V) - want).abs().max() < tol * 2
    for n, d in ((5, 64), (300, 50), (2, 2048)):
        x, y, g = torch.randn(n, d).to(F64), (torch.randn(n, d) * 7).to(F64), torch.tensor([-0.35]).to(F64)
        xd = _dev(x)
        r = torch.empty(n, d, dtype=dtype, device=DEV)
        ops.norm_add(xd, _dev(y), _dev(g), 1e-5, r)
        want = x + pv.scalar_norm(y, g, 1e-5)
        assert (xd.cpu().to(F64) - want).abs().max() < 2e-6 and (r.cpu().to(F64) - want).abs().max() < tol * 2
        ops.norm_add(xd, _dev(y), _dev(g), 1e-5)
        assert (xd.cpu().to(F64) - want - pv.scalar_norm(y, g, 1e-5)).abs().max() < 4e-6


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_rows_in_registers_many_rows_and_few(dtype):
    """The polynomial and the normed add keep a row in registers, with other threads a row for many rows than for few."""
    from glassbox_amd import ops
    torch.manual_seed(21)
    f = lambda t: t.to(dtype).to(F64)
    tol = 2e-5 if dtype == torch.float32 else 2e-2
    for n, ff in ((3, 1536), (700, 264), (520, 8200)):
        z = f(torch.randn(n, ff, dtype=F64) * 1.5)
        coef = torch.tensor([0.5, 0.4, -0.2, 0.3]).to(F64)
        out = torch.empty(n, ff + 8, dtype=dtype, device=DEV)[:, :ff]
        ops.poly_norm(_dev(z, dtype), _dev(coef), 1e-5, out)
        want = pv.poly_norm(z, coef, 1e-5)
        assert (out.cpu().to(F64) - want).abs().max() < tol * float(want.abs().max())
    for n, d in ((600, 72), (513, 4100)):
        x, y, g = torch.randn(n, d).to(F64), (torch.randn(n, d) * 3).to(F64), torch.tensor([0.8]).to(F64)
        xd, r = _dev(x), torch.empty(n, d, dtype=dtype, device=DEV)
        ops.norm_add(xd, _dev(y), _dev(g), 1e-5, r)
        want = x + pv.scalar_norm(y, g, 1e-5)
        assert (xd.cpu().to(F64) - want).abs().max() < 4e-6 and (r.cpu().to(F64) - want).abs().max() < tol * 2


def test_a_product_left_in_slices_and_the_normed_add_that_adds_them():
    """``gemm_partial`` leaves the sums over the runs of k side by side; their sum is the product, and ``norm_add`` with
    ``slices`` gives what it gives of the whole product."""
    from glassbox_amd import ops
    torch.manual_seed(4)
    for n, width, k in ((40, 64, 2048), (600, 128, 8192)):
        slices = ops.gemm_slices(n, width, k)
        assert slices > 1 and ops.gemm_split_floats(n, width, k) >= slices * n * width
        a, w = (torch.randn(n, k) * 0.5).to(torch.bfloat16), (torch.randn(width, k) * 0.1).to(torch.bfloat16)
        ws = torch.full((ops.gemm_split_floats(n, width, k) + 16,), 7.0, device=DEV)
        assert ops.gemm_partial(a.to(DEV), w.to(DEV), ws) == slices
        whole = torch.empty(n, width, device=DEV)
        ops.gemm(a.to(DEV), w.to(DEV), whole, workspace=torch.empty_like(ws))
        parts = ws[:slices * n * width].view(slices, n, width)
        assert (parts.to(F64).sum(0) - whole.to(F64)).abs().max() < 1e-4
        assert (whole.cpu().to(F64) - a.to(F64) @ w.to(F64).T).abs().max() < 2e-3
        assert torch.all(ws[slices * n * width:] == 7.0)
        x, g = torch.randn(n, width).to(F64), torch.tensor([1.7]).to(F64)
        one, two = _dev(x), _dev(x)
        r1, r2 = (torch.empty(n, width, dtype=torch.bfloat16, device=DEV) for _ in range(2))
        ops.norm_add(one, whole, _dev(g), 1e-5, r1)
        ops.norm_add(two, ws, _dev(g), 1e-5, r2, slices=slices)
        assert torch.equal(one, two) and torch.equal(r1, r2)
        assert (one.cpu().to(F64) - x - pv.scalar_norm(whole.cpu().to(F64), g, 1e-5)).abs().max() < 4e-6


@pytest.mark.parametrize("d, taps, dtype", [(64, 4, torch.float32), (96, 5, torch.bfloat16), (24, 2, torch.bfloat16), (16, 1, torch.float32)])
def test_the_normed_add_that_makes_the_next_convolutions_rows(d, taps, dtype):
    """Steps of single tokens: the pass that adds a normed sublayer into the residual also writes x + conv(x) of the new
    residual and moves the slots on.  One request begins in a portion that ``time_conv`` takes, the other at its first
    token in a slot that holds garbage; a third joins later."""
    from glassbox_amd import ops
    torch.manual_seed(d * taps)
    K = taps - 1
    lens = {0: 12, 1: 7, 2: 4}
    begin = {0: 0, 1: 0, 2: 3}            # the step in which a request begins (request 0 with a portion of 5)
    slots = {0: 3, 1: 1, 2: 0}
    w = torch.randn(d, taps).float()
    g = torch.tensor([0.7])
    state = torch.full((5, max(K, 1), d), 55.0, device=DEV) if K else None
    xs = {r: torch.randn(T, d).float() for r, T in lens.items()}           # the residual before the sublayer's rows are added
    ys = {r: (torch.randn(T, d) * 4).float() for r, T in lens.items()}
    new = {r: xs[r].to(F64) + pv.scalar_norm(ys[r].to(F64), g.to(F64), 1e-5) for r in lens}
    want = {r: pv.mixer_input(new[r], w.to(F64)) for r in lens}
    tol = 2e-5 if dtype == torch.float32 else 2e-2
    # request 0's first five rows in one portion: the residual as it is after the add, through the convolution's own kernel
    ctx = _step_ctx([(0, 0, 5)], slots)
    out = torch.empty(5, d, dtype=dtype, device=DEV)
    ops.time_conv(_dev(new[0][:5]), _dev(w.t()), state, ctx, out)
    assert (out.cpu().to(F64) - want[0][:5]).abs().max() < tol * float(want[0].abs().max())
    done = {0: 5, 1: 0, 2: 0}
    for step in range(8):
        rows = [(r, done[r], done[r] + 1) for r in lens if step >= begin[r] and done[r] < lens[r]]
        if not rows:
            break
        ctx = _step_ctx(rows, slots)
        x = _dev(torch.stack([xs[r][a] for r, a, _ in rows]))
        y = _dev(torch.stack([ys[r][a] for r, a, _ in rows]))
        out = torch.empty(len(rows), d, dtype=dtype, device=DEV)
        ops.norm_add(x, y, _dev(g), 1e-5, out, conv=(_dev(w.t()), state), ctx=ctx)
        for i, (r, a, b) in enumerate(rows):
            assert (x[i].cpu().to(F64) - new[r][a]).abs().max() < 4e-6
            assert (out[i].cpu().to(F64) - want[r][a]).abs().max() < tol * float(want[r].abs().max()), (step, r)
            done[r] = b
            if K:
                kept = state[slots[r]].cpu().to(F64)
                assert all((kept[i2] - new[r][b - K + i2]).abs().max() < 4e-6 for i2 in range(K) if b - K + i2 >= 0)
    if K:
        assert torch.all(state[2] == 55.0) and torch.all(state[4] == 55.0)


# ------------------------------------------------------------------------------------------ heads and their attention
def _pool(T, P, G, hc, dtype):
    from glassbox_amd import ops
    pages = torch.randperm(-(-T // P) + 7)[:-(-T // P)].tolist()     # the request's pages, scattered over the pool
    slots = [pages[i // P] * P + i % P for i in range(T)]
    k_pages = torch.full(ops.key_pages_shape(-(-T // P) + 8, G, P, hc), 77.0, dtype=dtype, device=DEV)
    v_pages = torch.full((-(-T // P) + 8, G, hc, P), 77.0, dtype=dtype, device=DEV)
    return pages, slots, k_pages, v_pages


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("H, dk, dr, rot, dv, window", [(2, 16, 8, 8, 16, 37), (3, 10, 2, 2, 6, 9), (1, 24, 32, 12, 64, 0), (2, 104, 32, 32, 40, 50)])
def test_latent_heads_at_the_windows_edges_and_far_back(dtype, H, dk, dr, rot, dv, window):
    """One request of 300 keys in pages of 16.  Every query is built so that three keys would dominate its softmax: the
    oldest key of its window, the key just before it, and key 2 far back (which a model without a window reads and one
    with a window must not).  The rotated columns of the queries are made by turning them back by their own position, so
    that the kernel's rotation brings them to the wanted key.  Heads are assembled and stored fifty rows at a time."""
    from glassbox_amd import ops
    from glassbox_amd.parts.attention import cache_head_cols
    torch.manual_seed(window + dk)
    T, P, base, scale = 300, 16, 100.0, 0.3
    f = lambda t: t.to(dtype).to(F64)
    hc = cache_head_cols(dk + dr, dv)
    pos = torch.arange(T)
    k_own, k_shared, v = f(torch.randn(T, H, dk, dtype=F64)), f(torch.randn(T, dr, dtype=F64)), f(torch.randn(T, H, dv, dtype=F64))
    turn = lambda x, p: torch.cat([pv.rotate_half_split(x[..., :rot], p, base), x[..., rot:]], -1) if rot else x
    keys = f(torch.cat([k_own, turn(k_shared, pos)[:, None, :].expand(T, H, dr)], -1))
    q_final = 0.3 * torch.randn(T, H, dk + dr, dtype=F64)
    for i in range(T):
        for j in ((i - window + 1, i - window, 2) if window else (2, i - 40)):
            if 0 <= j <= i:
                q_final[i] += 3.0 * keys[j] / math.sqrt(dk + dr) * 4
    q_raw = f(torch.cat([q_final[..., :dk], turn(q_final[..., dk:], -pos)], -1))       # turned back: the kernel turns it forth
    q = f(torch.cat([q_raw[..., :dk], turn(q_raw[..., dk:], pos)], -1))
    want = pv.softmax_heads(q, keys, v, scale, pv.visible(T, window))
    if window:   # the far key and the one just outside the window would change the result if they were read
        assert (pv.softmax_heads(q, keys, v, scale, pv.visible(T, window + 1))[window + 5:] - want[window + 5:]).abs().max() > 0.1
        assert (pv.softmax_heads(q, keys, v, scale, pv.visible(T, window - 1))[window + 5:] - want[window + 5:]).abs().max() > 0.1
    else:
        assert (pv.softmax_heads(q, keys, v, scale, pv.visible(T, 200))[250:] - want[250:]).abs().max() > 0.1
    pages, slots, k_pages, v_pages = _pool(T, P, H, hc, dtype)
    ang = pos.to(F64)[:, None] * torch.tensor([base ** (-2.0 * i / rot) for i in range(rot // 2)], dtype=F64)
    heads = torch.empty(T, 3 * H * hc, dtype=dtype, device=DEV)
    kv = torch.cat([k_own.reshape(T, -1), v.reshape(T, -1)], 1)
    for a in range(0, T, 50):
        b = min(T, a + 50)
        ops.latent_heads(_dev(q_raw.reshape(T, -1)[a:b], dtype), _dev(kv[a:b], dtype), _dev(k_shared[a:b], dtype),
                         _dev(ang.cos()[a:b]), _dev(ang.sin()[a:b]), rot, heads[a:b], hc, _i32(slots[a:b]), k_pages, v_pages, H, dk, dr, dv)
    got = heads.cpu().to(F64).view(T, 3 * H, hc)
    tol = 2e-5 if dtype == torch.float32 else 3e-2
    assert (got[:, :H, :dk + dr] - q).abs().max() < tol * float(q.abs().max()) and (got[:, H:2 * H, :dk + dr] - keys).abs().max() < tol * 4
    assert (got[:, 2 * H:, :dv] - v).abs().max() < tol * 4
    assert float(got[:, :2 * H, dk + dr:].abs().max() if hc > dk + dr else 0) == 0.0 and float(got[:, 2 * H:, dv:].abs().max() if hc > dv else 0) == 0.0
    stored = ops.unpack_keys(k_pages).cpu().to(F64)
    for p in (0, 15, 16, 17, T - 1):
        assert torch.equal(stored[pages[p // P], :, p % P], got[p, H:2 * H])
        assert torch.equal(v_pages[pages[p // P], :, :, p % P].cpu().to(F64), got[p, 2 * H:])
    out = torch.empty(T, H * hc, dtype=dtype, device=DEV)
    ops.attention_plain(heads[:, :H * hc], out, _i32(range(T)), _i32([0] * T), _i32(pages).view(1, -1), k_pages, v_pages, H, scale, window)
    err = (out.cpu().to(F64).view(T, H, hc)[:, :, :dv] - want).abs().amax((1, 2))
    assert float(err.max()) < (5e-5 if dtype == torch.float32 else 4e-2), (int(err.argmax()), float(err.max()))


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("H, G, dk, dv, every", [(4, 2, 16, 24, 7), (6, 1, 8, 48, 40), (2, 2, 72, 64, 0), (2, 1, 6, 10, 3)])
def test_differential_heads_two_maps_over_one_key_head(dtype, H, G, dk, dv, every):
    """One request of 300 keys.  The first map of every query looks for key 3 far back, the second for the key before
    its own: the two maps must come out as two attentions of their own over the same values, through query heads
    [q1 | 0] and [0 | q2] and one key head [k1 | k2]; then the difference, its norm and the constant."""
    from glassbox_amd import ops
    from glassbox_amd.parts.attention import cache_head_cols
    torch.manual_seed(dk + dv)
    T, P, scale, eps, coef, diff = 300, 16, 0.9, 1e-5, 0.7, 0.3
    f = lambda t: t.to(dtype).to(F64)
    hc = cache_head_cols(2 * dk, dv)
    group = H // G
    k_raw, v = f(torch.randn(T, G, 2, dk, dtype=F64)), f(torch.randn(T, G, dv, dtype=F64))
    wq, wk = torch.rand(dk).to(F64) + 0.5, torch.rand(dk).to(F64) + 0.5
    q_raw = 0.2 * torch.randn(T, H, 2, dk, dtype=F64)
    for i in range(4, T):
        kh = k_raw[:, torch.arange(H) // group]
        q_raw[i, :, 0] += kh[3, :, 0] * wk / wq
        q_raw[i, :, 1] += kh[i - 1, :, 1] * wk / wq
    q_raw = f(q_raw)
    temp = pv.query_temperature(torch.arange(T), coef, every) if every else torch.ones(T, dtype=F64)
    q = f(pv.unit_rms(q_raw, eps) * wq * temp[:, None, None, None] * 6.0 / 6.0)
    k = f(pv.unit_rms(k_raw, eps) * wk)
    kh, vh = k.repeat_interleave(group, 1), v.repeat_interleave(group, 1)
    a1 = pv.softmax_heads(q[:, :, 0], kh[:, :, 0], vh, scale, pv.visible(T))
    a2 = pv.softmax_heads(q[:, :, 1], kh[:, :, 1], vh, scale, pv.visible(T))
    assert (a1[200:] - a2[200:]).abs().max() > 0.1
    lam = torch.tensor([0.45])
    want = pv.unit_rms(a1 - float(lam) * a2, eps) * (1 - diff)
    pages, slots, k_pages, v_pages = _pool(T, P, G, hc, dtype)
    proj = torch.cat([q_raw.reshape(T, -1), k_raw.reshape(T, -1), v.reshape(T, -1)], 1)
    heads = torch.empty(T, (2 * H + 2 * G) * hc, dtype=dtype, device=DEV)
    for a in range(0, T, 60):
        b = min(T, a + 60)
        ops.diff_heads(_dev(proj[a:b], dtype), _dev(wq), _dev(wk), eps, coef, every, _i32(range(a, b)), heads[a:b], hc,
                       _i32(slots[a:b]), k_pages, v_pages, H, G, dk, dv)
    got = heads.cpu().to(F64).view(T, 2 * H + 2 * G, hc)
    tol = 2e-5 if dtype == torch.float32 else 3e-2
    qh = got[:, :2 * H].reshape(T, H, 2, hc)
    assert (qh[:, :, 0, :dk] - q[:, :, 0]).abs().max() < tol * 4 and (qh[:, :, 1, dk:2 * dk] - q[:, :, 1]).abs().max() < tol * 4
    assert float(qh[:, :, 0, dk:].abs().max()) == 0.0 and float(qh[:, :, 1, :dk].abs().max()) == 0.0
    assert (got[:, 2 * H:2 * H + G, :2 * dk] - k.reshape(T, G, 2 * dk)).abs().max() < tol * 4
    assert (got[:, 2 * H + G:, :dv] - v).abs().max() < tol * 4
    stored = ops.unpack_keys(k_pages).cpu().to(F64)
    for p in (0, 15, 16, T - 1):
        assert torch.equal(stored[pages[p // P], :, p % P], got[p, 2 * H:2 * H + G])
        assert torch.equal(v_pages[pages[p // P], :, :, p % P].cpu().to(F64), got[p, 2 * H + G:])
    att = torch.empty(T, 2 * H * hc, dtype=dtype, device=DEV)
    ops.attention_plain(heads[:, :2 * H * hc], att, _i32(range(T)), _i32([0] * T), _i32(pages).view(1, -1), k_pages, v_pages, 2 * H, scale, 0)
    maps = att.cpu().to(F64).view(T, H, 2, hc)
    atol = 5e-5 if dtype == torch.float32 else 4e-2
    assert (maps[:, :, 0, :dv] - a1).abs().max() < atol and (maps[:, :, 1, :dv] - a2).abs().max() < atol
    out = torch.empty(T, H * dv, dtype=dtype, device=DEV)
    ops.diff_combine(att, hc, _dev(lam), 1 - diff, eps, out, H, dv)
    again = pv.unit_rms(maps[:, :, 0, :dv] - float(lam) * maps[:, :, 1, :dv], eps) * (1 - diff)   # (the norm magnifies the maps' rounding)
    assert (out.cpu().to(F64).view(T, H, dv) - again).abs().max() < (1e-4 if dtype == torch.float32 else 3e-2)
    if dtype == torch.float32:
        assert (out.cpu().to(F64).view(T, H, dv) - want).abs().max() < 2e-3
    else:   # the maps in 32-bit beside a bfloat16 result: only the result is rounded
        wide = torch.empty_like(out)
        ops.diff_combine(att.float(), hc, _dev(lam), 1 - diff, eps, wide, H, dv)
        assert (wide.cpu().to(F64).view(T, H, dv) - again).abs().max() < 1e-2 * max(1.0, float(again.abs().max()))


def test_lambda_is_a_number_of_the_weights():
    from glassbox_amd.parts.attention import DifferentialAttention
    torch.manual_seed(1)
    m = DifferentialAttention(16, 2, 1, 4, 4, 0.5, 0.3)
    t = {n: torch.randn(s.shape, device=DEV) for n, s in m.tensor_specs().items()}
    m.load(t)
    want = math.exp(float(t["lq1"] @ t["lk1"])) - math.exp(float(t["lq2"] @ t["lk2"])) + 0.3
    assert m.lam.shape == (1,) and float(m.lam) == pytest.approx(want, rel=1e-5)


# ------------------------------------------------------------------------------------------ whole models
REQUESTS = {"a": 150, "b": 77, "c": 41, "d": 3, "e": 1, "f": 97}


def _requests(vocab: int, seed: int = 0):
    return {r: helpers.random_tokens(vocab, n, seed=seed + n) for r, n in REQUESTS.items()}


_ORACLE: dict = {}


def _want(folder: str, tokens, dtype: str) -> np.ndarray:
    key = (folder, tuple(tokens), dtype)
    if key not in _ORACLE:
        cfg, w = pv.load_folder(folder)
        _ORACLE[key] = pv.forward(cfg, rounded(w) if dtype == "bfloat16" else w, list(tokens)).numpy()
    return _ORACLE[key]


def _moved_by_rounding(folder: str, tokens) -> np.ndarray:
    """How far rounding the activations to bfloat16 moves each position's logits in the plain implementation (root mean
    square over the vocabulary): what a position's sensitivity to rounding is."""
    key = (folder, tuple(tokens), "moved")
    if key not in _ORACLE:
        cfg, w = pv.load_folder(folder)
        coarse = pv.forward(cfg, rounded(w), list(tokens), coarse=True).numpy()
        _ORACLE[key] = np.sqrt(((coarse - _want(folder, tokens, "bfloat16")) ** 2).mean(1))
    return _ORACLE[key]


#: A 32-bit engine is held to helpers.TOL_F32 of the request's largest logit at every position.  A bfloat16 engine is
#: compared with the plain implementation on the weights it holds by the root mean square of a position's logit
#: differences: at most 3 times what rounding the activations moves that position in the plain implementation itself, or
#: 1 % of the request's logits' root mean square where that is more.  One sample of rounding is no sharp bound on
#: another (a position that the plain implementation's roundings happen to move little is as sensitive as its
#: neighbours): a position's movement counts as at least the median over its request; no position may be beyond one and
#: a half times its limit, and one in fifty beyond the limit itself.
BF16_TIMES, BF16_FLOOR = 3.0, 1e-2


def _check(got, folder, requests, dtype, what):
    for r, toks in requests.items():
        want = _want(folder, toks, dtype)
        if dtype == "float32":
            tol = helpers.TOL_F32 * max(1.0, float(np.abs(want).max()))
            bad = helpers.first_bad(got[r], want, tol)
            assert bad is None, f"{what}, {dtype}, request {r} ({len(toks)} tokens): position {bad[0]} is {bad[1]:.3e} off (limit {tol:.3e})"
            continue
        err = np.sqrt(((got[r] - want) ** 2).mean(1))
        moved = _moved_by_rounding(folder, toks)
        lim = np.maximum(BF16_TIMES * np.maximum(moved, np.median(moved)), BF16_FLOOR * float(np.sqrt((want ** 2).mean())))
        over = np.nonzero(err > lim)[0]
        assert over.size <= max(1, len(toks) // 50) and float((err / lim).max()) <= 1.5, (
            f"{what}, {dtype}, request {r} ({len(toks)} tokens): position {over[0]} is {err[over[0]]:.3e} off "
            f"(limit {lim[over[0]]:.3e}); {over.size} positions over their limits, worst ratio {(err / lim).max():.2f}")


def _poison(engine) -> None:
    """Garbage in every page and state slot: whatever a request reads, it must have written itself."""
    for lc in engine.layers:
        for t in (lc.k_pages, lc.v_pages, lc.state):
            if t is not None:
                t.fill_(300.0)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", list(CASES))
def test_every_way_of_cutting_requests_into_steps(model_dirs, name, dtype):
    from glassbox_amd.engine import Engine
    folder = folder_of(model_dirs.base, name)
    requests = _requests(CASES[name]["vocab"])
    mixed, peak = helpers.schedule_mixed(requests, seed=3, live=3, tail=20)
    eng = Engine(folder, dtype=dtype, max_tokens=max(peak, 192), max_seqs=3)
    _poison(eng)
    for what, steps in (("whole", helpers.schedule_whole(requests)), ("last tokens one by one", helpers.schedule_tail(requests, 60)),
                        ("portions", helpers.schedule_chunks(requests)), ("portions of two", None), ("mixed batches", mixed)):
        if what == "portions of two":
            steps = helpers.schedule_chunks({r: t for r, t in requests.items() if len(t) < 80}, (2,))
        got = helpers.replay(eng, steps)
        _check(got, folder, {r: requests[r] for r in got}, dtype, what)
        assert eng.cache.num_seqs() == 0 and eng.cache.free_state_slots() == 3
        assert all(eng.cache.used_pages(g) == 0 for g in range(len(eng.group_keys)))
        eng.cache.check_invariants()


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_long_prompts_whole_and_in_long_portions(model_dirs, dtype):
    """A prompt of 700 tokens: the windows pass many times, the temperature steps a hundred times, and the
    differential layers read every key back to the first."""
    from glassbox_amd.engine import Engine
    folder = folder_of(model_dirs.base, "A")
    requests = {"long": helpers.random_tokens(211, 700, seed=23), "short": helpers.random_tokens(211, 40, seed=22)}
    eng = Engine(folder, dtype=dtype, max_tokens=1024, max_seqs=2)
    _poison(eng)
    for what, steps in (("whole", helpers.schedule_whole(requests)), ("long portions", helpers.schedule_chunks(requests, (300, 1, 399))),
                        ("a long portion beside single tokens", [
                            {"entries": [("short", requests["short"][:39], list(range(39)))], "end": []},
                            {"entries": [("long", requests["long"], list(range(700))), ("short", requests["short"][39:], [0])],
                             "end": ["long", "short"]}])):
        got = helpers.replay(eng, steps)
        _check(got, folder, requests, dtype, what)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_long_decoding_and_layers_replayed_from_the_first_of_their_kind(model_dirs, dtype):
    """250 tokens one by one after a prompt of four (windows and pages' edges pass many times over; in bfloat16 the
    steps are replayed from graphs), with the layers of a kind replayed and with every layer walked: the same bits."""
    from glassbox_amd import ops
    from glassbox_amd.engine import Engine
    folder = folder_of(model_dirs.base, "A")
    toks = helpers.random_tokens(211, 254, seed=11)
    steps = helpers.schedule_tail({"x": toks}, 250)
    outs = []
    for tapes in (True, False):
        before = ops.TAPE_COUNTS["replayed_layers"]
        eng = Engine(folder, dtype=dtype, max_tokens=320, max_seqs=2, layer_tapes=tapes)
        outs.append(helpers.replay(eng, steps)["x"])
        if dtype == "bfloat16" and tapes:
            assert eng.decode_graphs is not None and eng.decode_graphs.replays > 200
        # layers 2 and 3 use layer 0's tensors and are replayed from its launches
        assert (ops.TAPE_COUNTS["replayed_layers"] > before) == tapes
    _check({"x": outs[0]}, folder, {"x": toks}, dtype, "long decoding")
    assert np.array_equal(outs[0], outs[1])


def test_slots_and_pages_that_are_used_again(model_dirs):
    """Two slots, six requests one after the other in pairs: a request finds the slot (the convolution's last rows) and the
    pages of one that ended, and must start from nothing."""
    from glassbox_amd.engine import Engine
    folder = folder_of(model_dirs.base, "D")
    requests = {r: helpers.random_tokens(160, n, seed=70 + n) for r, n in {"p": 50, "q": 31, "r": 18, "s": 64, "t": 2, "u": 45}.items()}
    eng = Engine(folder, dtype="float32", max_tokens=128, max_seqs=2)
    _poison(eng)
    steps, _ = helpers.schedule_mixed(requests, seed=5, live=2, tail=6)
    got = helpers.replay(eng, steps)
    _check(got, folder, requests, "float32", "slots used again")


def test_batches_of_unequal_requests_give_each_what_it_gets_alone(model_dirs):
    """In 32-bit a request's logits do not depend on what else is in its batch, beyond rounding of the sums' order."""
    from glassbox_amd.engine import Engine
    folder = folder_of(model_dirs.base, "B")
    requests = _requests(130, seed=4)
    eng = Engine(folder, dtype="float32", max_tokens=1024, max_seqs=6)
    alone = helpers.replay(eng, helpers.schedule_whole(requests))
    together = helpers.replay(eng, [{"entries": [(r, t, list(range(len(t)))) for r, t in requests.items()], "end": list(requests)}])
    for r in requests:
        assert np.abs(alone[r] - together[r]).max() < 2e-5 * max(1.0, float(np.abs(alone[r]).max()))


# ------------------------------------------------------------------------------------------ generation
def _greedy(cfg, w, prompt, n):
    toks = list(prompt)
    for _ in range(n):
        toks.append(int(torch.argmax(pv.forward(cfg, w, toks)[-1])))
    return toks[len(prompt):]


@pytest.mark.parametrize("name", ["A", "C"])
def test_greedy_generation_through_the_entry_points(model_dirs, name):
    from glassbox_amd.engine import Engine, generate, greedy
    folder = folder_of(model_dirs.base, name, seed=2)
    cfg, w = pv.load_folder(folder)
    vocab = CASES[name]["vocab"]
    prompts = [helpers.random_tokens(vocab, n, seed=50 + n) for n in (5, 44, 1, 23, 70)]
    want = [_greedy(cfg, w, p, 12) for p in prompts]
    assert any(len(set(r)) > 2 for r in want), "replies that repeat one token show nothing"
    eng = Engine(folder, dtype="float32", max_tokens=1024, max_seqs=3)
    assert greedy(eng, prompts[1], 12) == want[1]
    # the scheduler: three live requests at most, prompts in portions of at most 16 tokens beside decoding requests
    assert generate(eng, prompts, max_tokens=12, token_budget=16, max_seqs=3) == want
    assert eng.cache.num_seqs() == 0 and eng.cache.free_state_slots() == 3


def test_the_command_line_runs_the_model(model_dirs, tmp_path):
    folder = folder_of(model_dirs.base, "B", seed=2)
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    run = lambda *args, stdin=None: subprocess.run([sys.executable, os.path.join(root, "bin", "glassbox"), *args],
                                                   capture_output=True, text=True, timeout=600, input=stdin)
    r = run("generate", "--model", folder, "--prompt", "5,17,3,99,41", "-n", "8", "--dtype", "float32", "--no-prefix-cache")
    assert r.returncode == 0, r.stderr
    cfg, w = pv.load_folder(folder)
    assert [int(t) for t in r.stdout.split()] == _greedy(cfg, w, [5, 17, 3, 99, 41], 8)
    steps = [{"step": 0, "entries": [{"id": "a", "tokens": [5, 17, 3, 9], "want": [1, 3]}], "end": []},
             {"step": 1, "entries": [{"id": "a", "tokens": [8], "want": [0]}, {"id": "b", "tokens": [4, 4], "want": []}], "end": ["a"]}]
    r = subprocess.run([os.path.join(root, "bin", "trace_run"), "--model", folder, "--dtype", "float32", "--out", str(tmp_path / "o"),
                        "--max-tokens", "128"], capture_output=True, text=True, timeout=600,
                       input="".join(json.dumps(s) + "\n" for s in steps))
    assert r.returncode == 0 and r.stdout.split() == ["done", "0", "done", "1"], r.stderr
    want = pv.forward(cfg, w, [5, 17, 3, 9, 8]).numpy()
    assert np.abs(np.fromfile(tmp_path / "o" / "0.f32", dtype="<f4").reshape(2, -1) - want[[1, 3]]).max() < 1e-4
    assert np.abs(np.fromfile(tmp_path / "o" / "1.f32", dtype="<f4") - want[4]).max() < 1e-4
