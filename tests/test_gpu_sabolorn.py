"""The Sabolorn mechanisms of the layer-list host layer (include/mi355_hybrid.h) against the float64 oracle of oracle/sabolorn.py:
every new mechanism alone through its C entry point (layer norm, the state-space scan over portions and reused slots, the gate in front
of the group norm, the convolution with a bias, attention with a distance bias over scattered pages with keys that stand out far
back, at page borders and at the first tokens, the sigmoid router with group-limited choice, the small glue), then whole models
through the step engine -- whole prompts against token-by-token decoding, portions down to two tokens, unequal batches against each
request alone, pages and slots that are freed and used again, long decoding, the first tokens, sizes that are 1 or equal, absent
parts -- greedy generation through run_engine and the scheduler, and the trace runner on a checkpoint folder.  Configurations and
weights are made here."""
import ctypes
import json
import math
import os
import struct
import subprocess
import sys

import numpy as np
import pytest

torch = pytest.importorskip("torch")

from oracle import sabolorn as S                        # noqa: E402

pytestmark = pytest.mark.gpu
F32, BF16 = 0, 2


def _gpu():
    if not torch.cuda.is_available():
        pytest.fail("GPU tests need a visible MI355X")


def _st():
    return torch.cuda.current_stream().cuda_stream


def dev(a, dt=np.float32):
    return torch.from_numpy(np.ascontiguousarray(np.asarray(a).astype(dt))).cuda()


def bits(a):
    u = np.ascontiguousarray(a, np.float32).view(np.uint32)
    return ((u + 0x7FFF + ((u >> 16) & 1)) >> 16).astype(np.uint16)


def dev_dt(a, dtype):
    return dev(a) if dtype == F32 else torch.from_numpy(bits(a).view(np.int16)).cuda()


def host_dt(t, dtype):
    if dtype == F32:
        return t.cpu().numpy().astype(np.float64)
    u = t.cpu().numpy().view(np.uint16).astype(np.uint32) << 16
    return u.view(np.float32).astype(np.float64)


def empty_dt(shape, dtype):
    return torch.zeros(shape, dtype=torch.float32 if dtype == F32 else torch.int16, device="cuda")


_KEEP = []


def P(a, dt=np.float32):
    t = dev(a, dt)
    _KEEP.append(t)
    return t.data_ptr()


def ok(rc):
    assert rc == 0, rc
    torch.cuda.synchronize()
    _KEEP.clear()


def f32(a):
    return np.asarray(a, np.float32).astype(np.float64)


def tol(dtype, f=2e-5, b=1.5e-2):
    return f if dtype == F32 else b


# ------------------------------------------------------------------------------------------------------------ mechanisms alone
@pytest.mark.parametrize("dtype", [F32, BF16])
@pytest.mark.parametrize("T,W,ld", [(5, 64, 64), (3, 50, 77), (2, 1000, 1000), (1, 1, 4)])
def test_layer_norm_and_rms_norm_of_rows(lib, dtype, T, W, ld):
    """both kinds of norm over rows of a wider buffer, a second f32 copy, and the gathered form for the last norm; a large mean must
    not cost the variance its digits"""
    _gpu()
    rng = np.random.default_rng(T * W)
    x, w = f32(50.0 + 3 * rng.standard_normal((T, ld))), f32(1 + 0.3 * rng.standard_normal(W))
    for kind, want in ((1, S.layer_norm(x[:, :W], w, 1e-5)), (0, S.rms_unit(x[:, :W], 1e-5) * w)):
        out, out2 = empty_dt((T, W), dtype), torch.zeros((T, W), device="cuda")
        ok(lib.mi355_hyb_pre_norm_ex(out.data_ptr(), dtype, out2.data_ptr(), P(x), ld, P(w), T, W, kind, 1e-5, _st()))
        scale = max(1.0, np.abs(want).max())
        assert np.abs(host_dt(out, dtype) - want).max() < tol(dtype, 5e-5) * scale, kind
        assert np.abs(out2.cpu().numpy() - want).max() < 5e-5 * scale
    rows = np.array([T - 1, 0, T - 1], np.int32)
    out = empty_dt((3, W), dtype)
    xc = np.ascontiguousarray(x[:, :W])
    ok(lib.mi355_hyb_gather_norm_ex(out.data_ptr(), dtype, P(xc), P(rows, np.int32), P(w), 3, W, 1, 1e-5, _st()))
    want = S.layer_norm(xc, w, 1e-5)[rows]
    assert np.abs(host_dt(out, dtype) - want).max() < tol(dtype, 5e-5) * max(1.0, np.abs(want).max())


@pytest.mark.parametrize("heads,G,N,vd", [(4, 2, 24, 16), (3, 1, 5, 1), (2, 2, 64, 24), (6, 3, 128, 64), (1, 1, 200, 80), (5, 5, 16, 70), (2, 1, 33, 8), (2, 2, 400, 20),
                                          (1, 1, 512, 3)])
def test_state_space_scan_over_portions_and_reused_slots(lib, heads, G, N, vd):
    """two sequences of unequal length side by side, in portions of 1, 2, 9, ... tokens that continue from their slots; the slots
    hold stale values at the start (position 0 starts from zero); then a new sequence takes over a used slot"""
    _gpu()
    rng = np.random.default_rng(heads * 1000 + N)
    inner, C = heads * vd, heads * vd + 2 * G * N
    ld, ldd, stride, n_slots = C + 3, heads + 2, heads * N * vd + 11, 3
    a_log, dtb, skip = f32(rng.normal(-0.5, 0.7, heads)), f32(rng.normal(-1, 1, heads)), f32(rng.normal(1, 0.3, heads))
    state = dev(rng.standard_normal((n_slots, stride)))

    def make(T):
        xbc, dt = f32(rng.standard_normal((T, ld))), f32(rng.standard_normal((T, ldd)))
        y, Sf = S.state_space_scan(xbc[:, :inner].reshape(T, heads, vd), xbc[:, inner:inner + G * N].reshape(T, G, N),
                                   xbc[:, inner + G * N:C].reshape(T, G, N), dt[:, :heads], a_log, dtb, skip)
        return xbc, dt, y, Sf

    def run(seqs):
        """seqs: [(xbc rows, dt rows, slot, context length after the portion)]"""
        xs, ds = np.concatenate([s[0] for s in seqs]), np.concatenate([s[1] for s in seqs])
        cu = np.cumsum([0] + [len(s[0]) for s in seqs])
        T = int(cu[-1])
        y = torch.zeros((T, heads, vd), device="cuda")
        ok(lib.mi355_hyb_ssd_scan(y.data_ptr(), state.data_ptr(), stride, P(xs), ld, P(ds), ldd, P(a_log), P(dtb), P(skip),
                                  P([s[3] for s in seqs], np.int32), P(cu, np.int32), P([s[2] for s in seqs], np.int32), len(seqs), T, heads, G, N, vd, _st()))
        return y.cpu().numpy(), cu
    A, Bq = make(40), make(17)
    cutsA, cutsB = [1, 2, 9, 1, 27], [3, 1, 1, 12, 0]
    la = lb = 0
    gotA, gotB = [], []
    for ca, cb in zip(cutsA, cutsB):
        seqs = [(A[0][la:la + ca], A[1][la:la + ca], 2, la + ca)]
        if cb:
            seqs.append((Bq[0][lb:lb + cb], Bq[1][lb:lb + cb], 0, lb + cb))
        y, cu = run(seqs)
        gotA.append(y[:ca]); la += ca
        if cb:
            gotB.append(y[ca:]); lb += cb
    for got, ref in ((np.concatenate(gotA), A), (np.concatenate(gotB), Bq)):
        assert np.abs(got - ref[2]).max() < 3e-5 * max(1.0, np.abs(ref[2]).max())
    st = state.cpu().numpy()
    assert np.abs(st[2, :heads * N * vd].reshape(heads, N, vd) - A[3]).max() < 3e-5 * max(1.0, np.abs(A[3]).max())
    Cq = make(6)                                                          # a new sequence in A's slot: nothing of A is left
    y, _ = run([(Cq[0], Cq[1], 2, 6)])
    assert np.abs(y - Cq[2]).max() < 3e-5 * max(1.0, np.abs(Cq[2]).max())


@pytest.mark.parametrize("dtype", [F32, BF16])
@pytest.mark.parametrize("T,n,groups", [(4, 64, 2), (3, 30, 1), (2, 1200, 3), (5, 8, 8)])
def test_gate_in_front_of_the_group_norm(lib, dtype, T, n, groups):
    _gpu()
    rng = np.random.default_rng(n)
    y, z, w = f32(3 * rng.standard_normal((T, n))), f32(rng.standard_normal((T, n + 5))), f32(1 + 0.2 * rng.standard_normal(n))
    out = empty_dt((T, n), dtype)
    ok(lib.mi355_hyb_gate_group_norm(out.data_ptr(), dtype, P(y), P(z), n + 5, P(w), T, n, groups, 1e-5, _st()))
    want = S.gate_then_group_norm(y, z[:, :n], w, groups, 1e-5)
    assert np.abs(host_dt(out, dtype) - want).max() < tol(dtype) * max(1.0, np.abs(want).max())


@pytest.mark.parametrize("taps,C", [(1, 9), (3, 40), (4, 130)])
def test_convolution_with_bias_over_portions(lib, taps, C):
    _gpu()
    rng = np.random.default_rng(taps)
    T, off, ld = 21, 3, C + 7
    u, w, b = f32(rng.standard_normal((T, ld))), f32(rng.standard_normal((C, taps))), f32(rng.standard_normal(C))
    want = S.silu(S.causal_conv(u[:, off:off + C], w, b))
    stride = C * max(taps - 1, 1) + 3
    state = dev(rng.standard_normal((2, stride)))
    lo, got = 0, []
    for n in (1, 2, 1, 6, 11):
        out, seq = torch.zeros((n, C), device="cuda"), torch.zeros(n, dtype=torch.int32, device="cuda")

        def args():
            return P([lo + n], np.int32), P([0, n], np.int32), P([1], np.int32)
        ok(lib.mi355_hyb_conv_bias(out.data_ptr(), P(u[lo:lo + n]), ld, off, P(w), P(b), state.data_ptr(), stride, *args(), seq.data_ptr(), 1, n, C, taps,
                                   1, _st()))
        ok(lib.mi355_hyb_conv_state_update(state.data_ptr(), stride, P(u[lo:lo + n]), ld, off, *args(), 1, C, taps, _st()))
        got.append(out.cpu().numpy())
        lo += n
    assert np.abs(np.concatenate(got) - want).max() < 2e-5 * max(1.0, np.abs(want).max())


def _scatter(n_rows, bs, rng):
    """a block table that uses the pool's pages in a random order, and the slot of every token row"""
    nb = -(-n_rows // bs)
    table = rng.permutation(nb + 3)[:nb].astype(np.int32)
    slots = np.array([table[t // bs] * bs + t % bs for t in range(n_rows)], np.int64)
    return table, slots, nb + 3


@pytest.mark.parametrize("dtype", [F32, BF16])
@pytest.mark.parametrize("Hh,G,d,vd,bs,L,n_new", [(4, 2, 16, 8, 16, 300, 1), (4, 2, 16, 8, 16, 300, 7), (3, 3, 32, 32, 64, 330, 130), (8, 2, 64, 64, 32, 400, 96),
                                                  (6, 2, 32, 16, 16, 270, 80), (2, 1, 24, 40, 8, 140, 70), (4, 4, 128, 128, 64, 200, 1), (4, 1, 48, 48, 64, 520, 64)])
def test_attention_with_distance_bias_and_keys_that_stand_out(lib, dtype, Hh, G, d, vd, bs, L, n_new):
    """the last n_new tokens of a sequence of L against its scattered pages: single decoded tokens, short portions and prompt-sized
    portions (the matrix-core kernels, one wave per head and grouped heads).  Some queries get one key whose score stands out: hundreds
    back, on both sides of a page border, the first token, the token itself -- there the bias decides how much of its value arrives"""
    _gpu()
    rng = np.random.default_rng(Hh * 100 + d + n_new)
    q, k, v = rng.standard_normal((L, Hh, d)), rng.standard_normal((L, G, d)), rng.standard_normal((L, G, vd))
    r1, r2 = rng.uniform(0.2, 1.5, Hh), rng.uniform(0.05, 2.0, Hh)
    scale = 1.0 / math.sqrt(d)
    u = rng.standard_normal(d); u /= np.linalg.norm(u)
    first = L - n_new
    pairs = [(L - 1, max(0, L - 1 - 257)), (L - 1, 0), (L - 1, ((L - 1) // bs) * bs), (L - 1, ((L - 1) // bs) * bs - 1)]
    if n_new > 4:
        pairs += [(first + 1, (first // bs) * bs), (first + 2, max(0, (first // bs) * bs - 1)), (first + 3, first + 3), (first, max(0, first - 129))]
    for i, j in pairs:                                                    # score of (i, j) = 30 before the bias: far above the rest
        q[i, :, :] = math.sqrt(30.0 / scale) * u
        k[j, :, :] = math.sqrt(30.0 / scale) * u
    if dtype == BF16:
        q, k, v = S.bf16_round(q), S.bf16_round(k), S.bf16_round(v)
    else:
        q, k, v = f32(q), f32(k), f32(v)
    r1, r2 = f32(r1), f32(r2)
    want = S.distance_bias_attention(q, k, v, scale, r1, r2)[first:]
    table, slots, nblk = _scatter(L, bs, rng)
    nq, nk, nv = Hh * d, G * d, G * vd
    src = np.concatenate([q.reshape(L, nq), k.reshape(L, nk), v.reshape(L, nv)], axis=1)
    qo, kp, vp = empty_dt((L, nq), dtype), empty_dt((nblk * bs, nk), dtype), empty_dt((nblk * bs, nv), dtype)
    ok(lib.mi355_hyb_attn_prepare_whole(qo.data_ptr(), kp.data_ptr(), vp.data_ptr(), P(src), nq + nk + nv, 0, nq, nq + nk, None, None, P(slots, np.int64), L,
                                        Hh, G, d, vd, 0, 1e-5, dtype, _st()))
    tok_seq = torch.zeros(n_new, dtype=torch.int32, device="cuda")
    out = torch.zeros((n_new, Hh * vd), device="cuda")
    qn = qo[first:].contiguous()
    ok(lib.mi355_hyb_biased_attention(out.data_ptr(), F32, Hh * vd, 0, qn.data_ptr(), kp.data_ptr(), vp.data_ptr(), P(table, np.int32), P([L], np.int32),
                                      P([0, n_new], np.int32), tok_seq.data_ptr(), None, P(np.concatenate([r1, r2])), 1, n_new, Hh, G, d, vd, bs, len(table), 0, 0,
                                      scale, 1.0, 0, 0, 0.0, 0, dtype, _st()))
    got = out.cpu().numpy().reshape(n_new, Hh, vd)
    assert np.abs(got - want).max() < tol(dtype, 3e-5, 2e-2) * max(1.0, np.abs(want).max())
    # without the bias the same launch gives the plain softmax
    ok(lib.mi355_hyb_biased_attention(out.data_ptr(), F32, Hh * vd, 0, qn.data_ptr(), kp.data_ptr(), vp.data_ptr(), P(table, np.int32), P([L], np.int32),
                                      P([0, n_new], np.int32), tok_seq.data_ptr(), None, None, 1, n_new, Hh, G, d, vd, bs, len(table), 0, 0,
                                      scale, 1.0, 0, 0, 0.0, 0, dtype, _st()))
    plain = S.distance_bias_attention(q, k, v, scale)[first:]
    assert np.abs(out.cpu().numpy().reshape(n_new, Hh, vd) - plain).max() < tol(dtype, 3e-5, 2e-2) * max(1.0, np.abs(plain).max())


@pytest.mark.parametrize("T,W,E,top,groups", [(9, 64, 16, 2, (2, 1)), (5, 50, 12, 3, (4, 2)), (7, 33, 70, 6, None), (3, 128, 8, 8, (8, 8)), (6, 40, 6, 1, (6, 2)),
                                              (4, 64, 130, 5, (10, 3)), (300, 32, 9, 2, (3, 2))])
def test_router_sigmoid_scores_best_groups_and_normalised_weights(lib, T, W, E, top, groups):
    """f32 logits, sigmoid scores, the correction (also negative) in the choice only, groups by the sum of their two best, weights
    divided by their sum; tokens whose choice is a close call are left out"""
    _gpu()
    rng = np.random.default_rng(E * 10 + top)
    h, R, corr = f32(rng.standard_normal((T, W))), f32(rng.standard_normal((E, W)) * 2 / math.sqrt(W)), f32(rng.uniform(-1.5, 0.3, E))
    margins = []
    ids_w, w_w = S.route(h @ R.T, corr, top, groups, margins)
    ids = torch.zeros((T, top), dtype=torch.int32, device="cuda")
    wts = torch.zeros((T, top), device="cuda")
    ok(lib.mi355_hyb_moe_route_ex(ids.data_ptr(), wts.data_ptr(), None, None, F32, P(h), None, P(R), P(corr), None, T, W, E, top, 1.0, 1e-5, 0, 1,
                                  groups[0] if groups else 0, groups[1] if groups else 0, 1, _st()))
    per_tok = np.full(T, np.inf)
    for n in range(len(margins) // T):
        per_tok = np.minimum(per_tok, np.abs(margins[n * T:(n + 1) * T]))
    sure = per_tok > 1e-5
    assert sure.sum() >= T // 2
    assert np.array_equal(ids.cpu().numpy()[sure], ids_w[sure])
    assert np.abs(wts.cpu().numpy()[sure] - w_w[sure]).max() < 1e-5
    assert np.abs(wts.cpu().numpy().sum(-1) - 1).max() < 1e-5


@pytest.mark.parametrize("dtype", [F32, BF16])
def test_small_glue(lib, dtype):
    """relu squared, the tanh cap, the elementwise gate, the token's side input behind its gelu gate, the average over the depth, the
    experts' sum without a norm, the scaled embedding, the sum of two sublayers"""
    _gpu()
    rng = np.random.default_rng(3)
    T, n = 7, 45
    a, b, c = f32(2 * rng.standard_normal((T, n))), f32(rng.standard_normal((T, n + 2))), f32(rng.standard_normal((T, n)))
    out = empty_dt((T, n), dtype)
    ok(lib.mi355_hyb_relu2(out.data_ptr(), dtype, P(a), T * n, _st()))
    assert np.abs(host_dt(out, dtype) - np.maximum(a, 0) ** 2).max() < tol(dtype) * 20
    ok(lib.mi355_hyb_elem_gate(out.data_ptr(), dtype, P(a), P(b), n + 2, T, n, _st()))
    assert np.abs(host_dt(out, dtype) - a * S.sigmoid(b[:, :n])).max() < tol(dtype) * 8
    x = dev(10 * a)
    ok(lib.mi355_hyb_tanh_cap(x.data_ptr(), 7.5, T * n, _st()))
    assert np.abs(x.cpu().numpy() - 7.5 * np.tanh(10 * a / 7.5)).max() < 1e-5
    x = dev(a)
    ok(lib.mi355_hyb_add2(x.data_ptr(), P(c), P(a), T * n, _st()))
    assert np.abs(x.cpu().numpy() - (2 * a + c)).max() < 1e-5
    ok(lib.mi355_hyb_add2(x.data_ptr(), P(c), None, T * n, _st()))
    assert np.abs(x.cpu().numpy() - (2 * a + 2 * c)).max() < 1e-5
    # side input: columns [col, col + dim) of the token's row, times gelu of the gate
    V_, cols, col, dim = 19, 30, 12, 9
    table, g, tok = S.bf16_round(rng.standard_normal((V_, cols))), f32(2 * rng.standard_normal((T, dim))), rng.integers(0, V_, T)
    out = empty_dt((T, dim), dtype)
    ok(lib.mi355_hyb_side_act(out.data_ptr(), dtype, P(g), dev_dt(table, dtype).data_ptr(), cols, col, P(tok, np.int32), T, dim, V_, dtype, _st()))
    assert np.abs(host_dt(out, dtype) - S.gelu_tanh(g) * table[tok][:, col:col + dim]).max() < tol(dtype) * 5
    # depth average: the newest result takes the last place, then the weighted sum
    terms = 4
    xs, w = f32(rng.standard_normal((terms, T * n))), f32(rng.uniform(0.1, 1, terms))
    xd, cur = dev(xs), dev(a)
    ok(lib.mi355_hyb_depth_average(cur.data_ptr(), xd.data_ptr(), P(w), terms, T * n, _st()))
    ref = np.concatenate([xs[:3], a.reshape(1, -1)])
    assert np.abs(xd.cpu().numpy() - ref).max() == 0 and np.abs(cur.cpu().numpy().reshape(-1) - (w[:, None] * ref).sum(0)).max() < 1e-5
    # experts' sum: x += y + sum_j w_j rows[pos]
    top, rows_n = 3, 40
    rows, pos, wt = f32(rng.standard_normal((rows_n, n))), rng.integers(0, rows_n, (T, top)), f32(rng.uniform(0, 1, (T, top)))
    x = dev(a)
    ok(lib.mi355_hyb_moe_combine_add(x.data_ptr(), P(c), P(rows), P(pos, np.int32), P(wt), T, n, top, _st()))
    assert np.abs(x.cpu().numpy() - (a + c + (wt[:, :, None] * rows[pos]).sum(1))).max() < 1e-5
    emb = S.bf16_round(rng.standard_normal((V_, n)))
    x = torch.zeros((T, n), device="cuda")
    ok(lib.mi355_hyb_embed_scaled(x.data_ptr(), dev_dt(emb, dtype).data_ptr(), P(tok, np.int32), T, n, V_, 0.375, dtype, _st()))
    assert np.abs(x.cpu().numpy() - emb[tok] * 0.375).max() < 1e-6


@pytest.mark.parametrize("dtype", [F32, BF16])
@pytest.mark.parametrize("T,W,terms,side,norm", [(5, 64, 3, True, True), (3, 50, 1, False, True), (2, 1100, 4, True, False), (4, 32, 0, True, True),
                                                 (1, 8, 0, False, True)])
def test_layer_tail_in_one_launch(lib, dtype, T, W, terms, side, norm):
    """the side input's norm and sum, the average over the depth and the next layer's norm in one launch equal the three steps alone,
    with any of them absent"""
    _gpu()
    rng = np.random.default_rng(T * W + terms)
    x, y, sw, nw = f32(5 + rng.standard_normal((T, W))), f32(3 * rng.standard_normal((T, W))), f32(rng.standard_normal(W)), f32(1 + 0.2 * rng.standard_normal(W))
    xs, dw = f32(rng.standard_normal((max(terms, 1), T * W))), f32(rng.uniform(0.1, 1, max(terms, 1)))
    want_x = x + S.rms_unit(y, 1e-5) * sw if side else x.copy()
    want_xs = xs.copy()
    if terms:
        want_xs[terms - 1] = want_x.reshape(-1)
        want_x = (dw[:, None] * want_xs[:terms]).sum(0).reshape(T, W)
    xd, xsd = dev(x), dev(xs)
    out, out2 = empty_dt((T, W), dtype), torch.zeros((T, W), device="cuda")
    ok(lib.mi355_hyb_layer_tail(xd.data_ptr(), P(y) if side else None, P(sw) if side else None, xsd.data_ptr(), P(dw) if terms else None, terms,
                                out.data_ptr(), dtype, out2.data_ptr(), P(nw) if norm else None, T, W, 1, 1e-5, _st()))
    assert np.abs(xd.cpu().numpy() - want_x).max() < 1e-5 * np.abs(want_x).max()
    assert np.abs(xsd.cpu().numpy() - want_xs).max() < 1e-5 * max(1.0, np.abs(want_xs).max())
    if norm:
        h = S.layer_norm(want_x, nw, 1e-5)
        assert np.abs(out2.cpu().numpy() - h).max() < 1e-4 * max(1.0, np.abs(h).max())
        assert np.abs(host_dt(out, dtype) - h).max() < tol(dtype, 1e-4) * max(1.0, np.abs(h).max())


# ------------------------------------------------------------------------------------------------------------ whole models
def _moe(E, top, ff, groups=None):
    r = {"experts": E, "top": top}
    if groups:
        r["groups"] = {"count": groups[0], "keep": groups[1]}
    return {"expert": {"ff": ff}, "kind": "moe", "router": r}


def _rot(dims, scaling=True):
    r = {"base": 3000.0, "dims": dims}
    if scaling:
        r["scaling"] = {"factor": 6.0, "fast": 16.0, "original": 64, "slow": 1.5}
    return r


def small_config(variant):
    if variant == 0:        # every mixer and both feed-forwards, sizes that are not each other's equals, borrowed pages two layers on
        lat = {"dim": 16, "heads": 2, "kv_rank": 32, "q_rank": 24, "rot": _rot(8), "rot_dim": 8, "scale": 0.21, "vdim": 24}
        layers = [{"type": "attention", "mixer": {"conv": 3, "dim": 16, "heads": 4, "kv_heads": 2, "scale": 0.27, "vdim": 8}, "mlp": _moe(8, 2, 24, (4, 2))},
                  {"type": "mamba2", "mixer": {"conv": 4, "groups": 2, "heads": 4, "norm_groups": 2, "state": 24, "vdim": 16}, "mlp": {"ff": 96, "kind": "dense"}},
                  {"type": "latent_attention", "mixer": lat, "mlp": _moe(6, 3, 20)},
                  {"type": "mamba2", "mixer": {"conv": 2, "groups": 1, "heads": 2, "norm_groups": 1, "state": 64, "vdim": 8}, "mlp": None},
                  {"type": "latent_attention", "mixer": dict(lat, kv_from=2), "mlp": _moe(5, 1, 16, (5, 2))}]
        return {"architecture": "Sabolorn", "embedding": {"scale": 0.5}, "layers": layers, "logit_softcap": 12.0, "norm": {"eps": 1e-5},
                "token_side": {"dim": 8}, "vocab": 131, "width": 64}
    if variant == 1:        # the latent layers first, head sizes of the matrix-core attention kernels, no token side input, no softcap
        lat = {"dim": 32, "heads": 3, "kv_rank": 48, "q_rank": 16, "rot": _rot(16, False), "rot_dim": 16, "scale": 0.15, "vdim": 32}
        layers = [{"type": "latent_attention", "mixer": lat, "mlp": {"ff": 64, "kind": "dense"}},
                  {"type": "latent_attention", "mixer": dict(lat, kv_from=0), "mlp": _moe(4, 2, 32)},
                  {"type": "attention", "mixer": {"conv": 1, "dim": 32, "heads": 3, "kv_heads": 3, "scale": 0.18, "vdim": 32}, "mlp": _moe(12, 4, 16, (3, 2))},
                  {"type": "mamba2", "mixer": {"conv": 3, "groups": 1, "heads": 3, "norm_groups": 3, "state": 128, "vdim": 32}, "mlp": {"ff": 40, "kind": "dense"}}]
        return {"architecture": "Sabolorn", "embedding": {"scale": 1.0}, "layers": layers, "norm": {"eps": 1e-6}, "vocab": 90, "width": 96}
    # grouped heads on one key/value head pair, long prompts
    layers = [{"type": "attention", "mixer": {"conv": 4, "dim": 64, "heads": 8, "kv_heads": 2, "scale": 0.125, "vdim": 64}, "mlp": {"ff": 128, "kind": "dense"}},
              {"type": "mamba2", "mixer": {"conv": 4, "groups": 4, "heads": 8, "norm_groups": 4, "state": 16, "vdim": 16}, "mlp": _moe(16, 2, 32, (2, 1))},
              {"type": "attention", "mixer": {"conv": 2, "dim": 32, "heads": 6, "kv_heads": 2, "scale": 0.2, "vdim": 16}, "mlp": None}]
    return {"architecture": "Sabolorn", "embedding": {"scale": 0.7}, "layers": layers, "logit_softcap": 30.0, "norm": {"eps": 1e-5},
            "token_side": {"dim": 16}, "vocab": 257, "width": 128}


def settle_router(W, rng):
    """routing for runs in 16 bits: rounding noise flips a choice between two experts whose scores are close, and the oracle cannot
    follow such a flip.  Corrections further apart than two sigmoid values can be settle which experts and groups a layer uses (a
    random order of 1.5 times the powers of two: no two pairs of them have the same sum, so groups cannot tie either); the weights
    still come from the router.  The choice by token is what the f32 runs cover."""
    for k in list(W):
        if k.endswith("mlp.correction"):
            W[k] = S.bf16_round(1.5 * 2.0 ** rng.permutation(W[k].shape[0]))


def build(cfg, dtype, seed=0, block_size=16, state_slots=4, drop=()):
    from candle_vllm_amd.hybrid_model import HybridModel, SabolornSpec
    rng = np.random.default_rng(seed)
    W = S.random_sabolorn(rng, cfg)
    for name in drop:
        del W[name]
    if dtype == "bfloat16":
        settle_router(W, rng)
    m = HybridModel(SabolornSpec(cfg, {k: v.shape for k, v in W.items()}), dtype=dtype, block_size=block_size, state_slots=state_slots)
    m.load_state_dict_f32(W)
    return m, W


def row_err(a, b):
    d = a - b
    d = d - d.mean(-1, keepdims=True)
    return np.sqrt((d * d).mean(-1)).max() / max(1e-9, np.sqrt((b * b).mean()))


TOL = {"float32": 3e-5, "bfloat16": 4e-2}
CLOSE_CALL = 1e-5           # a choice between two experts (or groups) whose scores lie closer than this may fall either way in f32


def oracle_logits(cfg, W, toks, rng=None):
    """the oracle's logits (and trace); no routing decision of the run may be a close call -- with `rng`, tokens are drawn again"""
    for _ in range(30):
        margins = []
        out, tr = S.forward(cfg, W, toks, margins)
        if not margins or min(margins) > CLOSE_CALL:
            return out, tr, toks
        assert rng is not None, "a routing decision of this test is a close call: take other tokens"
        toks = rng.integers(0, cfg["vocab"], len(toks)).tolist()
    raise AssertionError("no token sequence without a close call")


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("variant", [0, 1, 2])
def test_model_whole_portions_decode_against_oracle(lib, dtype, variant):
    """one request whole, with the residual stream behind every layer; then the same tokens in portions of 2, 1, 17, ... tokens and
    token by token: every way must give the oracle's logits at every position (convolution tails, recurrent state and borrowed pages
    cross every cut; pages of 16 tokens)"""
    _gpu()
    from candle_vllm_amd.step_engine import StepEngine
    cfg = small_config(variant)
    m, W = build(cfg, dtype, seed=variant, drop=("l1.dwa",) if variant == 1 else ())
    rng = np.random.default_rng(11)
    n = 330 if variant == 2 else 75
    toks = rng.integers(0, cfg["vocab"], n).tolist()
    want, want_trace, toks = oracle_logits(cfg, W, toks, rng)
    eng = StepEngine(m, 3 * 336)
    eng.feed("a", toks)
    got, tr = eng.step(["a"], [list(range(n))], trace=True)
    eng.finish("a")
    if dtype == "float32":
        assert np.abs(tr.cpu().numpy() - want_trace).max() < 1e-4 * np.abs(want_trace).max()
    assert row_err(got.cpu().numpy(), want) < TOL[dtype]
    for cuts in ([2, 1, 17, 1, 1, 2, 30, 3, 18], [40] + [1] * 35, [1] * 20 + [55]):
        cuts = cuts + ([n - 75] if n > 75 else [])
        assert sum(cuts) == n
        lo, rows = 0, []
        for c in cuts:
            eng.feed("b", toks[lo:lo + c])
            rows.append(eng.step(["b"], [list(range(c))]).cpu().numpy())
            lo += c
        eng.finish("b")
        assert row_err(np.concatenate(rows), want) < TOL[dtype], cuts
        assert eng.free_pages() == eng.num_blocks and eng.be.state_free_slots() == 4


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_unequal_batches_pages_and_slots_reused(lib, dtype):
    """five requests of unequal length through four slots and a pool that only fits them because pages come back: portions of some
    beside single tokens of others, a request that sits steps out, a late one that takes over a freed slot and freed pages --
    every logit must equal the request run alone in the oracle"""
    _gpu()
    from candle_vllm_amd.step_engine import StepEngine
    cfg = small_config(0)
    m, W = build(cfg, dtype, seed=3)
    rng = np.random.default_rng(21)
    lens = {"a": 70, "b": 33, "c": 5, "d": 48, "e": 41}
    toks = {r: oracle_logits(cfg, W, rng.integers(0, cfg["vocab"], n).tolist(), rng)[2] for r, n in lens.items()}
    want = {r: S.forward(cfg, W, toks[r])[0] for r in toks}
    eng = StepEngine(m, 80 + 48 + 16 + 48 + 0)                            # "e" (48 rounded) only fits after "b" and "c" have gone
    sched = [[("a", 2), ("b", 30)], [("a", 16), ("b", 1), ("c", 3)], [("a", 1), ("b", 1), ("c", 1), ("d", 47)], [("a", 30), ("c", 1), ("b", 1)],
             [("a", 1), ("d", 1), ("e", 2)], [("e", 38), ("a", 1)], [("a", 19), ("e", 1)]]
    at, got = {r: 0 for r in toks}, {r: [] for r in toks}
    for step in sched:
        ids, w = [], []
        for r, n in step:
            eng.feed(r, toks[r][at[r]:at[r] + n])
            at[r] += n
            ids.append(r); w.append(list(range(n)))
        out = eng.step(ids, w).cpu().numpy()
        lo = 0
        for r, n in step:
            got[r].append(out[lo:lo + n]); lo += n
        for r, _ in step:
            if at[r] == lens[r]:
                eng.finish(r)
    assert at == lens
    for r in toks:
        assert row_err(np.concatenate(got[r]), want[r]) < TOL[dtype], r
    assert eng.free_pages() == eng.num_blocks and eng.be.state_free_slots() == 4


def test_long_decoding_first_tokens_and_graph_replays(lib):
    """a prompt of one token, then 150 tokens one by one (decoding batches replay a captured hipGraph): the first tokens and every
    later one equal the oracle; the eager steps give the same logits bit for bit"""
    _gpu()
    from candle_vllm_amd.step_engine import StepEngine
    cfg = small_config(0)
    m, W = build(cfg, "float32", seed=8)
    rng = np.random.default_rng(9)
    want, _, toks = oracle_logits(cfg, W, rng.integers(0, cfg["vocab"], 151).tolist(), rng)
    outs = {}
    for use_graph in (True, False):
        eng = StepEngine(m, 160)
        eng.use_graph = use_graph
        rows = []
        for t in toks:
            eng.feed("a", [t])
            rows.append(eng.step(["a"]).cpu().numpy())
        eng.finish("a")
        outs[use_graph] = np.concatenate(rows)
    assert row_err(outs[True][:4], want[:4]) < TOL["float32"]
    assert row_err(outs[True], want) < TOL["float32"]
    assert np.array_equal(outs[True], outs[False])
    cap, rep = m.graph_stats()
    assert cap >= 1 and rep >= 100


def test_sizes_that_are_one(lib):
    """one head, one group, one expert of which one is used, one tap, one norm part, a state of one, a side input of one column"""
    _gpu()
    from candle_vllm_amd.step_engine import StepEngine
    lat = {"dim": 8, "heads": 1, "kv_rank": 8, "q_rank": 1, "rot": _rot(2), "rot_dim": 2, "scale": 0.3, "vdim": 8}
    layers = [{"type": "mamba2", "mixer": {"conv": 1, "groups": 1, "heads": 1, "norm_groups": 1, "state": 1, "vdim": 1}, "mlp": _moe(1, 1, 8)},
              {"type": "attention", "mixer": {"conv": 1, "dim": 1, "heads": 1, "kv_heads": 1, "scale": 1.0, "vdim": 1}, "mlp": {"ff": 1, "kind": "dense"}},
              {"type": "latent_attention", "mixer": lat, "mlp": _moe(3, 3, 4, (3, 3))}]
    cfg = {"architecture": "Sabolorn", "embedding": {"scale": 2.0}, "layers": layers, "logit_softcap": 5.0, "norm": {"eps": 1e-5}, "token_side": {"dim": 1},
           "vocab": 17, "width": 32}
    m, W = build(cfg, "float32", seed=5)
    rng = np.random.default_rng(5)
    want, _, toks = oracle_logits(cfg, W, rng.integers(0, 17, 40).tolist(), rng)
    eng = StepEngine(m, 64)
    lo, rows = 0, []
    for c in [1, 2, 20, 1, 1, 15]:
        eng.feed("a", toks[lo:lo + c])
        rows.append(eng.step(["a"], [list(range(c))]).cpu().numpy())
        lo += c
    assert row_err(np.concatenate(rows), want) < TOL["float32"]


@pytest.mark.parametrize("chunk", [0, 7])
def test_greedy_generation_through_scheduler(lib, chunk):
    """run_engine + the C++ scheduler (continuous batching, staggered arrivals, chunked prefill): every request generates exactly the
    tokens the oracle generates for it alone"""
    _gpu()
    from candle_vllm_amd import block_engine as be
    from candle_vllm_amd.engine import Request, run_engine
    cfg = small_config(0)
    m, W = build(cfg, "float32", seed=6)
    rng = np.random.default_rng(6)
    prompts = [rng.integers(0, cfg["vocab"], n).tolist() for n in (19, 3, 40, 11, 26)]
    n_new = 10
    want = []
    for p in prompts:
        seq, out = list(p), []
        for _ in range(n_new):
            lg = S.forward(cfg, W, seq)[0][-1]
            top2 = np.sort(lg)[-2:]
            assert top2[1] - top2[0] > 1e-4, "a greedy choice of this test is a close call: take another seed"
            out.append(int(lg.argmax()))
            seq.append(out[-1])
        want.append(out)
    nblk = 24
    sched = be.Scheduler(16, nblk, 0, 4, 64, prefill_chunk_size=chunk)
    sched.block_engine.state_init(4)
    m.alloc_cache(nblk)
    reqs = [Request(i, p, n_new, arrival_step=2 * i) for i, p in enumerate(prompts)]
    stats = run_engine(m, sched, reqs, chunk=chunk)
    assert stats["finished"] == len(prompts)
    for r, w in zip(reqs, want):
        assert r.tokens == w, (r.id, r.tokens, w)
    assert sched.block_engine.state_free_slots() == 4


def _write_model(folder, cfg, W):
    """config.json + model.safetensors (bf16; 8-byte header length, JSON header, data) of a configuration"""
    head, blobs, at = {}, [], 0
    for name, a in W.items():
        raw = bits(a).tobytes()
        head[name] = {"dtype": "BF16", "shape": list(np.shape(a)), "data_offsets": [at, at + len(raw)]}
        blobs.append(raw)
        at += len(raw)
    hb = json.dumps(head).encode()
    (folder / "model.safetensors").write_bytes(struct.pack("<Q", len(hb)) + hb + b"".join(blobs))
    (folder / "config.json").write_text(json.dumps(cfg))


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_trace_runner_replays_a_mixed_schedule_from_a_checkpoint_folder(lib, tmp_path, dtype):
    """bin/trace_run as a user starts it: a folder with config.json and model.safetensors, steps on standard input -- six requests over
    time, at most four alive, portions beside single tokens, a pool that only fits because ended requests give their pages and slots
    back -- and the logits it writes equal the oracle's for every request alone"""
    _gpu()
    cfg = small_config(1)
    rng = np.random.default_rng(17)
    W = S.random_sabolorn(rng, cfg)
    if dtype == "bfloat16":
        settle_router(W, rng)
    _write_model(tmp_path, cfg, W)
    lens = {"a": 150, "b": 40, "c": 3, "d": 90, "e": 61, "f": 130}
    toks = {r: oracle_logits(cfg, W, rng.integers(0, cfg["vocab"], n).tolist(), rng)[2] for r, n in lens.items()}
    want = {r: S.forward(cfg, W, toks[r])[0] for r in toks}
    sched = [[("a", 70), ("b", 2)], [("a", 1), ("b", 30), ("c", 3)], [("a", 64), ("b", 1), ("d", 65)], [("a", 1), ("b", 7), ("d", 1), ("e", 17)],
             [("a", 14), ("d", 24), ("e", 1), ("f", 2)], [("e", 43), ("f", 100)], [("f", 1)], [("f", 27)]]
    at, steps, rows = {r: 0 for r in toks}, [], []
    for n, step in enumerate(sched):
        entries, end, got = [], [], []
        for r, c in step:
            w = sorted(set([0, c - 1] + rng.integers(0, c, 3).tolist()))
            entries.append({"id": r, "tokens": toks[r][at[r]:at[r] + c], "want": w})
            got += [(r, at[r] + k) for k in w]
            at[r] += c
            if at[r] == lens[r]:
                end.append(r)
        steps.append(json.dumps({"step": n, "entries": entries, "end": end}))
        rows.append(got)
    assert at == lens
    out = tmp_path / "out"
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    r = subprocess.run([sys.executable, os.path.join(root, "bin", "trace_run"), "--model", str(tmp_path), "--dtype", dtype, "--out", str(out),
                        "--max-tokens", "448"], input="\n".join(steps) + "\n", capture_output=True, text=True, timeout=170)
    assert r.returncode == 0, r.stderr[-2000:]
    assert [l for l in r.stdout.splitlines() if l.startswith("done ")] == ["done %d" % n for n in range(len(sched))]
    for n, got in enumerate(rows):
        a = np.fromfile(out / ("%d.f32" % n), "<f4").reshape(len(got), cfg["vocab"])
        ref = np.stack([want[r_][p_] for r_, p_ in got])
        assert row_err(a, ref) < TOL[dtype], (n, dtype)


def random_config(rng):
    """sizes, head counts, depth, order, taps, expert counts and constants drawn at random (sizes that are not all multiples of 16 or
    32; layers without a feed-forward, routers without groups, latent layers on an earlier layer's pages)"""
    width = int(rng.choice([64, 100, 128, 160, 256]))
    side = int(rng.choice([0, 4, 24, 32]))

    def mlp():
        u = rng.random()
        if u < 0.15:
            return None
        if u < 0.45:
            return {"ff": int(rng.choice([24, 100, 256])), "kind": "dense"}
        cnt = int(rng.choice([1, 2, 4]))
        per = int(rng.choice([2, 3, 8]))
        keep = int(rng.integers(1, cnt + 1))
        return _moe(cnt * per, int(rng.integers(1, min(keep * per, 6) + 1)), int(rng.choice([16, 40, 64])), (cnt, keep) if rng.random() < 0.8 else None)
    layers, lenders = [], []
    for i in range(int(rng.integers(3, 7))):
        kind = str(rng.choice(["mamba2", "attention", "latent_attention"]))
        if kind == "mamba2":
            G = int(rng.choice([1, 2, 4]))
            heads, vd = G * int(rng.choice([1, 2, 3])), int(rng.choice([8, 16, 20, 64]))
            ng = int(rng.choice([g for g in (1, 2, 4, heads) if (heads * vd) % g == 0]))
            c = {"conv": int(rng.integers(1, 6)), "groups": G, "heads": heads, "norm_groups": ng, "state": int(rng.choice([8, 16, 48, 64, 100, 128])), "vdim": vd}
        elif kind == "attention":
            G, d = int(rng.choice([1, 2, 3])), int(rng.choice([16, 20, 32, 48, 64, 128]))
            c = {"conv": int(rng.integers(1, 6)), "dim": d, "heads": G * int(rng.choice([1, 2, 3, 4])), "kv_heads": G,
                 "scale": float(d ** -0.5 * rng.uniform(0.7, 1.5)), "vdim": int(rng.choice([8, 16, 24, 48, 64, 128]))}
        else:
            if lenders and rng.random() < 0.5:
                j = int(rng.choice(lenders))
                c = dict(layers[j]["mixer"], kv_from=j, heads=int(rng.choice([1, 2, 4])), vdim=int(rng.choice([16, 32, 40])))
            else:
                rd = int(rng.choice([2, 8, 16, 32, 64]))
                c = {"dim": int(rng.choice([16, 32, 64])), "heads": int(rng.choice([1, 2, 4, 6])), "kv_rank": int(rng.choice([32, 64, 96, 128])),
                     "q_rank": int(rng.choice([8, 48, 80])), "rot": {"base": float(rng.choice([1e3, 1e4, 5e5])), "dims": rd}, "rot_dim": rd,
                     "scale": float(rng.uniform(0.08, 0.2)), "vdim": int(rng.choice([16, 32, 64]))}
                if rng.random() < 0.8:
                    c["rot"]["scaling"] = {"factor": float(rng.choice([2.0, 8.0, 40.0])), "fast": float(rng.choice([8.0, 32.0])),
                                           "original": int(rng.choice([64, 1024, 4096])), "slow": float(rng.choice([0.5, 1.0, 2.0]))}
                lenders.append(i)
        layers.append({"type": kind, "mixer": c, "mlp": mlp()})
    cfg = {"architecture": "Sabolorn", "embedding": {"scale": float(rng.choice([1.0, 0.5, 3.0]))}, "layers": layers,
           "logit_softcap": float(rng.choice([8.0, 15.0, 50.0])), "norm": {"eps": float(rng.choice([1e-5, 1e-6]))}, "vocab": int(rng.integers(50, 600)),
           "width": width}
    if side:
        cfg["token_side"] = {"dim": side}
    return cfg


@pytest.mark.parametrize("seed", [2, 11, 21, 33, 47, 58])
def test_random_configurations_whole_and_mixed_schedules(lib, seed):
    """three unequal requests of a random configuration: each alone in one step, then together in a random schedule of portions (2, 3,
    17, 64, 65, 100 tokens; a request may sit a step out) that ends token by token -- on 64-token pages, in f32 and bf16"""
    _gpu()
    from candle_vllm_amd.step_engine import StepEngine
    from candle_vllm_amd.hybrid_model import HybridModel, SabolornSpec
    rng = np.random.default_rng(seed)
    cfg = random_config(rng)
    W = S.random_sabolorn(rng, cfg)
    lens = [int(rng.integers(150, 300)), int(rng.integers(1, 40)), int(rng.integers(60, 130))]
    toks = [oracle_logits(cfg, W, rng.integers(0, cfg["vocab"], n).tolist(), rng)[2] for n in lens]
    want = [S.forward(cfg, W, t)[0] for t in toks]
    for dtype in ("float32", "bfloat16"):
        if dtype == "bfloat16":
            settle_router(W, rng)
            want = [S.forward(cfg, W, t)[0] for t in toks]
        m = HybridModel(SabolornSpec(cfg, {k: v.shape for k, v in W.items()}), dtype=dtype, block_size=64, state_slots=4)
        m.load_state_dict_f32(W)
        eng = StepEngine(m, 64 * 10)
        for i, t in enumerate(toks):
            eng.feed("w", t)
            got = eng.step(["w"], [list(range(len(t)))]).cpu().numpy()
            eng.finish("w")
            assert row_err(got, want[i]) < TOL[dtype], (seed, dtype, "whole", i, cfg)
        at, got = [0, 0, 0], [[], [], []]
        srng = np.random.default_rng(seed + 1)
        while any(a < n for a, n in zip(at, lens)):
            ids, w, step = [], [], []
            for i in range(3):
                left = lens[i] - at[i]
                if left == 0 or srng.random() < 0.2:
                    continue
                c = 1 if left <= 8 else min(left - 8, int(srng.choice([2, 3, 17, 64, 65, 100])))
                eng.feed(str(i), toks[i][at[i]:at[i] + c])
                ids.append(str(i)); w.append(list(range(c))); step.append((i, c))
                at[i] += c
            if not ids:
                continue
            out = eng.step(ids, w).cpu().numpy()
            lo = 0
            for i, c in step:
                got[i].append(out[lo:lo + c]); lo += c
        for i in range(3):
            eng.finish(str(i))
            assert row_err(np.concatenate(got[i]), want[i]) < TOL[dtype], (seed, dtype, "mixed", i, cfg)
