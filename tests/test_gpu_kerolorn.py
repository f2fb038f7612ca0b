"""The Kerolorn mechanisms of the layer-list host layer (include/mi355_hybrid.h) against the float64 oracle of oracle/kerolorn.py:
every new mechanism alone through its C entry point (the norm in front of a sublayer, the convolution added to its input, interleaved
rotation with the norm behind it and a temperature per head, a window that keeps the first tokens, the router with its selection-only
correction, the grouping of (token, expert) pairs into blocks, grouped products, the weighted sum with the shared expert and the output
norm), then whole models through the step engine -- whole prompts against token-by-token decoding, portions down to two tokens,
unequal batches against each request alone, pages and slots that are freed and used again, dominant keys just inside / outside the
window and the kept first tokens and hundreds of tokens back, the first tokens, long decoding, sizes that are 1 or equal -- and
greedy generation through run_engine and the scheduler.  Configurations and weights are made here."""
import ctypes
import math

import numpy as np
import pytest

torch = pytest.importorskip("torch")

from oracle import hybrid as H                          # noqa: E402
from oracle import vivazen as V                         # noqa: E402
from oracle import kerolorn as K                        # noqa: E402

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


# ------------------------------------------------------------------------------------------------------------ mechanisms alone
@pytest.mark.parametrize("dtype", [F32, BF16])
@pytest.mark.parametrize("taps,C", [(1, 20), (2, 7), (4, 64), (5, 130)])
def test_pre_norm_and_input_convolution_over_portions(lib, dtype, taps, C):
    """h = norm(x) w, then h + conv(h) in portions of 1, 2, ... tokens continuing from the slot's tail; a sequence that starts at 0
    ignores whatever its slot held"""
    _gpu()
    rng = np.random.default_rng(taps * 100 + C)
    T, n_slots = 23, 3
    x, nw, w = f32(3 * rng.standard_normal((T, C))), f32(1 + 0.2 * rng.standard_normal(C)), f32(rng.standard_normal((C, taps)))
    h = H.rms_norm(x, nw, 1e-5)
    want, _ = K.conv_residual(h, w)
    stride = C * max(taps - 1, 1) + 5
    state = dev(rng.standard_normal((n_slots, stride)))                    # stale values everywhere
    lo, got = 0, []
    for n in (1, 2, 1, 7, 12):
        seq = torch.zeros(n, dtype=torch.int32, device="cuda")
        hn = torch.zeros((n, C), device="cuda")
        out = empty_dt((n, C), dtype)

        def args():
            return P([lo + n], np.int32), P([0, n], np.int32), P([2], np.int32)
        ok(lib.mi355_hyb_pre_norm(hn.data_ptr(), F32, P(x[lo:lo + n]), P(nw), n, C, 1e-5, _st()))
        assert np.abs(hn.cpu().numpy() - h[lo:lo + n]).max() < 1e-5
        ok(lib.mi355_hyb_conv_residual(out.data_ptr(), dtype, hn.data_ptr(), C, 0, P(w), state.data_ptr(), stride, *args(), seq.data_ptr(), 1, n, C,
                                       taps, _st()))
        ok(lib.mi355_hyb_conv_state_update(state.data_ptr(), stride, hn.data_ptr(), C, 0, *args(), 1, C, taps, _st()))
        got.append(host_dt(out, dtype))
        lo += n
    assert np.abs(np.concatenate(got) - want).max() < (2e-5 if dtype == F32 else 2e-2) * max(1.0, np.abs(want).max())
    # norm, convolution and (for single tokens) the move of the state in ONE launch: the same result, the same state
    state2 = dev(rng.standard_normal((n_slots, stride)))
    lo, got2 = 0, []
    for n in (1, 2, 1, 7, 1, 11):
        seq = torch.zeros(n, dtype=torch.int32, device="cuda")
        hn = torch.zeros((n, C), device="cuda")
        out = empty_dt((n, C), dtype)

        def args():
            return P([lo + n], np.int32), P([0, n], np.int32), P([2], np.int32)
        own = int(n == 1)
        ok(lib.mi355_hyb_norm_conv(out.data_ptr(), dtype, None if own else hn.data_ptr(), P(x[lo:lo + n]), P(nw), P(w), state2.data_ptr(), stride,
                                   *args(), seq.data_ptr(), 1, n, C, taps, own, 1e-5, _st()))
        if not own:
            ok(lib.mi355_hyb_conv_state_update(state2.data_ptr(), stride, hn.data_ptr(), C, 0, *args(), 1, C, taps, _st()))
        got2.append(host_dt(out, dtype))
        lo += n
    assert np.abs(np.concatenate(got2) - want).max() < (2e-5 if dtype == F32 else 2e-2) * max(1.0, np.abs(want).max())
    if taps > 1:
        assert np.abs(state2.cpu().numpy()[2, :C * (taps - 1)] - state.cpu().numpy()[2, :C * (taps - 1)]).max() < 1e-5
    # the rounded norm as the product's operand
    out = empty_dt((T, C), BF16)
    ok(lib.mi355_hyb_pre_norm(out.data_ptr(), BF16, P(x), P(nw), T, C, 1e-5, _st()))
    assert np.abs(host_dt(out, BF16) - h).max() < 1e-2 * np.abs(h).max()


def _tables(lib, dims, n_pos, base, scaling):
    """the framework's f64 table builder with the design's scaling"""
    from candle_vllm_amd.hybrid_model import KerolornSpec
    rs = KerolornSpec.rope_scaling({"dims": dims, "base": base, "scaling": scaling})
    cos, sin = np.zeros((n_pos, dims // 2), np.float32), np.zeros((n_pos, dims // 2), np.float32)
    assert lib.mi355_rope_tables_f64(cos.ctypes.data, sin.ctypes.data, dims, n_pos, float(base), ctypes.byref(rs), n_pos, n_pos) == 0
    return cos, sin


@pytest.mark.parametrize("dtype", [F32, BF16])
@pytest.mark.parametrize("Hh,G,d,vd,rot,scaling", [(4, 2, 16, 8, 8, {"factor": 6.0, "fast": 16.0, "original": 64, "slow": 1.5}),
                                                   (3, 3, 10, 5, 10, None), (1, 1, 2, 1, 2, {"factor": 0.5, "fast": 3.0, "original": 48, "slow": 0.25}),
                                                   (2, 1, 96, 64, 32, {"factor": 40.0, "fast": 32.0, "original": 128, "slow": 1.0}),
                                                   (2, 2, 24, 24, 0, None)])
def test_attn_prepare_interleaved_rotation_norm_behind_it_and_temperature(lib, dtype, Hh, G, d, vd, rot, scaling):
    """pairs (2i, 2i + 1) of the first `rot` dimensions turn (yarn frequencies, amplitude on cos and sin), THEN every head of q and k is
    divided by its root mean square (the amplitude only reaches the rotated part, so the order shows whenever rot < d), the query
    times the head's temperature; k and v land in their page rows"""
    _gpu()
    rng = np.random.default_rng(Hh * 7 + d)
    T, n_rows, base = 9, 40, 5000.0
    ldp = Hh * d + G * d + G * vd + 3
    proj = f32(2 * rng.standard_normal((T, ldp)))
    pos = rng.integers(0, 200, T)
    slots = rng.permutation(n_rows)[:T]
    temp = f32(rng.uniform(0.3, 1.5, Hh))
    q, k = proj[:, :Hh * d].reshape(T, Hh, d), proj[:, Hh * d:(Hh + G) * d].reshape(T, G, d)
    v = proj[:, (Hh + G) * d:(Hh + G) * d + G * vd].reshape(T, G, vd)
    if rot:
        f, amp = V.yarn_frequencies(base, rot, scaling)
        qr, kr = V.rotate_pairs(q, pos, f, amp), V.rotate_pairs(k, pos, f, amp)
        cos, sin = _tables(lib, rot, 256, base, scaling)
        pc, ps = P(cos), P(sin)
    else:
        qr, kr, pc, ps = q, k, None, None
    want_q, want_k = K.unit_rms(qr, 1e-5) * temp[None, :, None], K.unit_rms(kr, 1e-5)
    if rot and rot < d and scaling and scaling["factor"] != 1.0:           # the other order is a different function
        other = V.rotate_pairs(K.unit_rms(q, 1e-5), pos, f, amp) * temp[None, :, None]
        assert np.abs(other - want_q).max() > 1e-2
    qo, kp, vp = empty_dt((T, Hh, d), dtype), empty_dt((n_rows, G, d), dtype), empty_dt((n_rows, G, vd), dtype)
    ok(lib.mi355_hyb_attn_prepare_ex(qo.data_ptr(), kp.data_ptr(), vp.data_ptr(), P(proj), ldp, 0, Hh * d, (Hh + G) * d, None, None, pc, ps,
                                     P(pos, np.int64), P(slots, np.int64), T, Hh, G, d, vd, rot, 1, 2, P(temp), 1e-5, dtype, _st()))
    tol = 2e-6 if dtype == F32 else 8e-3
    assert np.abs(host_dt(qo, dtype) - want_q).max() < tol * max(1.0, np.abs(want_q).max())
    assert np.abs(host_dt(kp, dtype)[slots] - want_k).max() < tol * max(1.0, np.abs(want_k).max())
    assert np.abs(host_dt(vp, dtype)[slots] - v).max() < tol * max(1.0, np.abs(v).max())


def _scatter(n_rows, bs, free):
    nb = -(-n_rows // bs)
    table = [free.pop() for _ in range(nb)]
    slots = np.array([table[j // bs] * bs + j % bs for j in range(n_rows)])
    return table, slots


@pytest.mark.parametrize("dtype", [F32, BF16])
@pytest.mark.parametrize("Hh,G,d,vd,window,keep,bs,big", [(4, 2, 24, 40, 20, 5, 16, False), (3, 3, 8, 8, 9, 0, 8, False), (2, 1, 16, 130, 7, 30, 32, False),
                                                          (1, 1, 4, 2, 1, 1, 4, False), (2, 2, 16, 16, 0, 6, 16, False),
                                                          # prompt-sized steps; bf16 pages take the matrix-core kernel
                                                          (4, 2, 64, 48, 50, 11, 16, True), (6, 1, 96, 64, 80, 24, 64, True), (2, 1, 32, 16, 100, 130, 64, True),
                                                          (6, 2, 32, 32, 40, 7, 16, True), (3, 1, 128, 128, 0, 0, 32, True), (5, 1, 64, 64, 30, 2, 16, True)])
def test_window_that_keeps_the_first_tokens(lib, dtype, Hh, G, d, vd, window, keep, bs, big):
    """two unequal sequences in shuffled pages.  Dominant keys sit at the last kept position and at the first one that is not kept, at
    the window's first position and just below it -- seen from a late query each of them decides the output or must not be seen at all"""
    _gpu()
    rng = np.random.default_rng(Hh * 10 + d + window)
    lens, news = ([300, 213], [170, 213]) if big else ([90, 37], [9, 37])
    n_blocks = 64
    kp, vp = H.bf16_round(rng.standard_normal((n_blocks * bs, G, d))), H.bf16_round(rng.standard_normal((n_blocks * bs, G, vd)))
    free = list(rng.permutation(n_blocks))
    temp = np.ones(Hh)
    scale = 1.3 / math.sqrt(d)
    want, qs, tabs = [], [], []
    for L, n_new in zip(lens, news):
        k, v = H.bf16_round(rng.standard_normal((L, G, d))), H.bf16_round(rng.standard_normal((L, G, vd)))
        q = H.bf16_round(rng.standard_normal((n_new, Hh, d)))
        last = L - 1
        if window and last - window > keep + 1 > 1:
            for j in (keep - 1, keep, last - window + 1, last - window):    # kept, not kept, in the window, just out of it
                k[j, 0] = H.bf16_round(5.0 * q[n_new - 1, 0] * math.sqrt(d) / max(1e-6, np.linalg.norm(q[n_new - 1, 0])))
        table, slots = _scatter(L, bs, free)
        kp[slots], vp[slots] = k, v
        qs.append(q); tabs.append(table)
        qp = list(range(L - n_new, L))
        want.append(K.head_temperature_attention(q, k, v, qp, list(range(L)), scale, temp, window, keep))
        if window and last - window > keep + 1 > 1:
            for dw, dk in ((1, 0), (-1, 0), (0, 1), (0, -1)):              # one token off anywhere is another function
                o2 = K.head_temperature_attention(q, k, v, qp, list(range(L)), scale, temp, window + dw, keep + dk)
                assert np.abs(o2[-1] - want[-1][-1]).max() > 0.05
    T = sum(news)
    mb = max(len(t) for t in tabs)
    bt = np.zeros((2, mb), np.uint32)
    for i, t in enumerate(tabs):
        bt[i, :len(t)] = t
    cu = np.array([0, news[0], T], np.uint32)
    seq = torch.zeros(T, dtype=torch.int32, device="cuda")
    ok(lib.mi355_hyb_token_seq(seq.data_ptr(), P(cu, np.uint32), 2, _st()))
    dq, dk_, dv_ = dev_dt(np.concatenate(qs), dtype), dev_dt(kp, dtype), dev_dt(vp, dtype)
    wantc = np.concatenate(want)
    for mfma in (1, 2, 0):              # heads of a group in one workgroup; a wave per head; the generic kernel
        lib.mi355_hyb_set_attention_mfma(mfma)
        out = torch.zeros((T, Hh * vd), device="cuda")
        ok(lib.mi355_hyb_masked_attention(out.data_ptr(), F32, Hh * vd, 0, dq.data_ptr(), dk_.data_ptr(), dv_.data_ptr(), P(bt, np.uint32),
                                          P(lens, np.uint32), P(cu, np.uint32), seq.data_ptr(), None, 2, T, Hh, G, d, vd, bs, mb, window, keep,
                                          scale, 1.0, 0, 0, 0.0, 0, dtype, _st()))
        got = out.cpu().numpy().reshape(T, Hh, vd)
        assert np.abs(got - wantc).max() < (2e-5 if dtype == F32 else 2e-2) * max(1.0, np.abs(wantc).max()), mfma
    lib.mi355_hyb_set_attention_mfma(1)


@pytest.mark.parametrize("dtype", [F32, BF16])
@pytest.mark.parametrize("T,W,E,top,shared", [(5, 64, 8, 2, True), (3, 50, 5, 1, False), (7, 33, 70, 6, True), (2, 128, 130, 130, False),
                                              (4, 16, 1, 1, True), (40, 256, 16, 4, True)])
def test_router_softmax_correction_choice_and_weights(lib, dtype, T, W, E, top, shared):
    """the norm in front, f32 logits, softmax over ALL experts, the choice by s + correction (corrections large enough to overturn
    the order of s), weights = s of the chosen times the scale, not renormalised; the shared expert's sigmoid gate"""
    _gpu()
    rng = np.random.default_rng(T + W + E)
    x, nw = f32(2 * rng.standard_normal((T, W))), f32(1 + 0.2 * rng.standard_normal(W))
    wr, corr = f32(rng.standard_normal((E, W)) * 2.0 / math.sqrt(W)), f32(rng.choice([0.0, 0.02, 0.3], E))
    gate = f32(rng.standard_normal(W) / math.sqrt(W))
    h = H.rms_norm(x, nw, 1e-5)
    idx, wt = K.route(h, wr, corr, top, 1.7)
    plain, _ = K.route(h, wr, np.zeros(E), top, 1.7)
    if 1 < top < E and E > 4:
        assert not np.array_equal(np.sort(idx, 1), np.sort(plain, 1))       # the correction matters for the choice
    ids, wts, sg = torch.zeros((T, top), dtype=torch.int32, device="cuda"), torch.zeros((T, top), device="cuda"), torch.zeros(T, device="cuda")
    xn = empty_dt((T, W), dtype)
    ok(lib.mi355_hyb_moe_route(ids.data_ptr(), wts.data_ptr(), sg.data_ptr(), xn.data_ptr(), dtype, P(x), P(nw), P(wr), P(corr),
                               P(gate) if shared else None, T, W, E, top, 1.7, 1e-5, 0, _st()))
    assert np.array_equal(ids.cpu().numpy(), idx)
    assert np.abs(wts.cpu().numpy() - wt).max() < 2e-6 * 1.7
    assert np.abs(host_dt(xn, dtype) - h).max() < (2e-6 if dtype == F32 else 8e-3) * np.abs(h).max()
    if shared:
        assert np.abs(sg.cpu().numpy() - H.sigmoid(h @ gate)).max() < 2e-6
    if shared:                                                               # the shared expert as one more pair of every token
        ids2, wts2 = torch.zeros((T, top + 1), dtype=torch.int32, device="cuda"), torch.zeros((T, top + 1), device="cuda")
        ok(lib.mi355_hyb_moe_route(ids2.data_ptr(), wts2.data_ptr(), None, None, dtype, P(x), P(nw), P(wr), P(corr), P(gate), T, W, E, top, 1.7,
                                   1e-5, 1, _st()))
        assert np.array_equal(ids2.cpu().numpy(), np.concatenate([idx, np.full((T, 1), E)], axis=1))
        assert np.abs(wts2.cpu().numpy() - np.concatenate([wt, H.sigmoid(h @ gate)[:, None]], axis=1)).max() < 4e-6
    # without a norm in front and without a correction
    ok(lib.mi355_hyb_moe_route(ids.data_ptr(), wts.data_ptr(), None, None, dtype, P(h), None, P(wr), None, None, T, W, E, top, 1.0, 1e-5, 0, _st()))
    assert np.array_equal(ids.cpu().numpy(), plain)


@pytest.mark.parametrize("dtype", [F32, BF16])
@pytest.mark.parametrize("T,W,ff,E,top,bm", [(6, 64, 24, 6, 2, 16), (16, 48, 40, 70, 4, 16), (100, 64, 32, 4, 2, 64), (37, 50, 9, 3, 3, 64),
                                             (300, 128, 64, 3, 2, 128), (1, 32, 8, 5, 1, 16)])
def test_grouping_grouped_products_and_weighted_sum(lib, dtype, T, W, ff, E, top, bm):
    """(token, expert) pairs -> whole blocks of rows per expert; one launch multiplies every block with its expert's gate/up matrix,
    silu, one more with the down matrices; the weighted sum plus the gated shared output plus the output norm equals the oracle"""
    _gpu()
    if dtype == F32:
        bm = 64
    rng = np.random.default_rng(T + W + E)
    h = H.bf16_round(rng.standard_normal((T, W)))
    idx = np.stack([rng.permutation(E)[:top] for _ in range(T)]).astype(np.int32)
    if E > 2:
        idx[idx == 1] = 0 if top == 1 else idx[idx == 1]                 # (top 1: an expert that nobody chooses)
    wt = f32(rng.uniform(0.1, 1.0, (T, top)))
    Wt = {"m.e%d.%s" % (e, n): H.bf16_round(rng.standard_normal(s) / math.sqrt(s[1])) for e in range(E)
          for n, s in (("gate", (ff, W)), ("up", (ff, W)), ("down", (W, ff)))}
    shared_out, sgate = f32(rng.standard_normal((T, W))), f32(rng.uniform(0, 1, T))
    x0, nw = f32(rng.standard_normal((T, W))), f32(1 + 0.2 * rng.standard_normal(W))
    y = np.zeros((T, W))
    for t in range(T):
        for j in range(top):
            q = "m.e%d." % idx[t, j]
            y[t] += wt[t, j] * K.silu_expert(h[t:t + 1], Wt[q + "gate"], Wt[q + "up"], Wt[q + "down"])[0]
    want = x0 + H.rms_norm(y + sgate[:, None] * shared_out, nw, 1e-5)
    pairs = T * top
    nb = -(-pairs // bm) + E
    pos, rowtok, table = (torch.full((n,), -7, dtype=torch.int32, device="cuda") for n in (pairs, nb * bm, 2 * nb))
    ok(lib.mi355_hyb_moe_group(pos.data_ptr(), rowtok.data_ptr(), table.data_ptr(), P(idx, np.int32), pairs, top, E, bm, nb, _st()))
    pos_h, rt, tb = pos.cpu().numpy(), rowtok.cpu().numpy(), table.cpu().numpy().reshape(nb, 2)
    assert len(set(pos_h.tolist())) == pairs                                # every pair a row of its own ...
    for p_, r in enumerate(pos_h):
        e, end = tb[r // bm]
        assert e == idx.reshape(-1)[p_] and r < end and rt[r] == p_ // top  # ... inside a block of its expert, below the block's end
    counts = np.bincount(idx.reshape(-1), minlength=E)
    assert sum(-(-c // bm) for c in counts) == int((tb[:, 1] > 0).sum())
    gu_w = np.stack([np.concatenate([Wt["m.e%d.gate" % e], Wt["m.e%d.up" % e]]) for e in range(E)])
    dn_w = np.stack([Wt["m.e%d.down" % e] for e in range(E)])
    gu, act, yr = torch.zeros((nb * bm, 2 * ff), device="cuda"), empty_dt((nb * bm, ff), dtype), torch.zeros((nb * bm, W), device="cuda")
    dh, dgu, ddn = dev_dt(h, dtype), dev_dt(gu_w, dtype), dev_dt(dn_w, dtype)
    ok(lib.mi355_hyb_linear_grouped(gu.data_ptr(), 2 * ff, dh.data_ptr(), dtype, W, rowtok.data_ptr(), dgu.data_ptr(), 2 * ff * W, table.data_ptr(),
                                    bm, nb, 2 * ff, W, dtype, _st()))
    ok(lib.mi355_hyb_silu_glu(act.data_ptr(), dtype, gu.data_ptr(), nb * bm, ff, table.data_ptr(), bm, _st()))
    ok(lib.mi355_hyb_linear_grouped(yr.data_ptr(), W, act.data_ptr(), dtype, ff, None, ddn.data_ptr(), W * ff, table.data_ptr(), bm, nb, W, ff,
                                    dtype, _st()))
    dx = dev(x0)
    ok(lib.mi355_hyb_moe_combine_norm_add(dx.data_ptr(), None, yr.data_ptr(), pos.data_ptr(), P(wt), P(shared_out), P(sgate), P(nw), T, W, top,
                                          1e-5, _st()))
    assert np.abs(dx.cpu().numpy() - want).max() < (3e-5 if dtype == F32 else 3e-2) * max(1.0, np.abs(want).max())
    assert lib.mi355_hyb_moe_block_rows(pairs, E, 2 * ff, W, dtype) in (16, 64, 128)


# ------------------------------------------------------------------------------------------------------------ whole models
def _moe(E, top, ff, shared, scale=2.0):
    return {"expert": {"ff": ff}, "kind": "moe", "router": {"experts": E, "scale": scale, "top": top}, "shared": {"ff": shared} if shared else None}


def small_config(variant):
    if variant == 0:       # unequal layers: rotation on a part of the head with yarn, heads = kv heads, no mask, no feed-forward, no shared expert
        a0 = {"dim": 16, "heads": 4, "kv_heads": 2, "vdim": 8, "scale": 0.3, "mask": {"keep_first": 3, "size": 9},
              "rot": {"base": 2e4, "dims": 8, "scaling": {"factor": 6.0, "fast": 16.0, "original": 64, "slow": 1.5}}}
        a1 = {"dim": 8, "heads": 3, "kv_heads": 3, "vdim": 16, "scale": 0.4, "rot": {"base": 300.0, "dims": 8}}
        a2 = {"dim": 32, "heads": 2, "kv_heads": 1, "vdim": 32, "scale": 0.2, "mask": {"keep_first": 40, "size": 37},
              "rot": {"base": 1e6, "dims": 32, "scaling": {"factor": 0.5, "fast": 3.0, "original": 48, "slow": 0.25}}}
        a3 = {"dim": 16, "heads": 2, "kv_heads": 2, "vdim": 16, "scale": 0.25, "mask": {"keep_first": 0, "size": 70}, "rot": {"base": 1e4, "dims": 4}}
        layers = [{"type": "attention", "mixer": a0, "mlp": _moe(6, 2, 24, 40, 1.7)}, {"type": "attention", "mixer": a1, "mlp": None},
                  {"type": "attention", "mixer": a2, "mlp": _moe(5, 1, 16, 0, 0.8)}, {"type": "attention", "mixer": a3, "mlp": _moe(3, 3, 8, 8, 1.0)}]
        return {"architecture": "Kerolorn", "canon": {"taps": 3}, "layers": layers, "logit_scale": 1.5, "norm": {"eps": 1e-5}, "vocab": 100,
                "width": 64}
    if variant == 1:       # a configuration of ones
        a = {"dim": 2, "heads": 1, "kv_heads": 1, "vdim": 1, "scale": 1.0, "mask": {"keep_first": 1, "size": 1}, "rot": {"base": 10.0, "dims": 2}}
        return {"architecture": "Kerolorn", "canon": {"taps": 1}, "layers": [{"type": "attention", "mixer": a, "mlp": _moe(1, 1, 1, 1, 1.0)}],
                "logit_scale": 1.0, "norm": {"eps": 1e-6}, "vocab": 30, "width": 8}
    # sizes that take the matrix-core kernels (attention tiles, 64- and 128-row expert blocks)
    a = {"dim": 64, "heads": 4, "kv_heads": 2, "vdim": 32, "scale": 0.15, "mask": {"keep_first": 5, "size": 70},
         "rot": {"base": 5e5, "dims": 32, "scaling": {"factor": 4.0, "fast": 20.0, "original": 256, "slow": 1.5}}}
    # (a shared expert of the experts' size joins the grouped products; one of another size runs as dense products)
    layers = [{"type": "attention", "mixer": a, "mlp": _moe(8, 2, 64, 64, 2.25)}, {"type": "attention", "mixer": a, "mlp": _moe(2, 1, 32, 96, 1.0)}]
    return {"architecture": "Kerolorn", "canon": {"taps": 4}, "layers": layers, "logit_scale": 0.5, "norm": {"eps": 1e-5}, "vocab": 120, "width": 128}


def settle_router(W, rng):
    """routing for runs in 16 bits: rounding noise of about a percent in the residual stream flips a choice between two experts whose
    scores are close, and the oracle cannot follow such a flip.  Corrections that lie further apart than any two softmax values can
    (a random order of multiples of 1.5) settle WHICH experts a layer uses; the weights still come from the router's softmax.  The
    choice by token is what the f32 runs and the router's own test cover."""
    for k in list(W):
        if k.endswith("mlp.correction"):
            W[k] = H.bf16_round(1.5 * rng.permutation(W[k].shape[0]))


def build(cfg, dtype, seed=0, block_size=16, state_slots=4, sharp=False):
    from candle_vllm_amd.hybrid_model import HybridModel, KerolornSpec
    rng = np.random.default_rng(seed)
    W = K.random_kerolorn(rng, cfg)
    if sharp:
        settle_router(W, rng)
    spec = KerolornSpec(cfg, {k: v.shape for k, v in W.items()})
    m = HybridModel(spec, dtype=dtype, block_size=block_size, state_slots=state_slots)
    m.load_state_dict_f32(W)
    return m, W


def row_err(a, b):
    d = a - b
    d = d - d.mean(-1, keepdims=True)
    return np.sqrt((d * d).mean(-1)).max() / max(1e-9, np.sqrt((b * b).mean()))


TOL = {"float32": 3e-5, "bfloat16": 4e-2}
CLOSE_CALL = 3e-6          # a choice between two experts whose scores lie closer than this may fall either way in f32


def oracle_logits(cfg, W, toks, rng=None):
    """the oracle's logits (and trace) for one request; no routing decision of the run may be a close call -- with `rng`, tokens are
    drawn again until none is (the tokens are returned too)"""
    for _ in range(30):
        o = K.KerolornOracle(cfg, W)
        out, tr = o.feed(toks)
        if not o.margins or min(o.margins) > CLOSE_CALL:
            return out, tr, toks
        assert rng is not None, "a routing decision of this test is a close call: take other tokens"
        toks = rng.integers(0, cfg["vocab"], len(toks)).tolist()
    raise AssertionError("no token sequence without a close call")


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("variant", [0, 1, 2])
def test_model_whole_portions_decode_against_oracle(lib, dtype, variant):
    """one request whole, with the residual stream behind every layer; then the same tokens in portions of 2, 1, 17, ... tokens and
    token by token: every way must give the oracle's logits at every position (windows of 9, 37 and 70 and kept tokens pass over page
    borders of 16 in the prompt and in decoding; the convolution's tail crosses every cut)"""
    _gpu()
    from candle_vllm_amd.step_engine import StepEngine
    cfg = small_config(variant)
    m, W = build(cfg, dtype, seed=variant, sharp=dtype == "bfloat16")
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
    tol = TOL[dtype]
    assert row_err(got.cpu().numpy(), want) < tol
    for cuts in ([2, 1, 17, 1, 1, 2, 30, 3, 18], [40] + [1] * 35, [1] * 20 + [55]):
        cuts = cuts + ([n - 75] if n > 75 else [])
        assert sum(cuts) == n
        lo, rows = 0, []
        for c in cuts:
            eng.feed("b", toks[lo:lo + c])
            rows.append(eng.step(["b"], [list(range(c))]).cpu().numpy())
            lo += c
        eng.finish("b")
        assert row_err(np.concatenate(rows), want) < tol, cuts
        assert eng.free_pages() == eng.num_blocks and eng.be.state_free_slots() == 4


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_unequal_batches_pages_and_slots_reused(lib, dtype):
    """five requests of unequal length through four slots and a pool that only fits them because pages come back: portions of some
    beside single tokens of others, a request that sits steps out, a late one that takes over a freed slot and freed pages --
    every logit must equal the request run alone in the oracle"""
    _gpu()
    from candle_vllm_amd.step_engine import StepEngine
    cfg = small_config(0)
    m, W = build(cfg, dtype, seed=3, sharp=dtype == "bfloat16")
    rng = np.random.default_rng(21)
    lens = {"a": 70, "b": 33, "c": 5, "d": 48, "e": 41}
    toks = {r: rng.integers(0, cfg["vocab"], n).tolist() for r, n in lens.items()}
    for r in toks:
        toks[r] = oracle_logits(cfg, W, toks[r], rng)[2]
    want = {r: K.KerolornOracle(cfg, W).feed(toks[r])[0] for r in toks}
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


def _sharp_config(window, keep):
    a = {"dim": 8, "heads": 2, "kv_heads": 1, "vdim": 16, "scale": 6.0, "mask": {"keep_first": keep, "size": window}, "rot": {"base": 10.0, "dims": 2}}
    return {"architecture": "Kerolorn", "canon": {"taps": 2}, "layers": [{"type": "attention", "mixer": a, "mlp": None}], "logit_scale": 1.0,
            "norm": {"eps": 1e-5}, "vocab": 50, "width": 32}


def test_window_edge_kept_tokens_and_temperature_show_in_the_logits(lib):
    """an attention model made sharp (large scale): the oracle's logits with the window or the number of kept tokens one off, or
    with the temperatures left out, differ by far more than the tolerance, and the engine matches the right one, in the prompt and
    in decoding"""
    _gpu()
    from candle_vllm_amd.step_engine import StepEngine
    cfg = _sharp_config(21, 4)
    m, W = build(cfg, "float32", seed=8)
    W["l0.mix.temp"] = H.bf16_round(np.array([0.5, 1.75]))
    m.load_state_dict_f32(W)
    rng = np.random.default_rng(2)
    toks = rng.integers(0, 50, 60).tolist()
    want, _ = K.KerolornOracle(cfg, W).feed(toks)
    for dw, dk in ((-1, 0), (1, 0), (0, -1), (0, 1)):
        other, _ = K.KerolornOracle(_sharp_config(21 + dw, 4 + dk), W).feed(toks)
        assert row_err(other[30:], want[30:]) > 100 * TOL["float32"], (dw, dk)
    ones = dict(W)
    ones["l0.mix.temp"] = np.ones(2)
    assert row_err(K.KerolornOracle(cfg, ones).feed(toks)[0], want) > 100 * TOL["float32"]
    eng = StepEngine(m, 64)
    eng.feed("a", toks[:40])
    rows = [eng.step(["a"], [list(range(40))]).cpu().numpy()]
    for t in toks[40:]:
        eng.feed("a", [t])
        rows.append(eng.step(["a"]).cpu().numpy())
    assert row_err(np.concatenate(rows), want) < TOL["float32"]


def test_far_key_hundreds_back_decides_a_late_token(lib):
    """no window: the key of a token 400 positions back is made to match a late query exactly as well as the late token's own key
    (keys are the queries' first head; the two tokens' embeddings differ by a vector that this head's projection does not see), while
    their values differ -- so the late token's output is half the far value, and losing far pages changes the logits by far more than
    the tolerance.  Prompt in portions over many pages, then decoding"""
    _gpu()
    from candle_vllm_amd.step_engine import StepEngine
    a = {"dim": 16, "heads": 2, "kv_heads": 1, "vdim": 16, "scale": 5.0}
    cfg = {"architecture": "Kerolorn", "canon": {"taps": 2}, "layers": [{"type": "attention", "mixer": a, "mlp": None}], "logit_scale": 2.0,
           "norm": {"eps": 1e-5}, "vocab": 60, "width": 32}
    m, W = build(cfg, "float32", seed=9)
    W["l0.mix.k"] = W["l0.mix.q"][:16].copy()                              # key of a token = query of the same token (head 0)
    W["l0.canon1"][:] = 0.0                                                # the mixer reads the normed token alone
    W["l0.norm1"][:] = 1.0
    _, _, vt = np.linalg.svd(W["l0.mix.q"][:16])
    W["embed"][58] = H.bf16_round(W["embed"][59] + vt[16:].T @ np.random.default_rng(1).standard_normal(16))
    m.load_state_dict_f32(W)
    rng = np.random.default_rng(5)
    toks = rng.integers(0, 58, 470).tolist()
    toks[30] = 59                                                          # the only 59 ...
    toks[440] = 58                                                         # ... and the only 58, whose query points at it
    want, _ = K.KerolornOracle(cfg, W).feed(toks)
    cut = [t for i, t in enumerate(toks) if i != 30]                       # the same sequence without the far token
    other, _ = K.KerolornOracle(cfg, W).feed(cut)
    assert row_err(other[439:440], want[440:441]) > 100 * TOL["float32"]
    eng = StepEngine(m, 480)
    rows, lo = [], 0
    for c in [100, 3, 157, 2, 178]:
        eng.feed("a", toks[lo:lo + c])
        rows.append(eng.step(["a"], [list(range(c))]).cpu().numpy())
        lo += c
    for t in toks[440:]:
        eng.feed("a", [t])
        rows.append(eng.step(["a"]).cpu().numpy())
    assert row_err(np.concatenate(rows), want) < TOL["float32"]


def test_long_decoding_and_first_tokens(lib):
    _gpu()
    from candle_vllm_amd.step_engine import StepEngine
    cfg = small_config(0)
    m, W = build(cfg, "float32", seed=5)
    rng = np.random.default_rng(4)
    toks = rng.integers(0, cfg["vocab"], 200).tolist()
    want, _, toks = oracle_logits(cfg, W, toks, rng)
    eng = StepEngine(m, 208)
    rows = []
    for t in toks:                                                          # from the very first token on, one at a time
        eng.feed("a", [t])
        rows.append(eng.step(["a"]).cpu().numpy())
    assert row_err(np.concatenate(rows)[:4], want[:4]) < TOL["float32"]
    assert row_err(np.concatenate(rows), want) < TOL["float32"]


def test_more_taps_than_the_single_launch_takes(lib):
    """ten taps: the norm, the convolution and the move of its state run as three launches; portions shorter than the taps and single
    tokens continue from the slot"""
    _gpu()
    from candle_vllm_amd.step_engine import StepEngine
    cfg = dict(small_config(0), canon={"taps": 10})
    m, W = build(cfg, "float32", seed=14)
    rng = np.random.default_rng(15)
    toks = rng.integers(0, cfg["vocab"], 60).tolist()
    want, _, toks = oracle_logits(cfg, W, toks, rng)
    eng = StepEngine(m, 64)
    lo, rows = 0, []
    for c in [3, 1, 1, 12, 2, 9, 1, 1, 1, 29]:
        eng.feed("a", toks[lo:lo + c])
        rows.append(eng.step(["a"], [list(range(c))]).cpu().numpy())
        lo += c
    assert lo == 60 and row_err(np.concatenate(rows), want) < TOL["float32"]


def test_graph_replays_equal_eager_steps(lib):
    """decoding batches replay a captured hipGraph: every replay, with eager prompt portions of other requests between them, gives the
    eager step's logits bit for bit"""
    _gpu()
    from candle_vllm_amd.step_engine import StepEngine
    cfg = small_config(0)
    m, W = build(cfg, "bfloat16", seed=12)
    rng = np.random.default_rng(13)
    toks = {r: rng.integers(0, cfg["vocab"], 60).tolist() for r in "ab"}
    outs = {}
    for use_graph in (False, True):
        eng = StepEngine(m, 256)
        eng.use_graph = use_graph
        rows = []
        eng.feed("a", toks["a"][:20]); eng.feed("b", toks["b"][:33])
        rows.append(eng.step(["a", "b"]).cpu().numpy())
        for i in range(20):
            eng.feed("a", toks["a"][20 + i:21 + i]); eng.feed("b", toks["b"][33 + i:34 + i])
            rows.append(eng.step(["a", "b"]).cpu().numpy())
            if i == 7:
                eng.feed("c", toks["a"][:25]); rows.append(eng.step(["c"]).cpu().numpy()); eng.finish("c")
        eng.finish("a"); eng.finish("b")
        outs[use_graph] = np.concatenate(rows)
    assert np.array_equal(outs[False], outs[True])
    cap, rep = m.graph_stats()
    assert cap >= 1 and rep >= 15


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
    n_new = 12
    want = []
    for p in prompts:
        o = K.KerolornOracle(cfg, W)
        lg, _ = o.feed(p)
        out = []
        for _ in range(n_new):
            t = int(lg[-1].argmax())
            out.append(t)
            lg, _ = o.feed([t])
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


# ------------------------------------------------------------------------------------------------------------ random configurations
def random_config(rng):
    """sizes, head counts, depth, windows, kept tokens, taps, expert counts and constants drawn at random (sizes that are not all
    multiples of 16 or 32; layers without a feed-forward, without a shared expert, without a mask, with rotation on a part of the head)"""
    width = int(rng.choice([96, 100, 128, 160, 256, 320]))

    def att():
        G, d = int(rng.choice([1, 2, 3, 4])), int(rng.choice([16, 20, 32, 40, 64, 96, 128]))
        m = {"dim": d, "heads": G * int(rng.choice([1, 2, 3, 4])), "kv_heads": G, "scale": float(d ** -0.5 * rng.uniform(0.7, 1.5)),
             "vdim": int(rng.choice([8, 16, 24, 48, 64, 96, 128]))}
        if rng.random() < 0.85:
            m["mask"] = {"size": int(rng.integers(5, 200)), "keep_first": int(rng.choice([0, 1, 4, 20, 64, 100]))}
        if rng.random() < 0.9:
            m["rot"] = {"base": float(rng.choice([1e3, 1e4, 5e5, 123456.0])), "dims": int(rng.choice([r for r in (2, 8, 16, 32, 64, 96, 128) if r <= d]))}
            if rng.random() < 0.8:
                m["rot"]["scaling"] = {"factor": float(rng.choice([2.0, 3.5, 8.0, 16.0, 40.0])), "fast": float(rng.choice([8.0, 16.0, 32.0, 64.0])),
                                       "original": int(rng.choice([64, 256, 1024, 4096])), "slow": float(rng.choice([0.5, 1.0, 2.0]))}
        return m

    def mlp():
        if rng.random() < 0.15:
            return None
        E = int(rng.choice([2, 4, 7, 16, 24, 64]))
        return _moe(E, int(rng.integers(1, min(E, 8) + 1)), int(rng.choice([24, 50, 64, 96, 160])), int(rng.choice([0, 32, 96, 200])),
                    float(rng.choice([1.0, 3.0, 0.5])))
    kinds = [att() for _ in range(3)]
    layers = [{"type": "attention", "mixer": kinds[int(rng.integers(0, 3))], "mlp": mlp()} for _ in range(int(rng.integers(2, 7)))]
    return {"architecture": "Kerolorn", "canon": {"taps": int(rng.integers(2, 6))}, "layers": layers, "logit_scale": float(rng.choice([1.0, 2.0, 0.25])),
            "norm": {"eps": float(rng.choice([1e-5, 1e-6]))}, "vocab": int(rng.integers(50, 600)), "width": width}


@pytest.mark.parametrize("seed", [2, 11, 21, 33, 47])
def test_random_configurations_whole_and_mixed_schedules(lib, seed):
    """three unequal requests of a random configuration: each alone in one step, then together in a random schedule of portions (2, 3,
    17, 64, 65, 100 tokens; a request may sit a step out) that ends token by token -- on 64-token pages, in f32 and bf16"""
    _gpu()
    from candle_vllm_amd.step_engine import StepEngine
    from candle_vllm_amd.hybrid_model import HybridModel, KerolornSpec
    rng = np.random.default_rng(seed)
    cfg = random_config(rng)
    W = K.random_kerolorn(rng, cfg)
    lens = [int(rng.integers(150, 420)), int(rng.integers(1, 40)), int(rng.integers(60, 130))]
    toks = [rng.integers(0, cfg["vocab"], n).tolist() for n in lens]
    toks = [oracle_logits(cfg, W, t, rng)[2] for t in toks]
    want = [K.KerolornOracle(cfg, W).feed(t)[0] for t in toks]
    for dtype in ("float32", "bfloat16"):
        if dtype == "bfloat16":
            settle_router(W, rng)
            want = [K.KerolornOracle(cfg, W).feed(t)[0] for t in toks]
        m = HybridModel(KerolornSpec(cfg, {k: v.shape for k, v in W.items()}), dtype=dtype, block_size=64, state_slots=4)
        m.load_state_dict_f32(W)
        eng = StepEngine(m, 64 * 12)
        for i, t in enumerate(toks):
            eng.feed("w", t)
            assert row_err(eng.step(["w"], [list(range(len(t)))]).cpu().numpy(), want[i]) < TOL[dtype], (dtype, "whole", i)
            eng.finish("w")
        at, got = [0, 0, 0], [[], [], []]
        while any(a < n for a, n in zip(at, lens)):
            ids, w, take = [], [], []
            for i in range(3):
                if at[i] >= lens[i] or rng.random() < 0.2:
                    continue
                left = lens[i] - at[i]
                c = 1 if left <= 20 else int(min(left - 20, rng.choice([2, 3, 17, 64, 65, 100])))
                eng.feed("r%d" % i, toks[i][at[i]:at[i] + c])
                ids.append("r%d" % i); w.append(list(range(c))); take.append((i, c))
                at[i] += c
            if not ids:
                continue
            out, lo = eng.step(ids, w).cpu().numpy(), 0
            for i, c in take:
                got[i].append(out[lo:lo + c]); lo += c
                if at[i] == lens[i]:
                    eng.finish("r%d" % i)
        for i in range(3):
            assert row_err(np.concatenate(got[i]), want[i]) < TOL[dtype], (dtype, "schedule", i)
        assert eng.free_pages() == eng.num_blocks and eng.be.state_free_slots() == 4


# ------------------------------------------------------------------------------------------------------------ the trace runner
def _write_model(folder, cfg, W):
    """config.json + model.safetensors (bf16; 8-byte header length, JSON header, data) of a configuration"""
    import json
    import struct
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
    """bin/trace_run as a user starts it: a folder with config.json and model.safetensors of a configuration of other sizes, steps on
    standard input -- six requests over time, at most four alive, portions beside single tokens, a pool that only fits because ended
    requests give their pages and slots back -- and the logits it writes equal the oracle's for every request alone"""
    _gpu()
    import json
    import os
    import subprocess
    import sys
    cfg = small_config(0)
    rng = np.random.default_rng(17)
    W = K.random_kerolorn(rng, cfg)
    if dtype == "bfloat16":
        settle_router(W, rng)
    _write_model(tmp_path, cfg, W)
    lens = {"a": 150, "b": 40, "c": 3, "d": 90, "e": 61, "f": 130}
    toks = {r: oracle_logits(cfg, W, rng.integers(0, cfg["vocab"], n).tolist(), rng)[2] for r, n in lens.items()}
    want = {r: K.KerolornOracle(cfg, W).feed(toks[r])[0] for r in toks}
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
    # live at any time: a, b, c, d (64-token pages: 192 + 64 + 64 + 128), then e and f in what comes back
    r = subprocess.run([sys.executable, os.path.join(root, "bin", "trace_run"), "--model", str(tmp_path), "--dtype", dtype, "--out", str(out),
                        "--max-tokens", "448"], input="\n".join(steps) + "\n", capture_output=True, text=True, timeout=170)
    assert r.returncode == 0, r.stderr[-2000:]
    assert [l for l in r.stdout.splitlines() if l.startswith("done ")] == ["done %d" % n for n in range(len(sched))]
    V_ = cfg["vocab"]
    for n, got in enumerate(rows):
        a = np.fromfile(out / ("%d.f32" % n), "<f4").reshape(len(got), V_)
        ref = np.stack([want[r_][p_] for r_, p_ in got])
        assert row_err(a, ref) < TOL[dtype], (n, dtype)
