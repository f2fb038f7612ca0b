"""Host side of the Kerolorn design, no GPU: config.json -> layer structs and weight slots (every size from the config or a tensor's
shape, absent parts), the registry, what the host layer refuses, and the oracle's own invariants (portions equal the whole; the
window with kept first tokens, the router's choice and weights, the input convolution and the norm behind the rotation by hand)."""
import ctypes
import math

import numpy as np
import pytest

from oracle import hybrid as H
from oracle import vivazen as V
from oracle import kerolorn as K


def _cfg():
    rot = {"base": 3000.0, "dims": 6, "scaling": {"factor": 8.0, "fast": 6.0, "original": 40, "slow": 0.5}}
    a = {"dim": 10, "heads": 6, "kv_heads": 2, "vdim": 14, "scale": 0.4, "mask": {"keep_first": 3, "size": 11}, "rot": rot}
    b = {"dim": 8, "heads": 2, "kv_heads": 2, "vdim": 4, "scale": 0.7, "rot": {"base": 100.0, "dims": 8}}
    moe = {"expert": {"ff": 12}, "kind": "moe", "router": {"experts": 5, "scale": 1.5, "top": 2}, "shared": {"ff": 20}}
    moe2 = {"expert": {"ff": 7}, "kind": "moe", "router": {"experts": 3, "scale": 1.0, "top": 1}, "shared": None}
    return {"architecture": "Kerolorn", "canon": {"taps": 3}, "logit_scale": 1.5, "norm": {"eps": 1e-5}, "vocab": 97, "width": 56,
            "layers": [{"type": "attention", "mixer": a, "mlp": moe}, {"type": "attention", "mixer": b, "mlp": None},
                       {"type": "attention", "mixer": a, "mlp": moe2}]}


def test_spec_reads_every_size_from_config_and_shapes(lib):
    from candle_vllm_amd import hybrid_model as hm
    cfg = _cfg()
    W = K.random_kerolorn(np.random.default_rng(0), cfg)
    spec = hm.KerolornSpec(cfg, {k: v.shape for k, v in W.items()})
    a, b, c = spec.layers
    assert (spec.residual_form, spec.norm_groups, spec.logit_scale) == (2, 1, 1.5)
    assert (a.mixer, a.a_heads, a.a_kv_heads, a.a_dim, a.a_vdim, a.a_window, a.a_keep_first, a.a_rot_dims, a.a_rot_interleaved, a.a_qk_norm,
            a.a_norm_after_rot, a.a_head_temp, a.in_conv, a.a_has_sink) == (hm.MIX_ATTENTION, 6, 2, 10, 14, 11, 3, 6, 1, 1, 1, 1, 3, 0)
    assert (a.mlp_kind, a.mlp_ff, a.moe_experts, a.moe_top, a.moe_shared_ff) == (hm.MLP_MOE, 12, 5, 2, 20) and abs(a.moe_scale - 1.5) < 1e-7
    assert (b.a_window, b.a_keep_first, b.a_rot_dims, b.mlp_kind, b.moe_experts) == (0, 0, 8, 0, 0)
    assert (c.mlp_ff, c.moe_experts, c.moe_top, c.moe_shared_ff) == (7, 3, 1, 0)
    offs = (ctypes.c_int32 * 9)()
    assert lib.mi355_hybrid_in_proj_rows(ctypes.byref(a), offs) == 60 + 20 + 28 and list(offs)[:4] == [0, 60, 80, -1]
    s0 = spec.slots[0]
    assert s0[hm.HW_PRE_NORM1] == ["l0.norm1"] and s0[hm.HW_NORM1] == ["l0.norm1b"] and s0[hm.HW_PRE_NORM2] == ["l0.norm2"] and s0[hm.HW_NORM2] == ["l0.norm2b"]
    assert s0[hm.HW_MOE_ROUTER] == ["l0.mlp.router", "l0.mlp.shared.sg"] and spec.slots[2][hm.HW_MOE_ROUTER] == ["l2.mlp.router"]
    assert s0[hm.HW_MOE_GATE_UP][:3] == ["l0.mlp.e0.gate", "l0.mlp.e0.up", "l0.mlp.e1.gate"] and len(s0[hm.HW_MOE_GATE_UP]) == 10
    assert s0[hm.HW_MOE_DOWN] == ["l0.mlp.e%d.down" % e for e in range(5)]
    assert s0[hm.HW_MLP_GATE_UP] == ["l0.mlp.shared.gate", "l0.mlp.shared.up"] and hm.HW_MLP_GATE_UP not in spec.slots[2]
    assert s0[hm.HW_IN_CONV] == ["l0.canon1"] and s0[hm.HW_A_TEMP] == ["l0.mix.temp"]
    assert hm.HW_NORM2 not in spec.slots[1] and hm.HW_MOE_ROUTER not in spec.slots[1]
    used = {n for sl in spec.slots for names in sl.values() for n in names} | {"embed", "final.norm", "head"}
    assert used == set(W)                                                    # every tensor of the checkpoint has a slot
    rs = spec.rope_scaling(cfg["layers"][0]["mixer"]["rot"])
    assert (rs.type, rs.factor, rs.beta_fast, rs.beta_slow, rs.original_max_position_embeddings) == (hm.ROPE_YARN, 8.0, 6.0, 0.5, 40.0)
    assert spec.rope_scaling(cfg["layers"][1]["mixer"]["rot"]).type == hm.ROPE_DEFAULT
    with pytest.raises(ValueError):
        hm.KerolornSpec({**cfg, "layers": [{"type": "delta", "mixer": dict(cfg["layers"][0]["mixer"]), "mlp": None}]}, {})
    with pytest.raises(ValueError):
        hm.KerolornSpec({**cfg, "canon": {"taps": 4}}, {k: v.shape for k, v in W.items()})       # the tensors have three taps


def test_absent_parts(lib):
    from candle_vllm_amd import hybrid_model as hm
    cfg = _cfg()
    a = cfg["layers"][0]["mixer"]
    del a["rot"], a["mask"]
    W = K.random_kerolorn(np.random.default_rng(0), cfg)
    for k in [k for k in W if k.endswith(("canon1", "mix.temp", "mlp.correction"))]:
        del W[k]
    spec = hm.KerolornSpec(cfg, {k: v.shape for k, v in W.items()})
    L = spec.layers[0]
    assert (L.a_rot_dims, L.a_window, L.a_keep_first, L.in_conv, L.a_head_temp) == (0, 0, 0, 0, 0) and spec.rope[0] is None
    assert hm.HW_MOE_CORRECTION not in spec.slots[0] and hm.HW_IN_CONV not in spec.slots[0]


def test_shared_expert_of_the_experts_size_joins_the_grouped_matrices(lib):
    from candle_vllm_amd import hybrid_model as hm
    cfg = _cfg()
    cfg["layers"][0]["mlp"]["shared"] = {"ff": 12}
    W = K.random_kerolorn(np.random.default_rng(0), cfg)
    spec = hm.KerolornSpec(cfg, {k: v.shape for k, v in W.items()})
    s0 = spec.slots[0]
    assert s0[hm.HW_MOE_GATE_UP][-2:] == ["l0.mlp.shared.gate", "l0.mlp.shared.up"] and len(s0[hm.HW_MOE_GATE_UP]) == 12
    assert s0[hm.HW_MOE_DOWN][-1] == "l0.mlp.shared.down" and hm.HW_MLP_GATE_UP not in s0 and hm.HW_MLP_DOWN not in s0
    assert s0[hm.HW_MOE_ROUTER] == ["l0.mlp.router", "l0.mlp.shared.sg"]


def test_registry_knows_the_design_and_its_component(lib):
    from candle_vllm_amd import registry
    assert "Kerolorn" in registry.registered()
    assert registry.component_of({"architecture": "Kerolorn"}) == "hybrid"


def test_host_layer_refuses_what_it_cannot_run(lib):
    from candle_vllm_amd import hybrid_model as hm
    cfg = _cfg()
    W = K.random_kerolorn(np.random.default_rng(0), cfg)
    spec = hm.KerolornSpec(cfg, {k: v.shape for k, v in W.items()})
    n = len(spec.layers)
    arr = (hm.HybridLayer * n)(*spec.layers)
    c = hm.HybridConfig(width=56, vocab=97, n_layers=n, dtype=hm.DT_F32, block_size=16, state_slots=2, norm_eps=1e-5, unit_eps=1e-6,
                        residual_form=2, resid_alpha=1.0, norm_groups=1, logit_scale=1.5)
    h = lib.mi355_hybrid_create(ctypes.byref(c), arr)
    assert h
    # the state slot holds the input convolution's last rows of every layer
    assert lib.mi355_hybrid_state_floats_per_slot(h) == 3 * 56 * 2
    lib.mi355_hybrid_destroy(h)
    c.residual_form = 1                                                      # experts in front of a norm behind the residual sum
    assert not lib.mi355_hybrid_create(ctypes.byref(c), arr)
    c.residual_form = 2
    for field, bad in (("moe_top", 6), ("moe_experts", 0), ("a_keep_first", -1), ("in_conv", 17)):
        keep = getattr(arr[0], field)
        setattr(arr[0], field, bad)
        assert not lib.mi355_hybrid_create(ctypes.byref(c), arr), field
        setattr(arr[0], field, keep)
    assert lib.mi355_hyb_moe_block_rows(32, 64, 512, 256, hm.DT_BF16) == 16
    assert lib.mi355_hyb_moe_block_rows(8192, 8, 512, 256, hm.DT_BF16) == 128
    assert lib.mi355_hyb_moe_block_rows(8192, 8, 512, 250, hm.DT_BF16) == 64
    assert lib.mi355_hyb_moe_block_rows(8192, 8, 512, 256, hm.DT_F32) == 64


# ------------------------------------------------------------------------------------------------------------ the oracle itself
def test_oracle_portions_equal_the_whole():
    cfg = _cfg()
    W = K.random_kerolorn(np.random.default_rng(1), cfg)
    toks = np.random.default_rng(2).integers(0, 97, 50).tolist()
    whole, tr = K.KerolornOracle(cfg, W).feed(toks)
    o = K.KerolornOracle(cfg, W)
    parts = [o.feed(toks[lo:hi])[0] for lo, hi in ((0, 1), (1, 3), (3, 20), (20, 21), (21, 50))]
    assert np.abs(np.concatenate(parts) - whole).max() < 1e-9
    assert tr.shape == (3, 50, 56)
    half = {**cfg, "logit_scale": 0.75}
    assert np.allclose(K.KerolornOracle(half, W).feed(toks)[0] * 2, whole)


def test_oracle_mask_router_convolution_and_norm_order():
    rng = np.random.default_rng(3)
    # window 4 with 2 kept tokens: a query at 10 sees 7 .. 10 and 0, 1
    vis = K.window_keep_mask([10, 3], range(11), 4, 2)
    assert vis[0].nonzero()[0].tolist() == [0, 1, 7, 8, 9, 10] and vis[1].nonzero()[0].tolist() == [0, 1, 2, 3]
    assert K.window_keep_mask([10], range(11), 0, 2).sum() == 11
    # uniform scores: the output is the mean of the visible values; a temperature scales the scores of its head only
    T, Hh, G, d, vd = 11, 2, 1, 4, 3
    k, v = rng.standard_normal((T, G, d)), rng.standard_normal((T, G, vd))
    o = K.head_temperature_attention(np.zeros((1, Hh, d)), k, v, [10], range(T), 1.0, np.ones(Hh), 4, 2)
    assert np.allclose(o[0, 0], v[[0, 1, 7, 8, 9, 10], 0].mean(0))
    q = rng.standard_normal((1, Hh, d))
    a = K.head_temperature_attention(q, k, v, [10], range(T), 0.5, np.array([1.0, 3.0]), 0, 0)
    b = K.head_temperature_attention(q, k, v, [10], range(T), 1.5, np.array([1.0 / 3.0, 1.0]), 0, 0)
    assert np.allclose(a, b)
    # router: softmax over all experts, the correction moves the choice and not the weights
    h, wr = rng.standard_normal((6, 8)), rng.standard_normal((5, 8))
    z = h @ wr.T
    s = np.exp(z) / np.exp(z).sum(1, keepdims=True)
    idx, wt = K.route(h, wr, np.zeros(5), 2, 3.0)
    assert np.array_equal(idx[:, 0], s.argmax(1)) and np.allclose(wt[:, 0], 3.0 * s.max(1))
    corr = np.array([0.0, 0.0, 0.0, 0.0, 5.0])
    idx2, wt2 = K.route(h, wr, corr, 2, 3.0)
    assert np.all(idx2[:, 0] == 4) and np.allclose(wt2[:, 0], 3.0 * s[:, 4]) and np.array_equal(idx2[:, 1], idx[:, 0] * (idx[:, 0] != 4) + idx[:, 1] * (idx[:, 0] == 4))
    # h + conv(h): one tap = a scale; the last column multiplies the current row; portions with the tail equal the whole
    x = rng.standard_normal((9, 5))
    assert np.allclose(K.conv_residual(x, np.full((5, 1), 0.5))[0], 1.5 * x)
    w = rng.standard_normal((5, 3))
    y, _ = K.conv_residual(x, w)
    assert np.allclose(y[0], x[0] * (1 + w[:, 2])) and np.allclose(y[4], x[4] * (1 + w[:, 2]) + x[3] * w[:, 1] + x[2] * w[:, 0])
    y1, tail = K.conv_residual(x[:4], w)
    y2, _ = K.conv_residual(x[4:], w, tail)
    assert np.allclose(np.concatenate([y1, y2]), y)
    # the norm behind the rotation sees the amplitude of the rotated part only
    f, amp = V.yarn_frequencies(1000.0, 4, {"factor": 16.0, "fast": 32.0, "original": 64, "slow": 1.0})
    u = rng.standard_normal((3, 2, 8))
    r = K.unit_rms(V.rotate_pairs(u, [1, 5, 9], f, amp), 0.0)
    assert np.allclose((r ** 2).mean(-1), 1.0) and abs(amp - (0.1 * math.log(16.0) + 1)) < 1e-12
    assert not np.allclose(r, V.rotate_pairs(K.unit_rms(u, 0.0), [1, 5, 9], f, amp))
    # moe = weighted chosen experts + gated shared expert
    Wm = {"m.router": wr, "m.correction": corr}
    for e in range(5):
        Wm.update({"m.e%d.gate" % e: rng.standard_normal((3, 8)), "m.e%d.up" % e: rng.standard_normal((3, 8)), "m.e%d.down" % e: rng.standard_normal((8, 3))})
    Wm.update({"m.shared.gate": rng.standard_normal((4, 8)), "m.shared.up": rng.standard_normal((4, 8)), "m.shared.down": rng.standard_normal((8, 4)),
               "m.shared.sg": rng.standard_normal((1, 8))})
    y = K.moe(h, Wm, "m.", 5, 2, 3.0, True)
    t = 2
    by_hand = sum(wt2[t, j] * (H.silu(Wm["m.e%d.gate" % idx2[t, j]] @ h[t]) * (Wm["m.e%d.up" % idx2[t, j]] @ h[t])) @ Wm["m.e%d.down" % idx2[t, j]].T
                  for j in range(2))
    by_hand = by_hand + H.sigmoid(Wm["m.shared.sg"][0] @ h[t]) * ((H.silu(Wm["m.shared.gate"] @ h[t]) * (Wm["m.shared.up"] @ h[t])) @ Wm["m.shared.down"].T)
    assert np.allclose(y[t], by_hand)
