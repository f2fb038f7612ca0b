"""Host side of the Sabolorn design, no GPU: config.json -> layer structs and weight slots (every size from the config or a tensor's
shape, absent parts), the registry, the rotation tables against the oracle's angles for several scalings, what the host layer
refuses, and the oracle's own invariants by hand (the scan in portions equals the whole, the group-limited choice, the distance bias,
the convolution, the layer norm)."""
import ctypes
import math

import numpy as np
import pytest

from oracle import sabolorn as S


def _cfg():
    rot = {"base": 5000.0, "dims": 8, "scaling": {"factor": 4.0, "fast": 8.0, "original": 128, "slow": 0.5}}
    ssm = {"conv": 4, "groups": 1, "heads": 3, "norm_groups": 3, "state": 20, "vdim": 8}
    att = {"conv": 2, "dim": 12, "heads": 6, "kv_heads": 3, "scale": 0.3, "vdim": 10}
    lat = {"dim": 16, "heads": 2, "kv_rank": 24, "q_rank": 20, "rot": rot, "rot_dim": 8, "scale": 0.2, "vdim": 12}
    moe = {"expert": {"ff": 14}, "kind": "moe", "router": {"experts": 12, "groups": {"count": 4, "keep": 2}, "top": 3}}
    moe2 = {"expert": {"ff": 9}, "kind": "moe", "router": {"experts": 5, "top": 1}}
    return {"architecture": "Sabolorn", "embedding": {"scale": 0.25}, "logit_softcap": 9.0, "norm": {"eps": 1e-6}, "token_side": {"dim": 6},
            "vocab": 77, "width": 40,
            "layers": [{"type": "latent_attention", "mixer": lat, "mlp": moe}, {"type": "mamba2", "mixer": ssm, "mlp": None},
                       {"type": "latent_attention", "mixer": dict(lat, kv_from=0), "mlp": {"ff": 30, "kind": "dense"}},
                       {"type": "attention", "mixer": att, "mlp": moe2}]}


def test_spec_reads_every_size_from_config_and_shapes(lib):
    from candle_vllm_amd import hybrid_model as hm
    cfg = _cfg()
    W = S.random_sabolorn(np.random.default_rng(0), cfg)
    del W["l3.mlp.correction"]
    spec = hm.SabolornSpec(cfg, {k: v.shape for k, v in W.items()})
    a, b, c, d = spec.layers
    assert (spec.residual_form, spec.norm_kind, spec.tie_head, spec.side_cols, spec.side_dim) == (3, hm.NORM_LAYER, 1, 24, 6)
    assert abs(spec.embed_scale - 0.25) < 1e-9 and abs(spec.logit_softcap - 9.0) < 1e-9 and abs(spec.eps - 1e-6) < 1e-12
    assert (a.mixer, a.a_heads, a.a_dim, a.a_vdim, a.a_kv_rank, a.a_rot_dim, a.a_rot_dims, a.a_rot_interleaved, a.a_q_rank, a.a_out_gate, a.a_head_gate,
            a.kv_from) == (hm.MIX_LATENT, 2, 16, 12, 24, 8, 8, 1, 20, 1, 0, 0)
    assert (a.mlp_kind, a.mlp_ff, a.moe_experts, a.moe_top, a.moe_sigmoid, a.moe_normalise, a.moe_groups, a.moe_keep_groups) == (hm.MLP_MOE, 14, 12, 3, 1, 1, 4, 2)
    assert (b.mixer, b.d_heads, b.d_vdim, b.d_dim, b.d_kv_heads, b.d_conv, b.d_norm_groups, b.mlp_kind) == (hm.MIX_SSD, 3, 8, 20, 1, 4, 3, 0)
    assert (c.kv_from, c.mlp_kind, c.mlp_ff) == (1, hm.MLP_RELU2, 30)
    assert (d.mixer, d.a_heads, d.a_kv_heads, d.a_dim, d.a_vdim, d.a_conv, d.a_dist_bias, d.a_qk_norm, d.a_v_unit) == (hm.MIX_CONV_ATTENTION, 6, 3, 12, 10, 2, 1, 0, 0)
    assert (d.moe_groups, d.moe_experts, d.moe_top) == (0, 5, 1)
    assert [L.side_col for L in spec.layers] == [0, 6, 12, 18] and [L.depth_terms for L in spec.layers] == [2, 3, 4, 5]
    offs = (ctypes.c_int32 * 9)()
    assert lib.mi355_hybrid_in_proj_rows(ctypes.byref(a), offs) == 20 + 32 + 24 and (offs[0], offs[1], offs[8]) == (0, 20, 52)
    assert lib.mi355_hybrid_in_proj_rows(ctypes.byref(c), offs) == 20 + 24 and (offs[0], offs[1], offs[8]) == (0, -1, 20)
    assert lib.mi355_hybrid_in_proj_rows(ctypes.byref(b), offs) == 2 * 24 + 2 * 20 + 3 and (offs[8], offs[5], offs[4], offs[3], offs[7]) == (0, 24, 48, 68, 88)
    assert lib.mi355_hybrid_in_proj_rows(ctypes.byref(d), offs) == 72 + 36 + 30 and list(offs)[:3] == [0, 72, 108]
    s0, s1, s2, s3 = spec.slots
    assert s0[hm.HW_IN_PROJ] == ["l0.mix.dq", "l0.mix.dkv", "l0.mix.g"] and s2[hm.HW_IN_PROJ] == ["l2.mix.dq", "l2.mix.g"]
    assert hm.HW_L_CNORM in s0 and hm.HW_L_CNORM not in s2 and s2[hm.HW_L_UQ] == ["l2.mix.uq"]
    assert s1[hm.HW_CONV_BIAS] == ["l1.mix.conv.b"] and s1[hm.HW_D_SKIP] == ["l1.mix.D"] and hm.HW_MLP_GATE_UP not in s1
    assert s3[hm.HW_IN_BIAS] == ["l3.mix.q.b", "l3.mix.k.b", "l3.mix.v.b"] and s3[hm.HW_A_DIST] == ["l3.mix.r1", "l3.mix.r2"]
    assert hm.HW_MOE_CORRECTION in s0 and hm.HW_MOE_CORRECTION not in s3
    assert s2[hm.HW_MLP_GATE_UP] == ["l2.mlp.up"] and s2[hm.HW_DEPTH_W] == ["l2.dwa"] and s2[hm.HW_SIDE_GATE] == ["l2.side.gate"]
    used = {n if isinstance(n, str) else n.name for sl in spec.slots for names in sl.values() for n in names} | set(spec.globals_().values())
    assert used == set(W)                                                    # every tensor of the checkpoint has a slot
    with pytest.raises(ValueError):
        hm.SabolornSpec({**cfg, "layers": [{"type": "delta", "mixer": {}, "mlp": None}]}, {k: v.shape for k, v in W.items()})
    with pytest.raises(ValueError):
        hm.SabolornSpec({**cfg, "layers": [dict(cfg["layers"][1], mlp={"kind": "glu", "ff": 8})]}, {k: v.shape for k, v in W.items()})


def test_registry_serves_the_design():
    from candle_vllm_amd import registry
    assert "Sabolorn" in registry.registered()
    assert registry.component_of({"architecture": "Sabolorn"}) == "hybrid"


@pytest.mark.parametrize("rot", [{"base": 10000.0, "dims": 32, "scaling": {"factor": 2.0, "fast": 32.0, "original": 2048, "slow": 1.0}},
                                 {"base": 500000.0, "dims": 64, "scaling": {"factor": 40.0, "fast": 16.0, "original": 4096, "slow": 2.0}},
                                 {"base": 1000.0, "dims": 6, "scaling": {"factor": 3.5, "fast": 8.0, "original": 64, "slow": 0.5}},
                                 {"base": 123456.0, "dims": 16, "scaling": {"factor": 1.0, "fast": 32.0, "original": 256, "slow": 1.0}},
                                 {"base": 100.0, "dims": 2, "scaling": {"factor": 8.0, "fast": 4.0, "original": 16, "slow": 1.0}},
                                 {"base": 7000.0, "dims": 24}])
def test_rotation_tables_follow_the_oracles_angles(lib, rot):
    """the framework's table builder with the design's scaling: blended frequencies, amplitude 0.1 ln(factor) + 1 on cos and sin"""
    from candle_vllm_amd.hybrid_model import SabolornSpec
    n, dims = 700, rot["dims"]
    rs = SabolornSpec.rope_scaling(rot)
    cos, sin = np.zeros((n, dims // 2), np.float32), np.zeros((n, dims // 2), np.float32)
    assert lib.mi355_rope_tables_f64(cos.ctypes.data, sin.ctypes.data, dims, n, float(rot["base"]), ctypes.byref(rs), n, n) == 0
    ang, amp = S.yarn_angles(rot, n)
    assert np.abs(cos - np.cos(ang) * amp).max() < 2e-6 and np.abs(sin - np.sin(ang) * amp).max() < 2e-6


def test_scan_in_portions_equals_the_whole_and_one_step_by_hand():
    rng = np.random.default_rng(1)
    T, heads, vd, G, N = 13, 4, 5, 2, 7
    x, B, C = rng.standard_normal((T, heads, vd)), rng.standard_normal((T, G, N)), rng.standard_normal((T, G, N))
    dt, a_log, dtb, skip = rng.standard_normal((T, heads)), rng.standard_normal(heads), rng.standard_normal(heads), rng.standard_normal(heads)
    y, Sf = S.state_space_scan(x, B, C, dt, a_log, dtb, skip)
    st, parts = None, []
    for lo, hi in ((0, 1), (1, 3), (3, 4), (4, 13)):
        yp, st = S.state_space_scan(x[lo:hi], B[lo:hi], C[lo:hi], dt[lo:hi], a_log, dtb, skip, st)
        parts.append(yp)
    assert np.abs(np.concatenate(parts) - y).max() < 1e-12 and np.abs(st - Sf).max() < 1e-12
    step = math.log1p(math.exp(dt[0, 3] + dtb[3]))                          # the first token: S = dt B x^T, head 3 reads group 1
    assert np.allclose(y[0, 3], step * (B[0, 1] @ C[0, 1]) * x[0, 3] + skip[3] * x[0, 3])


def test_choice_among_the_best_groups_by_hand():
    z = np.log(np.array([[0.9, 0.1, 0.2, 0.3, 0.6, 0.55, 0.5, 0.05]]) / (1 - np.array([[0.9, 0.1, 0.2, 0.3, 0.6, 0.55, 0.5, 0.05]])))
    ids, w = S.route(z, None, 2)                                            # no groups: the two largest scores
    assert ids.tolist() == [[0, 4]] and np.allclose(w, [[0.9 / 1.5, 0.6 / 1.5]])
    ids, w = S.route(z, None, 2, (2, 1))                                    # group sums 0.9 + 0.3 = 1.2 against 0.6 + 0.55 = 1.15
    assert ids.tolist() == [[0, 3]] and np.allclose(w, [[0.9 / 1.2, 0.3 / 1.2]])
    ids, w = S.route(z, None, 2, (4, 1))                                    # pairs: 1.0, 0.5, 1.15, 0.55
    assert ids.tolist() == [[4, 5]]
    corr = np.array([-2.0, 0, 0, 0, 0, 0, 0, 0.0])                          # the correction decides the choice, not the weights; it may be negative
    ids, w = S.route(z, corr, 2, (2, 1))
    assert ids.tolist() == [[4, 5]] and np.allclose(w, [[0.6 / 1.15, 0.55 / 1.15]])
    ids, _ = S.route(z, np.array([-2.0, -3, -3, -3, -5, -5, -5, -5.0]), 2, (2, 1))      # negative choice scores: a closed group counts as minus infinity, not 0
    assert ids.tolist() == [[0, 3]]


def test_distance_bias_convolution_and_layer_norm_by_hand():
    q, k, v = np.ones((3, 1, 2)), np.ones((3, 1, 2)), np.array([[[1.0]], [[2.0]], [[4.0]]])
    out = S.distance_bias_attention(q, k, v, 0.5, np.array([2.0]), np.array([1.0]))
    w = np.array([1 / 9.0, 1 / 4.0, 1.0])                                   # exp(-2 ln(1 + distance)) = (1 + distance)^-2 at distances 2, 1, 0
    assert np.allclose(out[2, 0, 0], (w * [1, 2, 4]).sum() / w.sum()) and np.allclose(out[0, 0, 0], 1.0)
    u, cw = np.arange(1.0, 5.0)[:, None], np.array([[10.0, 1.0, 0.1]])
    assert np.allclose(S.causal_conv(u, cw, np.array([0.5]))[:, 0], [0.1 + 0.5, 0.2 + 1 + 0.5, 0.3 + 2 + 10 + 0.5, 0.4 + 3 + 20 + 0.5])
    x = np.array([[1.0, 2.0, 3.0, 6.0]])
    assert np.allclose(S.layer_norm(x, np.ones(4), 0.0), (x - 3.0) / math.sqrt(3.5))


def test_host_layer_refuses_what_it_does_not_serve(lib):
    """create() checks what needs no device: a borrowed page row of another size, groups that do not divide the experts, a state-space
    norm whose parts do not divide the inner width"""
    from candle_vllm_amd import hybrid_model as hm
    from candle_vllm_amd._lib import HybridConfig, HybridLayer
    cfg = _cfg()
    W = S.random_sabolorn(np.random.default_rng(0), cfg)

    def create(mutate):
        spec = hm.SabolornSpec(cfg, {k: v.shape for k, v in W.items()})
        mutate(spec.layers)
        arr = (HybridLayer * 4)(*spec.layers)
        c = HybridConfig(width=40, vocab=77, n_layers=4, dtype=0, block_size=16, state_slots=2, norm_eps=1e-6, unit_eps=1e-6, residual_form=3,
                         resid_alpha=1.0, norm_groups=1, logit_scale=1.0, norm_kind=1, embed_scale=0.25, logit_softcap=9.0, tie_head=1, side_cols=24)
        return lib.mi355_hybrid_create(ctypes.byref(c), arr)

    def set_(i, **kw):
        def f(layers):
            for k, v in kw.items():
                setattr(layers[i], k, v)
        return f
    h = create(lambda layers: None)
    assert h
    lib.mi355_hybrid_destroy(h)
    assert not create(set_(2, a_kv_rank=32))
    assert not create(set_(2, kv_from=3))
    assert not create(set_(0, moe_groups=5))
    assert not create(set_(0, moe_keep_groups=1, moe_top=4))               # three experts of one group cannot give four
    assert not create(set_(1, d_norm_groups=5))
    assert not create(set_(3, side_col=20))
    assert not create(set_(1, depth_terms=2))
