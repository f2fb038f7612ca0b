"""Python harness over the `mi355_hybrid_*` handle (include/mi355_hybrid.h): layer-list models whose layers mix tokens by
sliding-window attention with a sink, a gated delta rule, a minGRU, attention and delta rule side by side, latent attention, or
attention behind a short convolution with mixed head weights, or a state-space mixer, with dense or mixture-of-experts
feed-forwards.  The Sogodra, Vivazen, Kerolorn and Sabolorn designs are read here: a design's
config.json (`architecture`, `layers`, `norm`, `vocab`, `width`, ...) becomes the C structs, its tensors are concatenated into the
host layer's slots.  No CPU fallback; torch only holds device buffers."""
import ctypes
import json
import math
import os
import struct

import numpy as np
import torch

from ._lib import lib, HybridConfig, HybridLayer, RopeScaling

DT_F32, DT_BF16 = 0, 2
MIX_PARALLEL, MIX_MINGRU, MIX_DELTA, MIX_ATTENTION, MIX_LATENT, MIX_CONV_ATTENTION, MIX_SSD = 0, 1, 2, 3, 4, 5, 6
GATE_SILU, GATE_SIGMOID_LR = 0, 1
ROPE_DEFAULT, ROPE_LLAMA3, ROPE_YARN = 0, 2, 4
(HW_EMBED, HW_FINAL_NORM, HW_HEAD, HW_NORM1, HW_NORM2, HW_IN_PROJ, HW_IN_BIAS, HW_OUT_PROJ, HW_A_QNORM, HW_A_KNORM, HW_A_SINK, HW_D_CONV,
 HW_D_A_LOG, HW_D_DT_BIAS, HW_D_NORM, HW_D_A2, HW_D_G2, HW_MLP_GATE_UP, HW_MLP_DOWN, HW_A_CONV, HW_A_TALK, HW_L_UKT, HW_L_UV,
 HW_L_CNORM, HW_PRE_NORM1, HW_PRE_NORM2, HW_IN_CONV, HW_A_TEMP, HW_MOE_ROUTER, HW_MOE_CORRECTION, HW_MOE_GATE_UP,
 HW_MOE_DOWN, HW_D_SKIP, HW_CONV_BIAS, HW_A_DIST, HW_L_QNORM, HW_L_UQ, HW_SIDE_GATE, HW_SIDE_PROJ, HW_SIDE_NORM, HW_DEPTH_W,
 HW_SIDE_TABLE) = range(42)
MLP_CLAMPED_GLU, MLP_GELU_GLU, MLP_MOE, MLP_RELU2 = 1, 2, 3, 4
NORM_RMS, NORM_LAYER = 0, 1

# constants the Sogodra design fixes
SOGODRA_GLU_ALPHA = 1.702          # y = g sigmoid(1.702 g) (u + 1)
SOGODRA_UNIT_EPS = 1e-6            # inside the root of the unit norm of the delta rule's q and k
DEFAULT_BLOCK_SIZE = 64


def _check(rc, what):
    if rc != 0:
        raise RuntimeError(f"{what} failed with code {rc}")


def read_safetensors(path):
    """name -> (bf16 bits as uint16 ndarray | int32 ndarray, shape).  The format: 8-byte little-endian header length, that many
    bytes of JSON (name -> dtype, shape, data_offsets), then the data.  bf16 / f32 tensors come back as bf16 bits (f32 values must
    be exactly representable), integer tables as int32."""
    with open(path, "rb") as f:
        n = struct.unpack("<Q", f.read(8))[0]
        meta = json.loads(f.read(n))
        base = 8 + n
        out = {}
        for name, info in meta.items():
            if name == "__metadata__":
                continue
            lo, hi = info["data_offsets"]
            f.seek(base + lo)
            raw = f.read(hi - lo)
            shape = tuple(info["shape"])
            if info["dtype"] == "BF16":
                a = np.frombuffer(raw, np.uint16).copy()
            elif info["dtype"] == "F32":
                u = np.frombuffer(raw, np.uint32)
                if np.any(u & 0xFFFF):
                    raise ValueError(f"{name}: f32 values that bf16 cannot hold")
                a = (u >> 16).astype(np.uint16)
            elif info["dtype"] == "I32":
                a = np.frombuffer(raw, np.int32).copy()
            else:
                raise ValueError(f"{name}: dtype {info['dtype']} is not served")
            if a.size != int(np.prod(shape, dtype=np.int64)):
                raise ValueError(f"{name}: {a.size} elements for shape {shape}")
            out[name] = (a, shape)
    return out


def _bf16_bits(a):
    u = np.ascontiguousarray(a, np.float32).view(np.uint32)
    return ((u + 0x7FFF + ((u >> 16) & 1)) >> 16).astype(np.uint16)


class HeadTranspose:
    """a slot entry: tensor `name` [heads * a, b] stored as [heads, b, a] (every head's block transposed)"""

    def __init__(self, name, heads):
        self.name, self.heads = name, int(heads)

    def bits(self, bits, shapes):
        rows, cols = shapes[self.name]
        a = np.asarray(bits[self.name], np.uint16).reshape(self.heads, rows // self.heads, cols)
        return np.ascontiguousarray(a.transpose(0, 2, 1)).reshape(-1)


def yarn_scaling(rot):
    """`rot.scaling` = {factor, original, fast, slow} -> the table builder's yarn form: the frequency blend between the indices where a
    wavelength makes `fast` / `slow` turns over `original` positions, amplitude 0.1 ln(factor) + 1 on cos and sin for EVERY factor (the
    table builder keeps amplitude 1 up to factor 1, so there it is passed as the attention factor)"""
    rs = RopeScaling()
    sc = rot.get("scaling")
    if sc:
        rs.type, rs.factor, rs.original_max_position_embeddings = ROPE_YARN, float(sc["factor"]), float(sc["original"])
        rs.beta_fast, rs.beta_slow, rs.attn_factor = float(sc["fast"]), float(sc["slow"]), 1.0
        if rs.factor <= 1.0:
            rs.attn_factor = 0.1 * math.log(rs.factor) + 1.0
    else:
        rs.type = ROPE_DEFAULT
    return rs


class SogodraSpec:
    """config.json of a Sogodra model -> layer structs + the tensor names behind every weight slot"""
    residual_form, resid_alpha, norm_groups = 0, 1.0, 1          # x <- x + norm(sub(x)), one RMS over the whole vector

    @staticmethod
    def rope_scaling(rot):
        rs = RopeScaling()
        sc = rot.get("scaling")
        if sc:
            rs.type, rs.factor, rs.low_freq_factor, rs.high_freq_factor = ROPE_LLAMA3, float(sc["factor"]), float(sc["low"]), float(sc["high"])
            rs.original_max_position_embeddings = float(sc["original"])
        else:
            rs.type = ROPE_DEFAULT
        return rs

    def __init__(self, cfg, shapes):
        """cfg: the parsed config.json; shapes: tensor name -> shape (which optional tensors exist, ranks of low-rank parts)"""
        if cfg.get("architecture") != "Sogodra":
            raise ValueError("not a Sogodra config")
        self.cfg = cfg
        self.width, self.vocab = int(cfg["width"]), int(cfg["vocab"])
        self.eps = float(cfg["norm"]["eps"])
        self.layers, self.slots, self.rope = [], [], []
        for i, lc in enumerate(cfg["layers"]):
            L, slots, rope = self._layer("l%d." % i, lc, shapes)
            self.layers.append(L)
            self.slots.append(slots)
            self.rope.append(rope)

    def _attention(self, L, p, c, shapes, slots):
        L.a_heads, L.a_kv_heads, L.a_dim, L.a_vdim = int(c["heads"]), int(c["kv_heads"]), int(c["dim"]), int(c["vdim"])
        L.a_window = int(c["mask"]["size"]) if c.get("mask") else 0
        rot = c.get("rot")
        L.a_rot_dims = int(rot["dims"]) if rot else 0
        L.a_scale = float(c["scale"])
        L.a_has_sink = int(p + "sink" in shapes)
        L.a_qk_norm = int(p + "q.norm" in shapes)
        if L.a_qk_norm:
            slots[HW_A_QNORM], slots[HW_A_KNORM] = [p + "q.norm"], [p + "k.norm"]
        if L.a_has_sink:
            slots[HW_A_SINK] = [p + "sink"]
        return [p + "q", p + "k", p + "v"], [p + "o"], rot

    def _delta(self, L, p, c, shapes, slots, per_channel, gate):
        L.d_heads, L.d_kv_heads, L.d_dim, L.d_vdim, L.d_conv = (int(c["heads"]), int(c["kv_heads"]), int(c["dim"]), int(c["vdim"]),
                                                                int(c["conv"]))
        L.d_decay_channels, L.d_gate = int(per_channel), gate
        a_name, g_name = ("a1" if per_channel else "a"), ("g1" if gate == GATE_SIGMOID_LR else "g")
        if per_channel:
            L.d_a_rank = int(shapes[p + "a1"][0])
            slots[HW_D_A2] = [p + "a2"]
        if gate == GATE_SIGMOID_LR:
            L.d_g_rank = int(shapes[p + "g1"][0])
            slots[HW_D_G2] = [p + "g2"]
        slots[HW_D_CONV] = [p + "q.conv", p + "k.conv", p + "v.conv"]
        slots[HW_D_A_LOG], slots[HW_D_DT_BIAS], slots[HW_D_NORM] = [p + "A_log"], [p + "dt_bias"], [p + "norm"]
        return [p + "q", p + "k", p + "v", p + "b", p + a_name, p + g_name], [p + "o"]

    def _layer(self, p, lc, shapes):
        L, slots, rope = HybridLayer(), {HW_NORM1: [p + "norm1"]}, None
        m, kind = lc["mixer"], lc["type"]
        if kind == "parallel":
            L.mixer = MIX_PARALLEL
            ins, outs, rope = self._attention(L, p + "mix.left.", m["left"], shapes, slots)
            i2, o2 = self._delta(L, p + "mix.right.", m["right"], shapes, slots, True, GATE_SIGMOID_LR)
            ins, outs = ins + i2, outs + o2
            L.a_out_scale, L.d_out_scale = float(m["left_scale"]), float(m["right_scale"])
        elif kind == "delta":
            L.mixer = MIX_DELTA
            ins, outs = self._delta(L, p + "mix.", m, shapes, slots, False, GATE_SILU)
            L.d_out_scale = 1.0
        elif kind == "mingru":
            L.mixer = MIX_MINGRU
            L.g_width = int(m["width"])
            ins, outs = [p + "mix.z", p + "mix.x", p + "mix.g"], [p + "mix.o"]
            slots[HW_IN_BIAS] = [p + "mix.z.b", p + "mix.x.b", None]
        else:
            raise ValueError(f"layer type {kind!r} is not part of the design")
        slots[HW_IN_PROJ], slots[HW_OUT_PROJ] = ins, outs
        mlp = lc.get("mlp")
        if mlp:
            if mlp.get("kind") != "dense":
                raise ValueError(f"feed-forward kind {mlp.get('kind')!r} is not part of the design")
            L.mlp_kind, L.mlp_ff, L.mlp_limit, L.mlp_alpha = 1, int(mlp["ff"]), float(mlp["limit"]), SOGODRA_GLU_ALPHA
            slots[HW_NORM2] = [p + "norm2"]
            slots[HW_MLP_GATE_UP], slots[HW_MLP_DOWN] = [p + "mlp.gate", p + "mlp.up"], [p + "mlp.down"]
        return L, slots, rope


class VivazenSpec:
    """config.json of a Vivazen model -> layer structs + the tensor names behind every weight slot.  The design: the norm sits behind
    the residual sum, x <- N(alpha x + sub(x)), N = RMS norm over `norm.groups` parts of the vector; layers are latent attention
    (window, sink, head gate, interleaved rotation with yarn scaling on the rotated part) or attention behind a convolution (norms
    over the whole q / k projections, unit values, capped scores, mixed head weights); gelu-tanh gate/up feed-forward; a layer with
    `weights_of` runs on that layer's tensors with a cache of its own."""
    residual_form = 1

    rope_scaling = staticmethod(yarn_scaling)

    def __init__(self, cfg, shapes):
        if cfg.get("architecture") != "Vivazen":
            raise ValueError("not a Vivazen config")
        self.cfg = cfg
        self.width, self.vocab = int(cfg["width"]), int(cfg["vocab"])
        self.eps, self.norm_groups = float(cfg["norm"]["eps"]), int(cfg["norm"].get("groups", 1))
        self.resid_alpha = float(cfg.get("postln_alpha", 1.0))
        self.layers, self.slots, self.rope = [], [], []
        entries = cfg["layers"]
        for i, lc in enumerate(entries):
            src = i
            while "weights_of" in entries[src]:                 # the layer whose tensors this one runs on
                src = int(entries[src]["weights_of"])
                if src == i:
                    raise ValueError(f"layer {i}: weights_of runs in a circle")
            L, slots, rope = self._layer("l%d." % src, lc, shapes)
            if src != i:
                L.share_with, slots, rope = src + 1, {}, None
            self.layers.append(L)
            self.slots.append(slots)
            self.rope.append(rope)

    def _layer(self, p, lc, shapes):
        L, slots, rope = HybridLayer(), {HW_NORM1: [p + "norm1"]}, None
        c, kind, q = lc["mixer"], lc["type"], p + "mix."
        L.a_heads, L.a_dim, L.a_vdim, L.a_scale, L.a_out_scale = int(c["heads"]), int(c["dim"]), int(c["vdim"]), float(c["scale"]), 1.0
        L.a_window = int(c["mask"]["size"]) if c.get("mask") else 0
        L.a_softcap = float(c.get("softcap") or 0.0)
        L.a_has_sink = int(q + "sink" in shapes)
        if L.a_has_sink:
            slots[HW_A_SINK] = [q + "sink"]
        if kind == "latent_attention":
            L.mixer = MIX_LATENT
            L.a_kv_heads, L.a_kv_rank, L.a_rot_dim = 1, int(c["kv_rank"]), int(c["rot_dim"])
            rope = c.get("rot")
            L.a_rot_dims, L.a_rot_interleaved = (int(rope["dims"]) if rope else 0), 1
            L.a_head_gate = int(q + "g" in shapes)
            slots[HW_IN_PROJ] = [q + "q", q + "dkv"] + ([q + "g"] if L.a_head_gate else [])
            slots[HW_L_UKT], slots[HW_L_UV], slots[HW_L_CNORM] = [HeadTranspose(q + "uk", L.a_heads)], [q + "uv"], [q + "dkv.norm"]
        elif kind == "attention":
            L.mixer = MIX_CONV_ATTENTION
            L.a_kv_heads, L.a_conv = int(c["kv_heads"]), int(c.get("conv") or 1)
            L.a_qk_norm = L.a_norm_whole = int(q + "q.norm" in shapes)
            L.a_v_unit, L.a_talk = 1, int(q + "talk" in shapes)
            slots[HW_IN_PROJ] = [q + "q", q + "k", q + "v"]
            if L.a_qk_norm:
                slots[HW_A_QNORM], slots[HW_A_KNORM] = [q + "q.norm"], [q + "k.norm"]
            if L.a_conv > 1 or q + "q.conv" in shapes:
                slots[HW_A_CONV] = [q + "q.conv", q + "k.conv", q + "v.conv"]
            if L.a_talk:
                slots[HW_A_TALK] = [q + "talk"]
        else:
            raise ValueError(f"layer type {kind!r} is not part of the design")
        slots[HW_OUT_PROJ] = [q + "o"]
        mlp = lc.get("mlp")
        if mlp:
            if mlp.get("kind") != "dense":
                raise ValueError(f"feed-forward kind {mlp.get('kind')!r} is not part of the design")
            L.mlp_kind, L.mlp_ff = MLP_GELU_GLU, int(mlp["ff"])
            slots[HW_NORM2] = [p + "norm2"]
            slots[HW_MLP_GATE_UP], slots[HW_MLP_DOWN] = [p + "mlp.gate", p + "mlp.up"], [p + "mlp.down"]
        return L, slots, rope


class KerolornSpec:
    """config.json of a Kerolorn model -> layer structs + the tensor names behind every weight slot.  The design: a norm on both sides
    of every sublayer, x <- x + Nb(sub(Na(x))); the mixer's input h becomes h + conv(h) (`canon1`, a causal convolution over time per
    channel of the width); grouped-query attention with interleaved rotary pairs (yarn), a weightless RMS norm of q and k behind the
    rotation, a temperature per head, a sliding window that keeps the first tokens; mixture-of-experts feed-forward (softmax router,
    selection-only correction, scaled weights, shared expert behind a sigmoid gate); logits times `logit_scale`."""
    residual_form, resid_alpha, norm_groups = 2, 1.0, 1
    rope_scaling = staticmethod(yarn_scaling)

    def __init__(self, cfg, shapes):
        if cfg.get("architecture") != "Kerolorn":
            raise ValueError("not a Kerolorn config")
        self.cfg = cfg
        self.width, self.vocab = int(cfg["width"]), int(cfg["vocab"])
        self.eps = float(cfg["norm"]["eps"])
        self.logit_scale = float(cfg.get("logit_scale", 1.0))
        self.taps = int((cfg.get("canon") or {}).get("taps", 0))
        self.layers, self.slots, self.rope = [], [], []
        for i, lc in enumerate(cfg["layers"]):
            L, slots, rope = self._layer("l%d." % i, lc, shapes)
            self.layers.append(L)
            self.slots.append(slots)
            self.rope.append(rope)

    def _layer(self, p, lc, shapes):
        if lc["type"] != "attention":
            raise ValueError(f"layer type {lc['type']!r} is not part of the design")
        L, c, q = HybridLayer(), lc["mixer"], p + "mix."
        slots = {HW_PRE_NORM1: [p + "norm1"], HW_NORM1: [p + "norm1b"]}
        L.mixer = MIX_ATTENTION
        L.a_heads, L.a_kv_heads, L.a_dim, L.a_vdim = int(c["heads"]), int(c["kv_heads"]), int(c["dim"]), int(c["vdim"])
        L.a_scale, L.a_out_scale = float(c["scale"]), 1.0
        mask = c.get("mask") or {}
        L.a_window, L.a_keep_first = int(mask.get("size") or 0), int(mask.get("keep_first") or 0)
        rope = c.get("rot")
        L.a_rot_dims, L.a_rot_interleaved = (int(rope["dims"]) if rope else 0), 1
        if L.a_rot_dims <= 0:
            rope = None
        L.a_qk_norm, L.a_norm_after_rot = 1, 1
        L.a_head_temp = int(q + "temp" in shapes)
        if L.a_head_temp:
            slots[HW_A_TEMP] = [q + "temp"]
        if p + "canon1" in shapes:
            L.in_conv = int(shapes[p + "canon1"][1])
            if self.taps and L.in_conv != self.taps:
                raise ValueError(f"{p}canon1 has {L.in_conv} taps, the config says {self.taps}")
            slots[HW_IN_CONV] = [p + "canon1"]
        slots[HW_IN_PROJ], slots[HW_OUT_PROJ] = [q + "q", q + "k", q + "v"], [q + "o"]
        mlp = lc.get("mlp")
        if mlp:
            if mlp.get("kind", "moe") != "moe":
                raise ValueError(f"feed-forward kind {mlp.get('kind')!r} is not part of the design")
            m, r = p + "mlp.", mlp["router"]
            L.mlp_kind, L.mlp_ff = MLP_MOE, int(mlp["expert"]["ff"])
            L.moe_experts, L.moe_top, L.moe_scale = int(r["experts"]), int(r["top"]), float(r.get("scale", 1.0))
            shared = mlp.get("shared")
            L.moe_shared_ff = int(shared["ff"]) if shared else 0
            slots[HW_PRE_NORM2], slots[HW_NORM2] = [p + "norm2"], [p + "norm2b"]
            slots[HW_MOE_ROUTER] = [m + "router"] + ([m + "shared.sg"] if shared else [])
            if m + "correction" in shapes:
                slots[HW_MOE_CORRECTION] = [m + "correction"]
            slots[HW_MOE_GATE_UP] = [m + "e%d.%s" % (e, n) for e in range(L.moe_experts) for n in ("gate", "up")]
            slots[HW_MOE_DOWN] = [m + "e%d.down" % e for e in range(L.moe_experts)]
            if shared and L.moe_shared_ff == L.mlp_ff:      # of the experts' size: one more matrix of the grouped products
                slots[HW_MOE_GATE_UP] += [m + "shared.gate", m + "shared.up"]
                slots[HW_MOE_DOWN] += [m + "shared.down"]
            elif shared:
                slots[HW_MLP_GATE_UP], slots[HW_MLP_DOWN] = [m + "shared.gate", m + "shared.up"], [m + "shared.down"]
        return L, slots, rope


class Ones:
    """a slot entry: n ones (a convolution of one tap that the checkpoint leaves out)"""

    def __init__(self, n):
        self.n = int(n)

    def bits(self, bits, shapes):
        return np.full(self.n, 0x3F80, np.uint16)


class SabolornSpec:
    """config.json of a Sabolorn model -> layer structs + the tensor names behind every weight slot.  The design: ONE layer norm
    (weight, no bias) per layer and both sublayers read it, x <- x + mixer(h) + ff(h); then the token's own input to the layer (a
    slice of a second embedding table behind a gelu gate, RMS-normed), then a learned average over the embedding output and the
    results of all layers so far.  Mixers: a state-space mixer with a scalar decay per head (`mamba2`), attention with biases, a short
    convolution behind q / k / v and a logarithmic distance bias instead of a rotation (`attention`), latent attention with queries
    through a latent of their own, yarn-scaled interleaved rotation and an elementwise output gate, optionally on the cached rows of
    an earlier layer (`latent_attention`, `kv_from`).  Feed-forward: relu-squared dense or a mixture of experts with sigmoid scores,
    group-limited choice and normalised weights.  Scaled embedding, tied output table, tanh-capped logits."""
    residual_form, resid_alpha, norm_groups, norm_kind, tie_head = 3, 1.0, 1, NORM_LAYER, 1
    rope_scaling = staticmethod(yarn_scaling)

    def __init__(self, cfg, shapes):
        if cfg.get("architecture") != "Sabolorn":
            raise ValueError("not a Sabolorn config")
        self.cfg = cfg
        self.width, self.vocab = int(cfg["width"]), int(cfg["vocab"])
        self.eps = float(cfg["norm"]["eps"])
        self.embed_scale = float((cfg.get("embedding") or {}).get("scale", 1.0))
        self.logit_softcap = float(cfg.get("logit_softcap") or 0.0)
        side = cfg.get("token_side")
        self.side_dim = int(side["dim"]) if side else 0
        self.side_cols = int(shapes["side.embed"][1]) if side else 0
        self.layers, self.slots, self.rope = [], [], []
        for i, lc in enumerate(cfg["layers"]):
            L, slots, rope = self._layer(i, "l%d." % i, lc, shapes)
            self.layers.append(L)
            self.slots.append(slots)
            self.rope.append(rope)

    def globals_(self):
        """the tensors outside the layers: slot -> name"""
        g = {HW_EMBED: "embed", HW_FINAL_NORM: "final.norm"}
        if self.side_cols:
            g[HW_SIDE_TABLE] = "side.embed"
        return g

    def _layer(self, i, p, lc, shapes):
        L, slots, rope = HybridLayer(), {HW_NORM1: [p + "norm1"]}, None
        c, kind, q = lc["mixer"], lc["type"], p + "mix."
        if kind == "mamba2":
            L.mixer = MIX_SSD
            L.d_heads, L.d_vdim, L.d_dim, L.d_kv_heads = int(c["heads"]), int(c["vdim"]), int(c["state"]), int(c["groups"])
            L.d_conv, L.d_norm_groups = int(c["conv"]), int(c.get("norm_groups", 1))
            slots[HW_IN_PROJ], slots[HW_OUT_PROJ] = [q + "in"], [q + "o"]
            slots[HW_D_CONV], slots[HW_CONV_BIAS] = [q + "conv"], [q + "conv.b"]
            slots[HW_D_A_LOG], slots[HW_D_DT_BIAS], slots[HW_D_SKIP], slots[HW_D_NORM] = [q + "A_log"], [q + "dt_bias"], [q + "D"], [q + "norm"]
        elif kind == "attention":
            L.mixer = MIX_CONV_ATTENTION
            L.a_heads, L.a_kv_heads, L.a_dim, L.a_vdim = int(c["heads"]), int(c["kv_heads"]), int(c["dim"]), int(c["vdim"])
            L.a_scale, L.a_out_scale = float(c["scale"]), 1.0
            slots[HW_IN_PROJ] = [q + "q", q + "k", q + "v"]
            if q + "q.b" in shapes:
                slots[HW_IN_BIAS] = [q + "q.b", q + "k.b", q + "v.b"]
            if q + "q.conv" in shapes:
                L.a_conv = int(shapes[q + "q.conv"][1])
                slots[HW_A_CONV] = [q + "q.conv", q + "k.conv", q + "v.conv"]
            else:
                L.a_conv = 1
                slots[HW_A_CONV] = [Ones((L.a_heads + L.a_kv_heads) * L.a_dim + L.a_kv_heads * L.a_vdim)]
            if q + "r1" in shapes:
                L.a_dist_bias = 1
                slots[HW_A_DIST] = [q + "r1", q + "r2"]
            slots[HW_OUT_PROJ] = [q + "o"]
        elif kind == "latent_attention":
            L.mixer = MIX_LATENT
            L.a_heads, L.a_dim, L.a_vdim, L.a_scale, L.a_out_scale = int(c["heads"]), int(c["dim"]), int(c["vdim"]), float(c["scale"]), 1.0
            L.a_kv_heads, L.a_kv_rank, L.a_rot_dim = 1, int(c["kv_rank"]), int(c["rot_dim"])
            rope = c.get("rot")
            L.a_rot_dims, L.a_rot_interleaved = (int(rope["dims"]) if rope else 0), 1
            ins = []
            if q + "dq" in shapes:
                L.a_q_rank = int(shapes[q + "dq"][0])
                ins.append(q + "dq")
                slots[HW_L_QNORM], slots[HW_L_UQ] = [q + "dq.norm"], [q + "uq"]
            else:
                ins.append(q + "q")
            if c.get("kv_from") is not None:
                L.kv_from = int(c["kv_from"]) + 1
            else:
                ins.append(q + "dkv")
                slots[HW_L_CNORM] = [q + "dkv.norm"]
            if q + "g" in shapes:
                ins.append(q + "g")
                if int(shapes[q + "g"][0]) == L.a_heads * L.a_vdim:
                    L.a_out_gate = 1
                else:
                    L.a_head_gate = 1
            slots[HW_IN_PROJ], slots[HW_OUT_PROJ] = ins, [q + "o"]
            slots[HW_L_UKT], slots[HW_L_UV] = [HeadTranspose(q + "uk", L.a_heads)], [q + "uv"]
        else:
            raise ValueError(f"layer type {kind!r} is not part of the design")
        mlp = lc.get("mlp")
        if mlp:
            m = p + "mlp."
            if mlp.get("kind") == "dense":
                L.mlp_kind, L.mlp_ff = MLP_RELU2, int(mlp["ff"])
                slots[HW_MLP_GATE_UP], slots[HW_MLP_DOWN] = [m + "up"], [m + "down"]
            elif mlp.get("kind") == "moe":
                r = mlp["router"]
                L.mlp_kind, L.mlp_ff = MLP_MOE, int(mlp["expert"]["ff"])
                L.moe_experts, L.moe_top, L.moe_scale = int(r["experts"]), int(r["top"]), 1.0
                L.moe_sigmoid, L.moe_normalise = 1, 1
                gr = r.get("groups")
                if gr:
                    L.moe_groups, L.moe_keep_groups = int(gr["count"]), int(gr["keep"])
                slots[HW_MOE_ROUTER] = [m + "router"]
                if m + "correction" in shapes:
                    slots[HW_MOE_CORRECTION] = [m + "correction"]
                slots[HW_MOE_GATE_UP] = [m + "e%d.%s" % (e, n) for e in range(L.moe_experts) for n in ("gate", "up")]
                slots[HW_MOE_DOWN] = [m + "e%d.down" % e for e in range(L.moe_experts)]
            else:
                raise ValueError(f"feed-forward kind {mlp.get('kind')!r} is not part of the design")
        if self.side_dim:
            L.side_dim, L.side_col = self.side_dim, i * self.side_dim
            slots[HW_SIDE_GATE], slots[HW_SIDE_PROJ], slots[HW_SIDE_NORM] = [p + "side.gate"], [p + "side.proj"], [p + "side.norm"]
        if p + "dwa" in shapes:
            L.depth_terms = int(shapes[p + "dwa"][0])
            slots[HW_DEPTH_W] = [p + "dwa"]
        return L, slots, rope


SPECS = {"Sogodra": SogodraSpec, "Vivazen": VivazenSpec, "Kerolorn": KerolornSpec, "Sabolorn": SabolornSpec}       # config.json `architecture` -> its reader


class HybridModel:
    stateful = True                       # its layers carry state from token to token: a sequence needs a state slot

    def __init__(self, spec, dtype="bfloat16", block_size=DEFAULT_BLOCK_SIZE, state_slots=4):
        self.spec, self.block_size, self.state_slots = spec, int(block_size), int(state_slots)
        self.dtype = {"bfloat16": DT_BF16, "bf16": DT_BF16, "float32": DT_F32, "f32": DT_F32}[dtype]
        self.vocab, self.width = spec.vocab, spec.width
        n = len(spec.layers)
        self._layers = (HybridLayer * n)(*spec.layers)
        c = HybridConfig(width=spec.width, vocab=spec.vocab, n_layers=n, dtype=self.dtype, block_size=self.block_size,
                         state_slots=self.state_slots, norm_eps=spec.eps, unit_eps=SOGODRA_UNIT_EPS,
                         residual_form=int(spec.residual_form), resid_alpha=float(spec.resid_alpha), norm_groups=int(spec.norm_groups),
                         logit_scale=float(getattr(spec, "logit_scale", 1.0)), norm_kind=int(getattr(spec, "norm_kind", NORM_RMS)),
                         embed_scale=float(getattr(spec, "embed_scale", 1.0)), logit_softcap=float(getattr(spec, "logit_softcap", 0.0)),
                         tie_head=int(getattr(spec, "tie_head", 0)), side_cols=int(getattr(spec, "side_cols", 0)))
        self.h = lib.mi355_hybrid_create(ctypes.byref(c), self._layers)
        if not self.h:
            raise RuntimeError("mi355_hybrid_create refused the configuration")
        self.rope_positions = 0
        self.num_blocks = 0

    def __del__(self):
        if getattr(self, "h", None) and lib is not None:
            lib.mi355_hybrid_destroy(self.h)
            self.h = None

    # ---- weights
    @classmethod
    def from_pretrained(cls, model_dir, dtype="bfloat16", block_size=DEFAULT_BLOCK_SIZE, state_slots=4):
        cfg = json.load(open(os.path.join(model_dir, "config.json")))
        tensors = read_safetensors(os.path.join(model_dir, "model.safetensors"))
        if cfg.get("architecture") not in SPECS:
            raise ValueError(f"architecture {cfg.get('architecture')!r} is not a layer-list design (known: {sorted(SPECS)})")
        spec = SPECS[cfg["architecture"]](cfg, {k: v[1] for k, v in tensors.items()})
        m = cls(spec, dtype=dtype, block_size=block_size, state_slots=state_slots)
        m.load_tensors({k: v[0] for k, v in tensors.items()}, {k: v[1] for k, v in tensors.items()})
        return m

    def _put(self, layer, which, bits):
        bits = np.ascontiguousarray(bits, np.uint16).reshape(-1)
        _check(lib.mi355_hybrid_set_weight(self.h, layer, which, bits.ctypes.data, bits.size), f"set_weight layer {layer} slot {which}")

    def load_tensors(self, bits, shapes):
        """bits: tensor name -> bf16 bits (uint16, any shape); shapes: name -> shape.  Concatenates what the host layer keeps as one
        matrix: the input projections along the rows, the output projections along k."""
        spec = self.spec
        globals_ = spec.globals_() if hasattr(spec, "globals_") else {HW_EMBED: "embed", HW_FINAL_NORM: "final.norm", HW_HEAD: "head"}
        for which, name in globals_.items():
            self._put(-1, which, bits[name])
        for i, slots in enumerate(spec.slots):
            for which, names in slots.items():
                if which == HW_IN_BIAS:
                    offs = (ctypes.c_int32 * 9)()
                    rows = lib.mi355_hybrid_in_proj_rows(ctypes.byref(self._layers[i]), offs)
                    parts, total = [], 0
                    for nm, proj in zip(names, slots[HW_IN_PROJ]):
                        r = int(shapes[proj][0])
                        parts.append(np.asarray(bits[nm], np.uint16).reshape(-1) if nm else np.zeros(r, np.uint16))
                        total += r
                    assert total == rows
                    self._put(i, which, np.concatenate(parts))
                elif which == HW_OUT_PROJ and len(names) > 1:
                    mats = [np.asarray(bits[nm], np.uint16).reshape(shapes[nm]) for nm in names]
                    self._put(i, which, np.concatenate(mats, axis=1))
                elif which == HW_D_CONV:
                    mats = [np.asarray(bits[nm], np.uint16).reshape(shapes[nm]) for nm in names]
                    self._put(i, which, np.concatenate(mats, axis=0))
                else:
                    self._put(i, which, np.concatenate([nm.bits(bits, shapes) if isinstance(nm, (HeadTranspose, Ones))
                                                        else np.asarray(bits[nm], np.uint16).reshape(-1) for nm in names]))

    def load_state_dict_f32(self, W):
        """W: tensor name -> f32 ndarray (tests, synthetic weights); rounded to bf16"""
        self.load_tensors({k: _bf16_bits(v) for k, v in W.items()}, {k: tuple(np.shape(v)) for k, v in W.items()})

    # ---- cache
    def ensure_rope(self, n_positions):
        """cos / sin tables of every rotating layer up to n_positions (the framework's table builder in its f64 form; the scaling of
        the design when the config has `rot.scaling`)"""
        if n_positions <= self.rope_positions:
            return
        n = max(int(n_positions), 2 * self.rope_positions, 256)
        for i, (L, rot) in enumerate(zip(self.spec.layers, self.spec.rope)):
            if not rot or L.a_rot_dims <= 0:
                continue
            half = L.a_rot_dims // 2
            cos, sin = np.zeros((n, half), np.float32), np.zeros((n, half), np.float32)
            rs = self.spec.rope_scaling(rot)
            _check(lib.mi355_rope_tables_f64(cos.ctypes.data, sin.ctypes.data, L.a_rot_dims, n, float(rot["base"]), ctypes.byref(rs), n, n),
                   "rope_tables")
            _check(lib.mi355_hybrid_set_rope_tables(self.h, i, cos.ctypes.data, sin.ctypes.data, n), "set_rope_tables")
        self.rope_positions = n

    def alloc_cache(self, num_blocks):
        _check(lib.mi355_hybrid_alloc_cache(self.h, int(num_blocks)), "alloc_cache")
        self.num_blocks = int(num_blocks)
        self.ensure_rope(self.num_blocks * self.block_size)

    def cache_bytes(self, num_blocks):
        return int(lib.mi355_hybrid_cache_bytes(self.h, int(num_blocks)))

    # ---- one step
    GRAPH_MAX_TOKENS = 16                  # steps of up to this many tokens (decoding batches) replay a hipGraph; longer ones run eagerly

    def _stage(self, total):
        """pinned host + device staging of one step's inputs (one copy per step); grows, never shrinks"""
        if getattr(self, "_dev", None) is None or self._dev.numel() < total:
            n = max(2 * total, 1 << 16)
            self._host = torch.empty(n, dtype=torch.uint8, pin_memory=True)
            self._host_np = self._host.numpy()
            self._dev = torch.empty(n, dtype=torch.uint8, device="cuda")
            self._logits = {}
        if getattr(self, "_stream", None) is None:
            self._stream = torch.cuda.Stream()

    def step(self, meta, state_slots, want_rows=None, trace=False, sync=True, graph=True):
        """meta: BlockEngine.prepare_prompt's dict (every sequence brings its not yet cached tokens: a prompt, a portion of one, or
        one decoded token); state_slots: the sequences' slots (BlockEngine.state_acquire); want_rows: token rows whose logits are
        wanted (default: every sequence's last).  -> logits f32 [len(want_rows), vocab], valid until the next step of the same
        shape (and the residual stream behind every layer [n_layers, T, width] with trace=True).  The step's inputs travel in one
        copy into a static device buffer; steps of up to GRAPH_MAX_TOKENS tokens replay a captured hipGraph."""
        n = len(meta["context_lens"])
        T = len(meta["input_ids"])
        cu = np.asarray(meta["cu_seqlens_q"]).astype(np.int64)
        if want_rows is None:
            want_rows = (cu[1:] - 1).tolist()
        want = np.asarray(want_rows, np.int32)
        n_out = len(want)
        max_ctx = int(meta["max_context_len"])
        self.ensure_rope(max_ctx)
        if len(state_slots) != n or (n and (min(state_slots) < 0 or max(state_slots) >= self.state_slots)):
            raise ValueError("every sequence of a step needs a state slot of the pool")
        bt = np.asarray(meta["block_tables"]).astype(np.int64)
        Wb = max(8, -(-bt.shape[1] // 8) * 8)                 # table width in steps of 8 blocks: few distinct shapes
        Tc = max(16, 1 << max(0, T - 1).bit_length())
        nc = max(n, self.state_slots)
        sizes = [("tok", Tc * 4), ("pos", Tc * 8), ("slot", Tc * 8), ("want", Tc * 4), ("ctx", nc * 4), ("cu", (nc + 1) * 4),
                 ("st", nc * 4), ("bt", nc * Wb * 4)]
        off, total = {}, 0
        for name, b in sizes:
            off[name] = total
            total += -(-b // 16) * 16
        self._stage(total)
        if getattr(self, "_pending", False):
            self._stream.synchronize()
        h = self._host_np

        def put(name, a, dt):
            a = np.ascontiguousarray(np.asarray(a).astype(dt)).reshape(-1)
            h[off[name]:off[name] + a.nbytes] = a.view(np.uint8)
        put("tok", np.asarray(meta["input_ids"]).astype(np.int64), np.int32)
        put("pos", meta["positions"], np.int64)
        put("slot", meta["slot_mapping"], np.int64)
        put("want", want, np.int32)
        put("ctx", np.asarray(meta["context_lens"]).astype(np.int64), np.int32)
        put("cu", cu, np.int32)
        put("st", state_slots, np.int32)
        btw = np.zeros((n, Wb), np.int32)
        btw[:, :bt.shape[1]] = bt
        put("bt", btw, np.int32)
        base = self._dev.data_ptr()
        ptr = {k: base + v for k, v in off.items()}
        use_graph = bool(graph) and not trace and T <= self.GRAPH_MAX_TOKENS
        if use_graph:
            logits = self._logits.get(n_out)
            if logits is None:
                logits = self._logits[n_out] = torch.empty((max(n_out, 1), self.vocab), dtype=torch.float32, device="cuda")
        else:
            logits = torch.empty((max(n_out, 1), self.vocab), dtype=torch.float32, device="cuda")
        tr = torch.empty((len(self.spec.layers), T, self.width), dtype=torch.float32, device="cuda") if trace else None
        with torch.cuda.stream(self._stream):
            self._dev[:total].copy_(self._host[:total], non_blocking=True)
            s = self._stream.cuda_stream
            if use_graph:
                _check(lib.mi355_hybrid_forward_graph(self.h, ptr["tok"], ptr["pos"], ptr["slot"], ptr["bt"], ptr["ctx"], ptr["cu"], ptr["st"],
                                                      ptr["want"], n_out, n, T, Wb, max_ctx, logits.data_ptr(), s), "hybrid_forward_graph")
            else:
                _check(lib.mi355_hybrid_forward(self.h, ptr["tok"], ptr["pos"], ptr["slot"], ptr["bt"], ptr["ctx"], ptr["cu"], ptr["st"],
                                                ptr["want"], n_out, n, T, Wb, max_ctx, logits.data_ptr(),
                                                tr.data_ptr() if trace else None, s), "hybrid_forward")
        self._pending = True
        if sync:
            self._stream.synchronize()
            self._pending = False
        logits = logits[:n_out]
        return (logits, tr) if trace else logits

    def graph_stats(self):
        """(step graphs captured, steps replayed from one)"""
        return int(lib.mi355_hybrid_graph_captures(self.h)), int(lib.mi355_hybrid_graph_replays(self.h))

    def forward_prefill(self, meta, state_slots):
        """logits of the last new token of every sequence (the prompt step of the engine loop)"""
        return self.step(meta, state_slots)
