"""Slow float64 oracle of the Kerolorn design, one function per mechanism, written from the equations and sharing nothing with
candle_vllm_amd/ or csrc/.  Test infrastructure only.

The design: a layer-list decoder with a norm on BOTH sides of every sublayer,
    x <- x + Nb(mix(conv_in(Na(x))));   x <- x + Nd(ff(Nc(x))),
N = RMS norm with a weight.  conv_in(h) = h + C(h): a causal depthwise convolution over time added to its own input, in front of the
mixer only; the last taps - 1 rows of h are state.  One mixer: grouped-query attention with interleaved rotary pairs (yarn-scaled
frequencies and amplitude) on the leading dimensions of every head, a weightless RMS norm of q and k AFTER the rotation, a learned
temperature per head, and a mask that shows a sliding window plus the first few tokens of the sequence.  Feed-forward: a mixture of
small silu gate/up experts chosen by a softmax router with a selection-only correction, plus a shared expert behind a sigmoid gate.
Logits are multiplied by a constant."""
import math

import numpy as np

from .hybrid import bf16_round, sigmoid, silu, rms_norm
from .vivazen import yarn_frequencies, rotate_pairs


# ---------------------------------------------------------------------------------------------------------------- input convolution
def conv_residual(h, w, tail=None):
    """h [T, C], w [C, taps]: y_t = h_t + sum_j w[:, j] h_(t - taps + 1 + j), rows before the sequence's start are zeros; tail
    [taps - 1, C] = the rows of h before this portion.  -> (y, new tail)"""
    T, C = h.shape
    taps = w.shape[1]
    if tail is None:
        tail = np.zeros((taps - 1, C))
    hp = np.concatenate([tail, h], axis=0)
    y = np.array(h, dtype=np.float64)
    for t in range(T):
        for j in range(taps):
            y[t] += w[:, j] * hp[t + j]
    return y, (hp[len(hp) - (taps - 1):] if taps > 1 else np.zeros((0, C)))


# ---------------------------------------------------------------------------------------------------------------- attention
def unit_rms(x, eps):
    return x / np.sqrt(np.mean(x * x, axis=-1, keepdims=True) + eps)


def window_keep_mask(q_pos, k_pos, window, keep_first):
    """bool [queries, keys]: causal; with a window (0 = none) only the last `window` positions stay visible -- and the keys at
    positions below keep_first, whatever their distance"""
    i, j = np.asarray(q_pos)[:, None], np.asarray(k_pos)[None, :]
    vis = j <= i
    if window:
        vis &= ((i - j) < window) | (j < keep_first)
    return vis


def head_temperature_attention(q, k, v, q_pos, k_pos, scale, temp, window=0, keep_first=0):
    """q [Tq, H, d] (rotated, unit rms); k [Tk, G, d], v [Tk, G, vd] of the whole context.  score_h = (q_h . k_g) scale temp[h],
    g = h // (H / G); plain softmax over the visible keys -> [Tq, H, vd]"""
    Tq, H, _ = q.shape
    G, vd = k.shape[1], v.shape[2]
    vis = window_keep_mask(q_pos, k_pos, window, keep_first)
    out = np.zeros((Tq, H, vd))
    for h in range(H):
        g = h // (H // G)
        s = np.where(vis, (q[:, h] @ k[:, g].T) * scale * temp[h], -np.inf)
        e = np.exp(s - s.max(axis=1, keepdims=True))
        out[:, h] = (e / e.sum(axis=1, keepdims=True)) @ v[:, g]
    return out


# ---------------------------------------------------------------------------------------------------------------- mixture of experts
def route(h, w_router, correction, top, scale, margins=None):
    """h [T, W] -> (chosen experts [T, top] by descending choice score, weights [T, top]).  s = softmax(W_r h); the choice is made on
    s + correction, the weight of a chosen expert is its s times `scale` (no renormalisation).  margins: a list that receives, per
    token, the gap between the last chosen and the first rejected choice score (how close the call was)"""
    z = h @ w_router.T
    e = np.exp(z - z.max(axis=1, keepdims=True))
    s = e / e.sum(axis=1, keepdims=True)
    choice = s + correction
    order = np.argsort(-choice, axis=1, kind="stable")[:, :top]
    if margins is not None and top < choice.shape[1]:
        ranked = -np.sort(-choice, axis=1)
        margins.extend((ranked[:, top - 1] - ranked[:, top]).tolist())
    return order, np.take_along_axis(s, order, axis=1) * scale


def silu_expert(h, gate, up, down):
    return (silu(h @ gate.T) * (h @ up.T)) @ down.T


def moe(h, W, p, n_experts, top, scale, shared, margins=None):
    """W: name -> array, p: the feed-forward's prefix ('l3.mlp.')"""
    corr = W[p + "correction"] if p + "correction" in W else np.zeros(n_experts)
    idx, wt = route(h, W[p + "router"], corr, top, scale, margins)
    y = np.zeros((h.shape[0], W[p + "e0.down"].shape[0]))
    for e in range(n_experts):
        for t, k in zip(*np.nonzero(idx == e)):
            q = p + "e%d." % e
            y[t] += wt[t, k] * silu_expert(h[t:t + 1], W[q + "gate"], W[q + "up"], W[q + "down"])[0]
    if shared:
        q = p + "shared."
        y += sigmoid(h @ W[q + "sg"].T) * silu_expert(h, W[q + "gate"], W[q + "up"], W[q + "down"])
    return y


# ---------------------------------------------------------------------------------------------------------------- a model
class KerolornOracle:
    """cfg: the design's config dict; W: tensor name -> f64 array.  `feed(tokens)` runs the next tokens of ONE sequence behind what
    earlier calls fed and returns (logits of every fed token, residual stream behind every layer)."""

    def __init__(self, cfg, W):
        self.cfg, self.W = cfg, W
        self.eps = cfg["norm"]["eps"]
        self.reset()

    def reset(self):
        self.pos = 0
        self.state = [dict() for _ in self.cfg["layers"]]
        self.margins = []             # of every routing decision so far (route)

    def _attention(self, st, p, c, h, positions):
        W = self.W
        T = h.shape[0]
        H, G, d, vd = c["heads"], c["kv_heads"], c["dim"], c["vdim"]
        q = (h @ W[p + "q"].T).reshape(T, H, d)
        k = (h @ W[p + "k"].T).reshape(T, G, d)
        v = (h @ W[p + "v"].T).reshape(T, G, vd)
        rot = c.get("rot")
        if rot and rot["dims"] > 0:
            f, amp = yarn_frequencies(rot["base"], rot["dims"], rot.get("scaling"))
            q, k = rotate_pairs(q, positions, f, amp), rotate_pairs(k, positions, f, amp)
        q, k = unit_rms(q, self.eps), unit_rms(k, self.eps)
        st["k"] = k if "k" not in st else np.concatenate([st["k"], k])
        st["v"] = v if "v" not in st else np.concatenate([st["v"], v])
        mask = c.get("mask") or {}
        o = head_temperature_attention(q, st["k"], st["v"], positions, list(range(len(st["k"]))), c["scale"],
                                       W[p + "temp"] if p + "temp" in W else np.ones(H),
                                       int(mask.get("size", 0)), int(mask.get("keep_first", 0)))
        return o.reshape(T, H * vd) @ W[p + "o"].T

    def feed(self, tokens):
        W, cfg = self.W, self.cfg
        positions = list(range(self.pos, self.pos + len(tokens)))
        self.pos += len(tokens)
        x = W["embed"][np.asarray(tokens)]
        trace = []
        for i, lc in enumerate(cfg["layers"]):
            p, st = "l%d." % i, self.state[i]
            if lc["type"] != "attention":
                raise ValueError(lc["type"])
            h = rms_norm(x, W[p + "norm1"], self.eps)
            if p + "canon1" in W:
                h, st["tail"] = conv_residual(h, W[p + "canon1"], st.get("tail"))
            y = self._attention(st, p + "mix.", lc["mixer"], h, positions)
            x = x + rms_norm(y, W[p + "norm1b"], self.eps)
            mlp = lc.get("mlp")
            if mlp:
                h = rms_norm(x, W[p + "norm2"], self.eps)
                r = mlp["router"]
                y = moe(h, W, p + "mlp.", r["experts"], r["top"], r["scale"], bool(mlp.get("shared")), self.margins)
                x = x + rms_norm(y, W[p + "norm2b"], self.eps)
            trace.append(x.copy())
        return rms_norm(x, W["final.norm"], self.eps) @ W["head"].T * cfg.get("logit_scale", 1.0), np.stack(trace)


def random_kerolorn(rng, cfg, scale=1.0):
    """random bf16-representable weights for a config (f64 arrays): projections ~ N(0, 1/in), norms near 1"""
    W = {}

    def mat(name, rows, cols, s=None):
        W[name] = bf16_round(rng.standard_normal((rows, cols)) * (s if s is not None else scale / math.sqrt(cols)))

    def vec(name, n, mean=0.0, s=0.1):
        W[name] = bf16_round(mean + s * rng.standard_normal(n))

    Wd, V = cfg["width"], cfg["vocab"]
    taps = cfg["canon"]["taps"]
    mat("embed", V, Wd, 1.0)
    vec("final.norm", Wd, 1.0)
    mat("head", V, Wd)
    for i, lc in enumerate(cfg["layers"]):
        p, c = "l%d." % i, lc["mixer"]
        q = p + "mix."
        H, G, d, vd = c["heads"], c["kv_heads"], c["dim"], c["vdim"]
        vec(p + "norm1", Wd, 1.0); vec(p + "norm1b", Wd, 1.0)
        mat(p + "canon1", Wd, taps, 0.4)
        mat(q + "q", H * d, Wd); mat(q + "k", G * d, Wd); mat(q + "v", G * vd, Wd)
        vec(q + "temp", H, 1.0, 0.3)
        mat(q + "o", Wd, H * vd)
        mlp = lc.get("mlp")
        if mlp:
            vec(p + "norm2", Wd, 1.0); vec(p + "norm2b", Wd, 1.0)
            m, ff = p + "mlp.", mlp["expert"]["ff"]
            E = mlp["router"]["experts"]
            for e in range(E):
                mat(m + "e%d.gate" % e, ff, Wd); mat(m + "e%d.up" % e, ff, Wd); mat(m + "e%d.down" % e, Wd, ff)
            mat(m + "router", E, Wd, 2.0 / math.sqrt(Wd))
            W[m + "correction"] = bf16_round(rng.uniform(0.0, 2.0 / E, E))       # of the softmax values' size: both decide the choice
            if mlp.get("shared"):
                fs = mlp["shared"]["ff"]
                mat(m + "shared.gate", fs, Wd); mat(m + "shared.up", fs, Wd); mat(m + "shared.down", Wd, fs)
                mat(m + "shared.sg", 1, Wd)
    return W
