"""Slow float64 oracle of the Sabolorn design, one function per mechanism, written from the equations and sharing nothing with
candle_vllm_amd/ or csrc/.  Test infrastructure only.  Whole sequences only (no cache, no state: position t of a causal model is
the truth for every way of cutting the sequence into steps).

The design: a layer-list decoder with ONE layer norm (weight, no bias) per layer that both sublayers read,
    h = LN(x);  x <- x + mix(h) + ff(h);  x <- x + RMSnorm(W_p (gelu(W_g x) * e_token)) w;  x <- sum_j a_j X_j,
where e_token is the layer's slice of a second embedding table and X_j are the embedding output and the results of all layers so
far.  Mixers: a state-space mixer with a scalar decay per head, attention with biases, a short convolution behind q / k / v and a
logarithmic distance bias, latent attention (queries through a latent, interleaved yarn rotation on a shared key part, elementwise
sigmoid output gate, optionally on an earlier layer's cached rows).  Feed-forward: relu^2 dense, or experts chosen by sigmoid scores
with a selection-only correction among the best groups, weights normalised.  Scaled embedding, tied output, tanh-capped logits.

A model is (cfg, W): cfg the parsed config.json, W a dict name -> float64 ndarray."""
import math

import numpy as np


def gelu_tanh(z):
    return 0.5 * z * (1.0 + np.tanh(math.sqrt(2.0 / math.pi) * (z + 0.044715 * z ** 3)))


def silu(z):
    return z / (1.0 + np.exp(-z))


def sigmoid(z):
    return 1.0 / (1.0 + np.exp(-z))


def softplus(z):
    return np.logaddexp(0.0, z)


def rms_unit(x, eps):
    return x / np.sqrt(np.mean(x * x, axis=-1, keepdims=True) + eps)


def layer_norm(x, w, eps):
    d = x - np.mean(x, axis=-1, keepdims=True)
    return d / np.sqrt(np.mean(d * d, axis=-1, keepdims=True) + eps) * w


def causal_conv(u, w, bias=None):
    """u [T, C], w [C, taps]: y_t = sum_j w[:, j] u_(t - taps + 1 + j), zeros before the start"""
    T, taps = u.shape[0], w.shape[1]
    y = np.zeros_like(u)
    for j in range(taps):
        back = taps - 1 - j
        if back < T:
            y[back:] += u[:T - back] * w[:, j]
    return y if bias is None else y + bias


def state_space_scan(x, B, C, dt_raw, a_log, dt_bias, skip, S=None):
    """x [T, heads, vd], B and C [T, G, N], dt_raw [T, heads]: S_t = exp(-exp(a_log) dt) S_(t-1) + dt B_t x_t^T, y_t = S_t^T C_t +
    skip x_t with dt = softplus(dt_raw + dt_bias); head h reads group h // (heads / G).  -> (y [T, heads, vd], S [heads, N, vd])"""
    T, heads, vd = x.shape
    G, N = B.shape[1], B.shape[2]
    dt = softplus(dt_raw + dt_bias)
    decay = np.exp(-np.exp(a_log) * dt)
    y = np.zeros((T, heads, vd))
    S = np.zeros((heads, N, vd)) if S is None else np.array(S, dtype=np.float64)
    per = heads // G
    for t in range(T):
        for hd in range(heads):
            g = hd // per
            S[hd] = decay[t, hd] * S[hd] + dt[t, hd] * np.outer(B[t, g], x[t, hd])
            y[t, hd] = S[hd].T @ C[t, g] + skip[hd] * x[t, hd]
    return y, S


def gate_then_group_norm(y, z, w, groups, eps):
    """(y silu(z)), every one of `groups` equal parts divided by its own root mean square, times w"""
    T, n = y.shape
    g = y * silu(z)
    return rms_unit(g.reshape(T, groups, n // groups), eps).reshape(T, n) * w


def mamba2(h, W, p, c, eps):
    heads, vd, N, G, ng = c["heads"], c["vdim"], c["state"], c["groups"], c.get("norm_groups", 1)
    inner = heads * vd
    T = h.shape[0]
    a = h @ W[p + "in"].T
    z, xbc, dt = a[:, :inner], a[:, inner:2 * inner + 2 * G * N], a[:, 2 * inner + 2 * G * N:]
    xbc = silu(causal_conv(xbc, W[p + "conv"], W[p + "conv.b"]))
    x = xbc[:, :inner].reshape(T, heads, vd)
    B = xbc[:, inner:inner + G * N].reshape(T, G, N)
    C = xbc[:, inner + G * N:].reshape(T, G, N)
    y, _ = state_space_scan(x, B, C, dt, W[p + "A_log"], W[p + "dt_bias"], W[p + "D"])
    return gate_then_group_norm(y.reshape(T, inner), z, W[p + "norm"], ng, eps) @ W[p + "o"].T


def softmax_rows(s, mask):
    s = np.where(mask, s, -np.inf)
    s = s - np.max(s, axis=-1, keepdims=True)
    e = np.exp(s)
    return e / np.sum(e, axis=-1, keepdims=True)


def distance_bias_attention(q, k, v, scale, r1=None, r2=None):
    """q [T, H, d], k [T, G, d], v [T, G, vd], causal: score = (q . k) scale - r1[h] ln(1 + r2[h] (i - j)) -> [T, H, vd]"""
    T, H, _ = q.shape
    G, vd = k.shape[1], v.shape[2]
    i = np.arange(T)
    dist = (i[:, None] - i[None, :]).astype(np.float64)
    mask = dist >= 0
    out = np.zeros((T, H, vd))
    for hd in range(H):
        g = hd // (H // G)
        s = (q[:, hd] @ k[:, g].T) * scale
        if r1 is not None:
            s = s - r1[hd] * np.log1p(r2[hd] * np.maximum(dist, 0.0))
        out[:, hd] = softmax_rows(s, mask) @ v[:, g]
    return out


def conv_attention(h, W, p, c):
    H, G, d, vd = c["heads"], c["kv_heads"], c["dim"], c["vdim"]
    T = h.shape[0]
    q = causal_conv(h @ W[p + "q"].T + W[p + "q.b"], W[p + "q.conv"]).reshape(T, H, d)
    k = causal_conv(h @ W[p + "k"].T + W[p + "k.b"], W[p + "k.conv"]).reshape(T, G, d)
    v = causal_conv(h @ W[p + "v"].T + W[p + "v.b"], W[p + "v.conv"]).reshape(T, G, vd)
    out = distance_bias_attention(q, k, v, c["scale"], W[p + "r1"], W[p + "r2"])
    return out.reshape(T, H * vd) @ W[p + "o"].T


def yarn_angles(rot, T):
    """[T, dims / 2] angles and the amplitude on cos and sin"""
    dims, base = int(rot["dims"]), float(rot["base"])
    i = np.arange(dims // 2, dtype=np.float64)
    f = base ** (-2.0 * i / dims)
    amp = 1.0
    sc = rot.get("scaling")
    if sc:
        def at(turns):
            return dims * math.log(sc["original"] / (2.0 * math.pi * turns)) / (2.0 * math.log(base))
        lo = max(math.floor(at(sc["fast"])), 0)
        hi = min(math.ceil(at(sc["slow"])), dims - 1)
        ramp = np.clip((i - lo) / max(hi - lo, 0.001), 0.0, 1.0)
        f = f / sc["factor"] * ramp + f * (1.0 - ramp)
        amp = 0.1 * math.log(sc["factor"]) + 1.0
    return np.arange(T, dtype=np.float64)[:, None] * f[None, :], amp


def rotate_pairs(x, ang, amp, dims):
    """x [T, ..., n]: the first `dims` of the last axis turn in pairs (2i, 2i + 1)"""
    y = x.copy()
    shape = [ang.shape[0]] + [1] * (x.ndim - 2) + [ang.shape[1]]
    cos, sin = (np.cos(ang) * amp).reshape(shape), (np.sin(ang) * amp).reshape(shape)
    u, v = x[..., 0:dims:2], x[..., 1:dims:2]
    y[..., 0:dims:2] = u * cos - v * sin
    y[..., 1:dims:2] = v * cos + u * sin
    return y


def latent_kv(h, W, p, c, eps):
    """what a latent layer caches: the normed latent [T, kv_rank] and the rotated shared key part [T, rot_dim]"""
    R, rd = c["kv_rank"], c["rot_dim"]
    T = h.shape[0]
    a = h @ W[p + "dkv"].T
    lat = rms_unit(a[:, :R], eps) * W[p + "dkv.norm"]
    ang, amp = yarn_angles(c["rot"], T)
    return lat, rotate_pairs(a[:, R:R + rd], ang, amp, int(c["rot"]["dims"]))


def latent_attention(h, W, p, c, eps, kv):
    H, d, rd, vd, R = c["heads"], c["dim"], c["rot_dim"], c["vdim"], c["kv_rank"]
    T = h.shape[0]
    lat, kr = kv
    cq = rms_unit(h @ W[p + "dq"].T, eps) * W[p + "dq.norm"]
    q = (cq @ W[p + "uq"].T).reshape(T, H, d + rd)
    ang, amp = yarn_angles(c["rot"], T)
    qr = rotate_pairs(q[:, :, d:], ang, amp, int(c["rot"]["dims"]))
    ku = (lat @ W[p + "uk"].T).reshape(T, H, d)
    vv = (lat @ W[p + "uv"].T).reshape(T, H, vd)
    mask = np.tril(np.ones((T, T), bool))
    out = np.zeros((T, H, vd))
    for hd in range(H):
        s = (q[:, hd, :d] @ ku[:, hd].T + qr[:, hd] @ kr.T) * c["scale"]
        out[:, hd] = softmax_rows(s, mask) @ vv[:, hd]
    out = out.reshape(T, H * vd) * sigmoid(h @ W[p + "g"].T)
    return out @ W[p + "o"].T


def dense_ff(h, W, p):
    return np.maximum(h @ W[p + "up"].T, 0.0) ** 2 @ W[p + "down"].T


def route(z, correction, top, groups=None, margins=None):
    """z [T, E] router logits -> chosen experts [T, top] (largest choice score first, ties to the lower expert) and their weights:
    scores s = sigmoid(z); choice = s + correction; only experts of the groups[1] groups (of groups[0] equal groups of neighbours)
    with the largest sum of their two best choice scores can be chosen; weights = s[chosen] / (their sum + 1e-20).
    margins: a list that receives, per token, the smallest gap by which a group or an expert won its place"""
    E = z.shape[1]
    s = sigmoid(z)
    choice = s + correction if correction is not None else s.copy()
    if groups:
        cnt, keep = groups
        per = E // cnt
        gs = np.sort(choice.reshape(-1, cnt, per), axis=-1)[:, :, -2:].sum(-1)
        order = np.argsort(-gs, axis=-1, kind="stable")[:, :keep]
        if margins is not None and keep < cnt:
            g2 = -np.sort(-gs, axis=-1)
            margins.extend((g2[:, keep - 1] - g2[:, keep]).tolist())
        ok = np.zeros((z.shape[0], cnt), bool)
        np.put_along_axis(ok, order, True, axis=-1)
        choice = np.where(np.repeat(ok, per, axis=-1), choice, -np.inf)
    ids = np.argsort(-choice, axis=-1, kind="stable")[:, :top]
    if margins is not None and top < E:
        c2 = -np.sort(-choice, axis=-1)
        margins.extend(np.where(np.isfinite(c2[:, top]), c2[:, top - 1] - c2[:, top], np.inf).tolist())
    w = np.take_along_axis(s, ids, axis=-1)
    return ids, w / (w.sum(-1, keepdims=True) + 1e-20)


def moe_choice(h, W, p, r, margins=None):
    gr = r.get("groups")
    return route(h @ W[p + "router"].T, W.get(p + "correction"), r["top"], (gr["count"], gr["keep"]) if gr else None, margins)


def moe_ff(h, W, p, m, margins=None):
    ids, w = moe_choice(h, W, p, m["router"], margins)
    out = np.zeros((h.shape[0], W[p + "e0.down"].shape[0]))
    for t in range(h.shape[0]):
        for e, wt in zip(ids[t], w[t]):
            q = p + "e%d." % e
            out[t] += wt * ((silu(W[q + "gate"] @ h[t]) * (W[q + "up"] @ h[t])) @ W[q + "down"].T)
    return out


def side_input(x, tokens, W, p, i, dim, eps):
    e = W["side.embed"][tokens][:, i * dim:(i + 1) * dim]
    y = (gelu_tanh(x @ W[p + "side.gate"].T) * e) @ W[p + "side.proj"].T
    return x + rms_unit(y, eps) * W[p + "side.norm"]


def forward(cfg, W, tokens, margins=None):
    """-> logits [T, vocab], the residual stream behind every layer [n_layers, T, width]; margins: see route()"""
    tokens = np.asarray(tokens, np.int64)
    eps = float(cfg["norm"]["eps"])
    x = W["embed"][tokens] * float(cfg["embedding"]["scale"])
    X, trace, kv = [x], [], {}
    for i, lc in enumerate(cfg["layers"]):
        p, c = "l%d." % i, lc["mixer"]
        h = layer_norm(x, W[p + "norm1"], eps)
        if lc["type"] == "mamba2":
            mix = mamba2(h, W, p + "mix.", c, eps)
        elif lc["type"] == "attention":
            mix = conv_attention(h, W, p + "mix.", c)
        elif lc["type"] == "latent_attention":
            if "kv_from" in c:
                kv[i] = kv[int(c["kv_from"])]
            else:
                kv[i] = latent_kv(h, W, p + "mix.", c, eps)
            mix = latent_attention(h, W, p + "mix.", c, eps, kv[i])
        else:
            raise ValueError(lc["type"])
        m = lc.get("mlp")
        ff = 0.0
        if m:
            ff = dense_ff(h, W, p + "mlp.") if m["kind"] == "dense" else moe_ff(h, W, p + "mlp.", m, margins)
        x = x + (mix + ff)
        if cfg.get("token_side"):
            x = side_input(x, tokens, W, p, i, int(cfg["token_side"]["dim"]), eps)
        X.append(x)
        if p + "dwa" in W:
            x = sum(W[p + "dwa"][j] * X[j] for j in range(i + 2))
        trace.append(x)
    y = layer_norm(x, W["final.norm"], eps) @ W["embed"].T
    cap = cfg.get("logit_softcap")
    if cap:
        y = cap * np.tanh(y / cap)
    return y, np.stack(trace)


# ---------------------------------------------------------------------------------------------------------------- weights for tests
def bf16_round(a):
    u = np.ascontiguousarray(a, np.float32).view(np.uint32)
    r = ((u + 0x7FFF + ((u >> 16) & 1)) >> 16).astype(np.uint32) << 16
    return r.view(np.float32).astype(np.float64)


def random_sabolorn(rng, cfg):
    """random bf16-representable weights for a config (f64 arrays): projections ~ N(0, 1/in), norms near 1"""
    W = {}

    def mat(name, rows, cols, s=None):
        W[name] = bf16_round(rng.standard_normal((rows, cols)) * (s if s is not None else 1.0 / math.sqrt(cols)))

    def vec(name, n, mean=0.0, s=0.1):
        W[name] = bf16_round(mean + s * rng.standard_normal(n))

    Wd, V, n_layers = cfg["width"], cfg["vocab"], len(cfg["layers"])
    mat("embed", V, Wd, 0.25)                                             # also the output table: logits of a few units, below the cap
    vec("final.norm", Wd, 1.0)
    side = (cfg.get("token_side") or {}).get("dim", 0)
    if side:
        mat("side.embed", V, side * n_layers, 1.0)
    for i, lc in enumerate(cfg["layers"]):
        p, c = "l%d." % i, lc["mixer"]
        q = p + "mix."
        vec(p + "norm1", Wd, 1.0)
        if lc["type"] == "mamba2":
            heads, vd, N, G = c["heads"], c["vdim"], c["state"], c["groups"]
            inner, ch = heads * vd, heads * vd + 2 * G * N
            mat(q + "in", 2 * inner + 2 * G * N + heads, Wd)
            mat(q + "conv", ch, c["conv"], 0.5); vec(q + "conv.b", ch, 0.0, 0.2)
            vec(q + "dt_bias", heads, -1.0, 1.0); vec(q + "A_log", heads, -0.5, 0.7); vec(q + "D", heads, 1.0, 0.3)
            vec(q + "norm", inner, 1.0); mat(q + "o", Wd, inner)
        elif lc["type"] == "attention":
            H, G, d, vd = c["heads"], c["kv_heads"], c["dim"], c["vdim"]
            for n, rows in (("q", H * d), ("k", G * d), ("v", G * vd)):
                mat(q + n, rows, Wd); vec(q + n + ".b", rows, 0.0, 0.3); mat(q + n + ".conv", rows, c["conv"], 0.6)
            W[q + "r1"] = bf16_round(rng.uniform(0.1, 1.5, H)); W[q + "r2"] = bf16_round(rng.uniform(0.05, 2.0, H))
            mat(q + "o", Wd, H * vd)
        else:
            H, d, rd, vd, R, Q = c["heads"], c["dim"], c["rot_dim"], c["vdim"], c["kv_rank"], c["q_rank"]
            mat(q + "dq", Q, Wd); vec(q + "dq.norm", Q, 1.0); mat(q + "uq", H * (d + rd), Q)
            if "kv_from" not in c:
                mat(q + "dkv", R + rd, Wd); vec(q + "dkv.norm", R, 1.0)
            mat(q + "uk", H * d, R); mat(q + "uv", H * vd, R); mat(q + "g", H * vd, Wd); mat(q + "o", Wd, H * vd)
        mlp = lc.get("mlp")
        if mlp and mlp["kind"] == "dense":
            mat(p + "mlp.up", mlp["ff"], Wd); mat(p + "mlp.down", Wd, mlp["ff"])
        elif mlp:
            m, ff, E = p + "mlp.", mlp["expert"]["ff"], mlp["router"]["experts"]
            for e in range(E):
                mat(m + "e%d.gate" % e, ff, Wd); mat(m + "e%d.up" % e, ff, Wd); mat(m + "e%d.down" % e, Wd, ff)
            mat(m + "router", E, Wd, 2.0 / math.sqrt(Wd))
            W[m + "correction"] = bf16_round(rng.uniform(-0.3, 0.3, E))
        if side:
            mat(p + "side.gate", side, Wd); mat(p + "side.proj", Wd, side); vec(p + "side.norm", Wd, 0.5)
        a = rng.uniform(0.1, 1.0, i + 2)
        W[p + "dwa"] = bf16_round(a / a.sum())
    return W
