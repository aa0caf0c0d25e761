"""Slow float64 oracle of the layer-list ("hybrid") models, one function per mechanism, written from the equations and sharing
nothing with candle_vllm_amd/ or csrc/.  Test infrastructure only.

Notation: T tokens of one sequence, W model width; a layer is x <- x + N1(mix(x)); x <- x + N2(ff(x)) with N(y) = y / rms(y) * w
(the norm sits on the sublayer's output, the sublayers read x itself).  Every recurrent mechanism takes and returns its state, so a
sequence can be fed whole, in portions or token by token."""
import math

import numpy as np


def bf16_round(a):
    """f32 values rounded to the nearest bf16 (ties to even), returned as f64"""
    u = np.ascontiguousarray(a, np.float32).view(np.uint32).astype(np.uint64)
    u = ((u + 0x7FFF + ((u >> 16) & 1)) >> 16) << 16
    return u.astype(np.uint32).view(np.float32).astype(np.float64)


def sigmoid(x):
    return 1.0 / (1.0 + np.exp(-x))


def silu(x):
    return x * sigmoid(x)


def softplus(x):
    return np.logaddexp(0.0, x)


def rms_norm(x, w, eps):
    return x / np.sqrt(np.mean(x * x, axis=-1, keepdims=True) + eps) * w


# ---------------------------------------------------------------------------------------------------------------- attention
def rotary_frequencies(base, dims, scaling=None):
    """f_i = base^(-2i/dims), i < dims/2; with `scaling` = (factor, low, high, original): wavelengths 2 pi / f shorter than
    original/high keep f, longer than original/low use f / factor, between them a linear blend in original/wavelength"""
    f = np.array([base ** (-2.0 * i / dims) for i in range(dims // 2)])
    if scaling is None:
        return f
    factor, low, high, original = scaling
    out = []
    for fi in f:
        wl = 2 * math.pi / fi
        if wl < original / high:
            out.append(fi)
        elif wl > original / low:
            out.append(fi / factor)
        else:
            s = (original / wl - low) / (high - low)
            out.append((1 - s) * fi / factor + s * fi)
    return np.array(out)


def rotate_half(x, positions, freqs):
    """x [T, heads, d]; the first 2 len(freqs) dimensions of every head are rotated, dimension i paired with i + len(freqs)"""
    h = len(freqs)
    if h == 0:
        return x
    ang = np.asarray(positions, np.float64)[:, None] * freqs[None, :]
    c, s = np.cos(ang)[:, None, :], np.sin(ang)[:, None, :]
    y = x.copy()
    a, b = x[..., :h], x[..., h:2 * h]
    y[..., :h] = a * c - b * s
    y[..., h:2 * h] = b * c + a * s
    return y


def window_sink_attention(q, k, v, q_pos, k_pos, scale, window=0, sink=None):
    """q [Tq, H, d] at positions q_pos; k [Tk, G, d], v [Tk, G, vd] at positions k_pos (the whole context, new tokens included).
    A query at position i sees keys at j with j <= i and (window == 0 or i - j < window).  sink [H] or None: one more term
    exp(sink_h) in the denominator, with no value.  -> [Tq, H, vd]"""
    Tq, H, _ = q.shape
    G, vd = k.shape[1], v.shape[2]
    out = np.zeros((Tq, H, vd))
    for a in range(Tq):
        i = q_pos[a]
        sel = [b for b, j in enumerate(k_pos) if j <= i and (window == 0 or i - j < window)]
        for h in range(H):
            g = h // (H // G)
            sc = np.array([np.dot(q[a, h], k[b, g]) * scale for b in sel])
            m = max(sc.max(), sink[h]) if sink is not None else sc.max()
            e = np.exp(sc - m)
            den = e.sum() + (math.exp(sink[h] - m) if sink is not None else 0.0)
            out[a, h] = (e[:, None] * v[sel, g]).sum(0) / den
    return out


# ---------------------------------------------------------------------------------------------------------------- delta rule
def causal_conv_silu(x, w, tail=None):
    """x [T, C], w [C, taps] (last column = the current token); tail [taps-1, C] = the inputs before x (zeros at the start).
    -> (silu(conv) [T, C], new tail)"""
    T, C = x.shape
    taps = w.shape[1]
    if tail is None:
        tail = np.zeros((taps - 1, C))
    xp = np.concatenate([tail, x], axis=0)
    y = np.zeros((T, C))
    for t in range(T):
        for i in range(taps):
            y[t] += w[:, i] * xp[t + i]
    return silu(y), xp[len(xp) - (taps - 1):] if taps > 1 else np.zeros((0, C))


def gated_delta_rule(q, k, v, beta, g, S=None):
    """q, k [T, G, d] (already unit vectors, q scaled), v [T, H, vd], beta [T, H], g [T, H, d] (decay per key channel; a per-head
    decay is g broadcast over d).  State S [H, d, vd].  Per token and head:
        S <- diag(g) S;  u = beta (v - S^T k);  S <- S + k u^T;  o = S^T q
    -> (o [T, H, vd], S)"""
    T, G, d = q.shape
    H, vd = v.shape[1], v.shape[2]
    if S is None:
        S = np.zeros((H, d, vd))
    S = S.copy()
    o = np.zeros((T, H, vd))
    for t in range(T):
        for h in range(H):
            j = h // (H // G)
            S[h] = g[t, h][:, None] * S[h]
            u = beta[t, h] * (v[t, h] - S[h].T @ k[t, j])
            S[h] = S[h] + np.outer(k[t, j], u)
            o[t, h] = S[h].T @ q[t, j]
    return o, S


def unit_heads(x, eps):
    return x / np.sqrt(np.sum(x * x, axis=-1, keepdims=True) + eps)


def decay(a_log, pre, dt_bias):
    """exp(-exp(a_log) * softplus(pre + dt_bias)); a_log per head, pre / dt_bias per head or per (head, channel)"""
    return np.exp(-np.exp(a_log) * softplus(pre + dt_bias))


# ---------------------------------------------------------------------------------------------------------------- minGRU
def min_gru(z_pre, u, S=None):
    """z = sigmoid(z_pre); candidate c = u + 1/2 where u >= 0, sigmoid(u) where u < 0; S_t = (1 - z) S_(t-1) + z c.  -> (S_t, S_T)"""
    T, C = u.shape
    S = np.zeros(C) if S is None else S.copy()
    z = sigmoid(z_pre)
    c = np.where(u >= 0, u + 0.5, sigmoid(u))
    out = np.zeros((T, C))
    for t in range(T):
        S = (1 - z[t]) * S + z[t] * c[t]
        out[t] = S
    return out, S


def clamped_glu(gate, up, limit, alpha):
    g = np.minimum(gate, limit)
    u = np.clip(up, -limit, limit)
    return g * sigmoid(alpha * g) * (u + 1.0)


# ---------------------------------------------------------------------------------------------------------------- a Sogodra model
UNIT_EPS = 1e-6
GLU_ALPHA = 1.702


class SogodraOracle:
    """cfg: the design's config dict; W: tensor name -> f64 array.  `feed(tokens)` runs the next tokens of ONE sequence from the
    state earlier calls left and returns the logits of every fed token (and the residual stream behind every layer)."""

    def __init__(self, cfg, W):
        self.cfg, self.W = cfg, W
        self.eps = cfg["norm"]["eps"]
        self.reset()

    def reset(self):
        self.pos = 0
        self.state = [dict() for _ in self.cfg["layers"]]

    def _attention(self, st, p, c, h, positions):
        W = self.W
        T = h.shape[0]
        H, G, d, vd = c["heads"], c["kv_heads"], c["dim"], c["vdim"]
        q = (h @ W[p + "q"].T).reshape(T, H, d)
        k = (h @ W[p + "k"].T).reshape(T, G, d)
        v = (h @ W[p + "v"].T).reshape(T, G, vd)
        if p + "q.norm" in W:
            q, k = rms_norm(q, W[p + "q.norm"], self.eps), rms_norm(k, W[p + "k.norm"], self.eps)
        rot = c.get("rot")
        if rot:
            sc = rot.get("scaling")
            f = rotary_frequencies(rot["base"], rot["dims"], (sc["factor"], sc["low"], sc["high"], sc["original"]) if sc else None)
            q, k = rotate_half(q, positions, f), rotate_half(k, positions, f)
        st["k"] = k if "k" not in st else np.concatenate([st["k"], k])
        st["v"] = v if "v" not in st else np.concatenate([st["v"], v])
        window = c["mask"]["size"] if c.get("mask") else 0
        o = window_sink_attention(q, st["k"], st["v"], positions, list(range(len(st["k"]))), c["scale"], window, W.get(p + "sink"))
        return o.reshape(T, H * vd) @ W[p + "o"].T

    def _delta(self, st, p, c, h, per_channel, low_rank_gate):
        W = self.W
        T = h.shape[0]
        H, G, d, vd = c["heads"], c["kv_heads"], c["dim"], c["vdim"]
        outs = []
        for name in ("q", "k", "v"):
            y, st["tail_" + name] = causal_conv_silu(h @ W[p + name].T, W[p + name + ".conv"], st.get("tail_" + name))
            outs.append(y)
        q = unit_heads(outs[0].reshape(T, G, d), UNIT_EPS) * d ** -0.5
        k = unit_heads(outs[1].reshape(T, G, d), UNIT_EPS)
        v = outs[2].reshape(T, H, vd)
        beta = sigmoid(h @ W[p + "b"].T)
        if per_channel:
            pre = ((h @ W[p + "a1"].T) @ W[p + "a2"].T).reshape(T, H, d)
            g = decay(W[p + "A_log"][None, :, None], pre, W[p + "dt_bias"].reshape(1, H, d))
        else:
            g = decay(W[p + "A_log"][None, :], h @ W[p + "a"].T, W[p + "dt_bias"][None, :])[:, :, None] * np.ones((1, 1, d))
        o, st["S"] = gated_delta_rule(q, k, v, beta, g, st.get("S"))
        o = rms_norm(o, W[p + "norm"], self.eps)
        gate = sigmoid((h @ W[p + "g1"].T) @ W[p + "g2"].T) if low_rank_gate else silu(h @ W[p + "g"].T)
        return (o * gate.reshape(T, H, vd)).reshape(T, H * vd) @ W[p + "o"].T

    def _mingru(self, st, p, h):
        W = self.W
        S, st["S"] = min_gru(h @ W[p + "z"].T + W[p + "z.b"], h @ W[p + "x"].T + W[p + "x.b"], st.get("S"))
        return (S * silu(h @ W[p + "g"].T)) @ W[p + "o"].T

    def feed(self, tokens):
        W, cfg = self.W, self.cfg
        positions = list(range(self.pos, self.pos + len(tokens)))
        self.pos += len(tokens)
        x = W["embed"][np.asarray(tokens)]
        trace = []
        for i, lc in enumerate(cfg["layers"]):
            p, st, m = "l%d." % i, self.state[i], lc["mixer"]
            if lc["type"] == "parallel":
                y = (m["left_scale"] * self._attention(st.setdefault("left", {}), p + "mix.left.", m["left"], x, positions)
                     + m["right_scale"] * self._delta(st.setdefault("right", {}), p + "mix.right.", m["right"], x, True, True))
            elif lc["type"] == "delta":
                y = self._delta(st, p + "mix.", m, x, False, False)
            elif lc["type"] == "mingru":
                y = self._mingru(st, p + "mix.", x)
            else:
                raise ValueError(lc["type"])
            x = x + rms_norm(y, W[p + "norm1"], self.eps)
            if lc.get("mlp"):
                f = lc["mlp"]
                a = clamped_glu(x @ W[p + "mlp.gate"].T, x @ W[p + "mlp.up"].T, f["limit"], GLU_ALPHA)
                x = x + rms_norm(a @ W[p + "mlp.down"].T, W[p + "norm2"], self.eps)
            trace.append(x.copy())
        return rms_norm(x, W["final.norm"], self.eps) @ W["head"].T, np.stack(trace)


def random_sogodra(rng, cfg, scale=1.0):
    """random bf16-representable weights for a config (f64 arrays): projections ~ N(0, 1/in), norms near 1, biases small"""
    W = {}

    def mat(name, rows, cols, s=None):
        W[name] = bf16_round(rng.standard_normal((rows, cols)) * (s if s is not None else scale / math.sqrt(cols)))

    def vec(name, n, mean=0.0, s=0.1):
        W[name] = bf16_round(mean + s * rng.standard_normal(n))

    Wd, V = cfg["width"], cfg["vocab"]
    mat("embed", V, Wd, 1.0)
    vec("final.norm", Wd, 1.0)
    mat("head", V, Wd)

    def delta(p, c, per_channel, low_rank):
        H, G, d, vd, taps = c["heads"], c["kv_heads"], c["dim"], c["vdim"], c["conv"]
        mat(p + "q", G * d, Wd); mat(p + "k", G * d, Wd); mat(p + "v", H * vd, Wd)
        for n, ch in (("q", G * d), ("k", G * d), ("v", H * vd)):
            mat(p + n + ".conv", ch, taps, 0.6)
        mat(p + "b", H, Wd)
        vec(p + "A_log", H, -0.5, 0.5)
        vec(p + "norm", vd, 1.0)
        if per_channel:
            r = c.get("_a_rank", 4)
            mat(p + "a1", r, Wd); mat(p + "a2", H * d, r); vec(p + "dt_bias", H * d, 0.0, 0.5)
        else:
            mat(p + "a", H, Wd); vec(p + "dt_bias", H, 0.0, 0.5)
        if low_rank:
            r = c.get("_g_rank", 4)
            mat(p + "g1", r, Wd); mat(p + "g2", H * vd, r)
        else:
            mat(p + "g", H * vd, Wd)
        mat(p + "o", Wd, H * vd)

    for i, lc in enumerate(cfg["layers"]):
        p, m = "l%d." % i, lc["mixer"]
        vec(p + "norm1", Wd, 1.0)
        if lc["type"] == "parallel":
            c = m["left"]
            q = p + "mix.left."
            mat(q + "q", c["heads"] * c["dim"], Wd); mat(q + "k", c["kv_heads"] * c["dim"], Wd); mat(q + "v", c["kv_heads"] * c["vdim"], Wd)
            if c.get("_qk_norm", True):
                vec(q + "q.norm", c["dim"], 1.0); vec(q + "k.norm", c["dim"], 1.0)
            if c.get("_sink", True):
                vec(q + "sink", c["heads"], 0.5, 1.0)
            mat(q + "o", Wd, c["heads"] * c["vdim"])
            delta(p + "mix.right.", m["right"], True, True)
        elif lc["type"] == "delta":
            delta(p + "mix.", m, False, False)
        else:
            w = m["width"]
            mat(p + "mix.z", w, Wd); mat(p + "mix.x", w, Wd); mat(p + "mix.g", w, Wd); mat(p + "mix.o", Wd, w)
            vec(p + "mix.z.b", w); vec(p + "mix.x.b", w)
        if lc.get("mlp"):
            ff = lc["mlp"]["ff"]
            vec(p + "norm2", Wd, 1.0)
            mat(p + "mlp.gate", ff, Wd); mat(p + "mlp.up", ff, Wd); mat(p + "mlp.down", Wd, ff)
    return W
