"""Slow float64 oracle of the Vivazen design, one function per mechanism, written from the equations and sharing nothing with
candle_vllm_amd/ or csrc/.  Test infrastructure only.

The design: a layer-list decoder with the norm BEHIND the residual sum,
    x <- N1(alpha x + mix(x));  x <- N2(alpha x + ff(x)),
N = an RMS norm taken separately over `groups` equal consecutive parts of the vector, then one weight over the whole vector.
Two mixers:
  * latent attention: keys and values are both read off one small latent vector c per token (plus one rotated key part that all
    heads share); sliding window, a sink in the softmax denominator, a sigmoid gate per head on the output;
  * attention with a short causal convolution behind the q / k / v projections, RMS norms over the WHOLE q and k projections,
    unit-RMS values, tanh-capped scores, and a [heads, heads] matrix that mixes the heads' softmax weights before they meet the values.
A layer may borrow another layer's weights and still keeps its own cache.  Feed-forward: down(gelu_tanh(gate h) * (up h))."""
import math

import numpy as np

from .hybrid import bf16_round, sigmoid


# ---------------------------------------------------------------------------------------------------------------- norms, glue
def group_rms_norm(x, w, eps, groups):
    """x [..., n] cut into `groups` equal consecutive parts; every part divided by its own sqrt(mean(part^2) + eps); times w [n]"""
    n = x.shape[-1]
    parts = x.reshape(x.shape[:-1] + (groups, n // groups))
    parts = parts / np.sqrt(np.mean(parts * parts, axis=-1, keepdims=True) + eps)
    return parts.reshape(x.shape) * w


def gelu_tanh(z):
    return 0.5 * z * (1.0 + np.tanh(math.sqrt(2.0 / math.pi) * (z + 0.044715 * z ** 3)))


def gelu_glu(gate, up):
    return gelu_tanh(gate) * up


# ---------------------------------------------------------------------------------------------------------------- rotation
def yarn_frequencies(base, dims, scaling=None):
    """f_i = base^(-2i/dims); with scaling = dict(factor, original, fast, slow): the index where a wavelength completes t turns over
    `original` positions is D(t) = dims ln(original / (2 pi t)) / (2 ln base); between lo = floor(D(fast)) and hi = ceil(D(slow))
    (clipped to [0, dims - 1]) a ramp r_i goes from 0 to 1 and f_i <- r_i f_i / factor + (1 - r_i) f_i.
    -> (frequencies [dims / 2], amplitude) where amplitude = 0.1 ln(factor) + 1 multiplies both cos and sin (1 without scaling)"""
    f = np.array([base ** (-2.0 * i / dims) for i in range(dims // 2)])
    if not scaling:
        return f, 1.0
    factor = scaling["factor"]

    def D(t):
        return dims * math.log(scaling["original"] / (2 * math.pi * t)) / (2 * math.log(base))
    lo = max(math.floor(D(scaling["fast"])), 0)
    hi = min(math.ceil(D(scaling["slow"])), dims - 1)
    r = np.clip((np.arange(dims // 2) - lo) / max(hi - lo, 0.001), 0.0, 1.0)
    return f / factor * r + f * (1 - r), 0.1 * math.log(factor) + 1.0


def rotate_pairs(x, positions, freqs, amplitude=1.0):
    """x [T, ..., n]: dimensions (2i, 2i+1), i < len(freqs), turn by positions * freqs[i]; cos and sin carry `amplitude`; the rest
    of the vector passes"""
    x = np.array(x, dtype=np.float64)
    ang = np.asarray(positions, np.float64)[:, None] * freqs[None, :]
    shape = (x.shape[0],) + (1,) * (x.ndim - 2) + (len(freqs),)
    c, s = (np.cos(ang) * amplitude).reshape(shape), (np.sin(ang) * amplitude).reshape(shape)
    n = 2 * len(freqs)
    u, v = x[..., 0:n:2].copy(), x[..., 1:n:2].copy()
    x[..., 0:n:2] = u * c - v * s
    x[..., 1:n:2] = v * c + u * s
    return x


# ---------------------------------------------------------------------------------------------------------------- attention
def softmax_weights(scores, visible, sink=None):
    """scores [Tq, Tk], visible bool [Tq, Tk]; sink: one more term exp(sink) in the denominator that has no key -> weights [Tq, Tk]"""
    s = np.where(visible, scores, -np.inf)
    m = s.max(axis=1, keepdims=True)
    if sink is not None:
        m = np.maximum(m, sink)
    e = np.where(visible, np.exp(s - m), 0.0)
    den = e.sum(axis=1, keepdims=True) + (np.exp(sink - m) if sink is not None else 0.0)
    return e / den


def visible_mask(q_pos, k_pos, window=0):
    i, j = np.asarray(q_pos)[:, None], np.asarray(k_pos)[None, :]
    vis = j <= i
    if window:
        vis &= (i - j) < window
    return vis


def latent_attention(q_plain, q_rot, c, k_rot, uk, uv, q_pos, k_pos, scale, window=0, sink=None):
    """q_plain [Tq, H, d], q_rot [Tq, H, r] (already rotated); c [Tk, rank] latents and k_rot [Tk, r] (rotated, shared by the heads)
    of the whole context; uk [H d, rank], uv [H vd, rank].  Head h: key = uk_h c, value = uv_h c,
    score = (q_plain . key + q_rot . k_rot) scale.  -> [Tq, H, vd]"""
    Tq, H, d = q_plain.shape
    vd = uv.shape[0] // H
    vis = visible_mask(q_pos, k_pos, window)
    out = np.zeros((Tq, H, vd))
    for h in range(H):
        keys = c @ uk[h * d:(h + 1) * d].T
        vals = c @ uv[h * vd:(h + 1) * vd].T
        s = (q_plain[:, h] @ keys.T + q_rot[:, h] @ k_rot.T) * scale
        out[:, h] = softmax_weights(s, vis, None if sink is None else sink[h]) @ vals
    return out


def causal_conv(u, w, tail=None):
    """u [T, C], w [C, taps]: y_t = sum_j w[:, j] u_(t - taps + 1 + j), zeros before the start; tail [taps - 1, C] = the inputs before
    u.  No activation.  -> (y, new tail)"""
    T, C = u.shape
    taps = w.shape[1]
    if tail is None:
        tail = np.zeros((taps - 1, C))
    up = np.concatenate([tail, u], axis=0)
    y = np.zeros((T, C))
    for t in range(T):
        for j in range(taps):
            y[t] += w[:, j] * up[t + j]
    return y, up[len(up) - (taps - 1):] if taps > 1 else np.zeros((0, C))


def unit_rms(x, eps):
    return x / np.sqrt(np.mean(x * x, axis=-1, keepdims=True) + eps)


def mixed_head_attention(q, k, v, q_pos, k_pos, scale, softcap, talk):
    """q [Tq, H, d]; k [Tk, G, d], v [Tk, G, vd] of the whole context.  Scores (q . k) scale, then cap tanh(s / cap); causal softmax
    per head; the heads' weights are mixed, w'_h = sum_g talk[h, g] w_g; head h applies w'_h to the values of ITS key/value head."""
    Tq, H, _ = q.shape
    G, vd = k.shape[1], v.shape[2]
    vis = visible_mask(q_pos, k_pos)
    w = np.zeros((H, Tq, len(k_pos)))
    for h in range(H):
        s = (q[:, h] @ k[:, h // (H // G)].T) * scale
        if softcap:
            s = softcap * np.tanh(s / softcap)
        w[h] = softmax_weights(s, vis)
    mixed = np.einsum("hg,gqk->hqk", talk, w)
    out = np.zeros((Tq, H, vd))
    for h in range(H):
        out[:, h] = mixed[h] @ v[:, h // (H // G)]
    return out


# ---------------------------------------------------------------------------------------------------------------- a model
class VivazenOracle:
    """cfg: the design's config dict; W: tensor name -> f64 array.  `feed(tokens)` runs the next tokens of ONE sequence behind what
    earlier calls fed and returns (logits of every fed token, residual stream behind every layer)."""

    def __init__(self, cfg, W):
        self.cfg, self.W = cfg, W
        self.eps, self.groups, self.alpha = cfg["norm"]["eps"], cfg["norm"]["groups"], cfg["postln_alpha"]
        self.reset()

    def reset(self):
        self.pos = 0
        self.state = [dict() for _ in self.cfg["layers"]]

    def _norm(self, x, name):
        return group_rms_norm(x, self.W[name], self.eps, self.groups)

    def _latent(self, st, p, c, h, positions):
        W = self.W
        T = h.shape[0]
        H, d, r, vd, rank = c["heads"], c["dim"], c["rot_dim"], c["vdim"], c["kv_rank"]
        q = (h @ W[p + "q"].T).reshape(T, H, d + r)
        dkv = h @ W[p + "dkv"].T
        lat = unit_rms(dkv[:, :rank], self.eps) * W[p + "dkv.norm"]
        rot = c["rot"]
        f, amp = yarn_frequencies(rot["base"], rot["dims"], rot.get("scaling"))
        q_rot = rotate_pairs(q[:, :, d:], positions, f, amp)
        k_rot = rotate_pairs(dkv[:, rank:], positions, f, amp)
        st["c"] = lat if "c" not in st else np.concatenate([st["c"], lat])
        st["kr"] = k_rot if "kr" not in st else np.concatenate([st["kr"], k_rot])
        window = c["mask"]["size"] if c.get("mask") else 0
        o = latent_attention(q[:, :, :d], q_rot, st["c"], st["kr"], W[p + "uk"], W[p + "uv"], positions, list(range(len(st["c"]))),
                             c["scale"], window, W.get(p + "sink"))
        o = o * sigmoid(h @ W[p + "g"].T)[:, :, None]
        return o.reshape(T, H * vd) @ W[p + "o"].T

    def _attention(self, st, p, c, h, positions):
        W = self.W
        T = h.shape[0]
        H, G, d, vd = c["heads"], c["kv_heads"], c["dim"], c["vdim"]
        outs = []
        for name in ("q", "k", "v"):
            y, st["tail_" + name] = causal_conv(h @ W[p + name].T, W[p + name + ".conv"], st.get("tail_" + name))
            outs.append(y)
        q = (unit_rms(outs[0], self.eps) * W[p + "q.norm"]).reshape(T, H, d)
        k = (unit_rms(outs[1], self.eps) * W[p + "k.norm"]).reshape(T, G, d)
        v = unit_rms(outs[2].reshape(T, G, vd), self.eps)
        st["k"] = k if "k" not in st else np.concatenate([st["k"], k])
        st["v"] = v if "v" not in st else np.concatenate([st["v"], v])
        o = mixed_head_attention(q, st["k"], st["v"], positions, list(range(len(st["k"]))), c["scale"], c.get("softcap", 0.0), W[p + "talk"])
        return o.reshape(T, H * vd) @ W[p + "o"].T

    def feed(self, tokens):
        W, cfg = self.W, self.cfg
        positions = list(range(self.pos, self.pos + len(tokens)))
        self.pos += len(tokens)
        x = W["embed"][np.asarray(tokens)]
        trace = []
        for i, lc in enumerate(cfg["layers"]):
            src = lc.get("weights_of", i)
            p, st, m = "l%d." % src, self.state[i], lc["mixer"]
            if lc["type"] == "latent_attention":
                y = self._latent(st, p + "mix.", m, x, positions)
            elif lc["type"] == "attention":
                y = self._attention(st, p + "mix.", m, x, positions)
            else:
                raise ValueError(lc["type"])
            x = self._norm(self.alpha * x + y, p + "norm1")
            if lc.get("mlp"):
                a = gelu_glu(x @ W[p + "mlp.gate"].T, x @ W[p + "mlp.up"].T)
                x = self._norm(self.alpha * x + a @ W[p + "mlp.down"].T, p + "norm2")
            trace.append(x.copy())
        return self._norm(x, "final.norm") @ W["head"].T, np.stack(trace)


def random_vivazen(rng, cfg, scale=1.0):
    """random bf16-representable weights for a config (f64 arrays): projections ~ N(0, 1/in), norms near 1"""
    W = {}

    def mat(name, rows, cols, s=None):
        W[name] = bf16_round(rng.standard_normal((rows, cols)) * (s if s is not None else scale / math.sqrt(cols)))

    def vec(name, n, mean=0.0, s=0.1):
        W[name] = bf16_round(mean + s * rng.standard_normal(n))

    Wd, V = cfg["width"], cfg["vocab"]
    mat("embed", V, Wd, 1.0)
    vec("final.norm", Wd, 1.0)
    mat("head", V, Wd)
    for i, lc in enumerate(cfg["layers"]):
        if "weights_of" in lc:
            continue
        p, c = "l%d." % i, lc["mixer"]
        q = p + "mix."
        vec(p + "norm1", Wd, 1.0)
        if lc["type"] == "latent_attention":
            H, d, r, vd, rank = c["heads"], c["dim"], c["rot_dim"], c["vdim"], c["kv_rank"]
            mat(q + "q", H * (d + r), Wd, 2.0 / math.sqrt(Wd)); mat(q + "dkv", rank + r, Wd, 2.0 / math.sqrt(Wd))
            vec(q + "dkv.norm", rank, 1.0)
            mat(q + "uk", H * d, rank); mat(q + "uv", H * vd, rank)
            vec(q + "sink", H, 0.5, 1.0)
            mat(q + "g", H, Wd)
            mat(q + "o", Wd, H * vd)
        else:
            H, G, d, vd, taps = c["heads"], c["kv_heads"], c["dim"], c["vdim"], c["conv"]
            for n, ch in (("q", H * d), ("k", G * d), ("v", G * vd)):
                mat(q + n, ch, Wd)
                mat(q + n + ".conv", ch, taps, 0.6)
            vec(q + "q.norm", H * d, 1.0, 0.3); vec(q + "k.norm", G * d, 1.0, 0.3)
            W[q + "talk"] = bf16_round(np.eye(H) * 0.7 + 0.3 * rng.standard_normal((H, H)))
            mat(q + "o", Wd, H * vd)
        if lc.get("mlp"):
            ff = lc["mlp"]["ff"]
            vec(p + "norm2", Wd, 1.0)
            mat(p + "mlp.gate", ff, Wd); mat(p + "mlp.up", ff, Wd); mat(p + "mlp.down", Wd, ff)
    return W
