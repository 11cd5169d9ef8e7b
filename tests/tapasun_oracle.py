"""A plain float64 implementation of the Tapasun design, one function per mechanism, one token at
a time.  It shares no code with mxserve: the tests compare the engine against it.

A model is (config dict, {tensor name: float64 numpy array}).  `Oracle.step(token)` feeds one token
of one sequence and returns (logits, the residual stream after every layer).

Notation: h is a sublayer's input [width]; RMS norm is x / sqrt(mean(x^2) + eps).
"""
from __future__ import annotations

import math

import numpy as np


# ------------------------------------------------------------------------------------- small pieces
def rms_norm(x, eps):
    return x / np.sqrt(np.mean(x * x, axis=-1, keepdims=True) + eps)


def silu(z):
    return z / (1.0 + np.exp(-z))


def sigmoid(z):
    return 1.0 / (1.0 + np.exp(-z))


def softplus(z):
    return np.logaddexp(0.0, z)


def rotary_frequencies(rot: dict) -> np.ndarray:
    """f_i = base^(-2i/dims), then the scaling the config asks for: three bands by wavelength when it
    gives `original` (long waves slowed by `factor`, short ones kept, a linear blend between), else a
    plain division by `factor`."""
    dims = int(rot["dims"])
    f = np.array([float(rot["base"]) ** (-2.0 * i / dims) for i in range(dims // 2)])
    sc = rot.get("scaling") or None
    if not sc:
        return f
    factor = float(sc["factor"])
    if "original" not in sc:
        return f / factor
    orig, low, high = float(sc["original"]), float(sc["low"]), float(sc["high"])
    out = np.empty_like(f)
    for i, fi in enumerate(f):
        wave = 2.0 * math.pi / fi
        if wave < orig / high:
            out[i] = fi
        elif wave > orig / low:
            out[i] = fi / factor
        else:
            s = (orig / wave - low) / (high - low)
            out[i] = (1.0 - s) * fi / factor + s * fi
    return out


def rotate_pairs(x, pos, freqs, sign=1.0):
    """Turns the pair (x[2i], x[2i+1]) by sign * pos * freqs[i]; dimensions past 2 * len(freqs) pass."""
    y = x.copy()
    n = len(freqs)
    a = sign * pos * freqs
    c, s = np.cos(a), np.sin(a)
    u, v = x[..., 0:2 * n:2], x[..., 1:2 * n:2]
    y[..., 0:2 * n:2] = u * c - v * s
    y[..., 1:2 * n:2] = v * c + u * s
    return y


def causal_conv_step(hist: list, x, w, b, taps: int):
    """hist: the earlier inputs of this sequence (only the last taps - 1 matter).  Returns the filter's
    output for the input x; the last column of w weighs x itself."""
    acc = np.zeros_like(x) if b is None else b.copy()
    for j in range(taps):
        back = taps - 1 - j  # how many tokens ago
        if back == 0:
            acc = acc + w[:, j] * x
        elif back <= len(hist):
            acc = acc + w[:, j] * hist[-back]
    return acc


# ------------------------------------------------------------------------------------- mixers
class Mamba2:
    def __init__(self, mc, w, p, eps):
        self.H, self.P, self.N, self.G = int(mc["heads"]), int(mc["vdim"]), int(mc["state"]), int(mc["groups"])
        self.taps, self.ng, self.eps = int(mc["conv"]), int(mc["norm_groups"]), eps
        self.w, self.p = w, p
        self.hist: list = []
        self.S = np.zeros((self.H, self.N, self.P))

    def step(self, h, pos, caches):
        w, p, H, P, N, G = self.w, self.p, self.H, self.P, self.N, self.G
        inner = H * P
        y = w[p + "in"] @ h
        z, xbc, dt = y[:inner], y[inner:2 * inner + 2 * G * N], y[2 * inner + 2 * G * N:]
        c = silu(causal_conv_step(self.hist, xbc, w[p + "conv"], w[p + "conv.b"], self.taps))
        self.hist.append(xbc)
        self.hist = self.hist[-(self.taps - 1):] if self.taps > 1 else []
        x = c[:inner].reshape(H, P)
        B = c[inner:inner + G * N].reshape(G, N)
        C = c[inner + G * N:].reshape(G, N)
        dt = softplus(dt + w[p + "dt_bias"])
        out = np.zeros((H, P))
        for hd in range(H):
            g = hd // (H // G)
            a = math.exp(-math.exp(w[p + "A_log"][hd]) * dt[hd])
            self.S[hd] = a * self.S[hd] + dt[hd] * np.outer(B[g], x[hd])
            out[hd] = self.S[hd].T @ C[g] + w[p + "D"][hd] * x[hd]
        o = out.reshape(-1) * silu(z)
        o = rms_norm(o.reshape(self.ng, -1), self.eps).reshape(-1) * w[p + "norm"]
        return w[p + "o"] @ o


class Attention:
    """Softmax attention with rotary positions and a sink in the denominator.  `sink`: None for the
    fixed sink of score 0, else the name of the per-head tensor.  rot_values: values are turned by
    their position when cached and the head's output is turned back by the query's position."""

    def __init__(self, mc, w, p, eps, layer, qk_norm, learned_sink, rot_values):
        self.H, self.G, self.dk, self.dv = int(mc["heads"]), int(mc["kv_heads"]), int(mc["dim"]), int(mc["vdim"])
        self.scale, self.eps, self.w, self.p, self.layer = float(mc["scale"]), eps, w, p, layer
        self.freqs = rotary_frequencies(mc["rot"])
        self.kv_from = mc.get("kv_from")
        self.qk_norm, self.learned_sink, self.rot_values = qk_norm, learned_sink, rot_values
        if rot_values:
            self.vfreqs = np.array([float(mc["rot"]["base"]) ** (-2.0 * m / self.dv) for m in range(self.dv // 2)])

    def step(self, h, pos, caches):
        w, p, H, G = self.w, self.p, self.H, self.G
        q = (w[p + "q"] @ h).reshape(H, self.dk)
        if self.qk_norm:
            q = rms_norm(q, self.eps) * w[p + "q.norm"]
        q = rotate_pairs(q, pos, self.freqs)
        if self.kv_from is None:
            k = (w[p + "k"] @ h).reshape(G, self.dk)
            v = (w[p + "v"] @ h).reshape(G, self.dv)
            if self.qk_norm:
                k = rms_norm(k, self.eps) * w[p + "k.norm"]
            k = rotate_pairs(k, pos, self.freqs)
            if self.rot_values:
                v = rotate_pairs(v, pos, self.vfreqs)
            ks, vs = caches.setdefault(self.layer, ([], []))
            ks.append(k)
            vs.append(v)
        else:
            ks, vs = caches[int(self.kv_from)]
        K, V = np.stack(ks), np.stack(vs)  # [n, G, d]
        out = np.zeros((H, self.dv))
        for hd in range(H):
            g = hd // (H // G)
            s = (K[:, g] @ q[hd]) * self.scale
            z = w[p + "sink"][hd] if self.learned_sink else 0.0
            m = max(float(s.max()), z)
            e = np.exp(s - m)
            out[hd] = (e @ V[:, g]) / (e.sum() + math.exp(z - m))
        if self.rot_values:
            out = rotate_pairs(out, pos, self.vfreqs, sign=-1.0)
        return w[p + "o"] @ out.reshape(-1)


class GatedDeltaRule:
    def __init__(self, mc, w, p, eps):
        self.H, self.G, self.dk, self.dv = int(mc["heads"]), int(mc["kv_heads"]), int(mc["dim"]), int(mc["vdim"])
        self.taps, self.eps, self.w, self.p = int(mc["conv"]), eps, w, p
        self.hq, self.hk, self.hv = [], [], []
        self.S = np.zeros((self.H, self.dk, self.dv))

    def _conv(self, hist, x, name):
        y = silu(causal_conv_step(hist, x, self.w[self.p + name + ".conv"], None, self.taps))
        hist.append(x)
        del hist[:max(0, len(hist) - (self.taps - 1))]
        return y

    def step(self, h, pos, caches):
        w, p, H, G, dk, dv = self.w, self.p, self.H, self.G, self.dk, self.dv
        q = self._conv(self.hq, w[p + "q"] @ h, "q").reshape(G, dk)
        k = self._conv(self.hk, w[p + "k"] @ h, "k").reshape(G, dk)
        v = self._conv(self.hv, w[p + "v"] @ h, "v").reshape(H, dv)
        q = q / np.sqrt((q * q).sum(-1, keepdims=True) + 1e-6) * dk ** -0.5
        k = k / np.sqrt((k * k).sum(-1, keepdims=True) + 1e-6)
        beta = sigmoid(w[p + "b"] @ h)
        decay = softplus(w[p + "a2"] @ (w[p + "a1"] @ h) + w[p + "dt_bias"]).reshape(H, dk)
        gate = sigmoid(w[p + "g2"] @ (w[p + "g1"] @ h)).reshape(H, dv)
        out = np.zeros((H, dv))
        for hd in range(H):
            g = hd // (H // G)
            a = np.exp(-math.exp(w[p + "A_log"][hd]) * decay[hd])  # one per key channel
            S = self.S[hd] * a[:, None]
            u = beta[hd] * (v[hd] - S.T @ k[g])
            S = S + np.outer(k[g], u)
            self.S[hd] = S
            out[hd] = S.T @ q[g]
        out = rms_norm(out, self.eps) * w[p + "norm"] * gate
        return w[p + "o"] @ out.reshape(-1)


class Parallel:
    def __init__(self, mc, w, p, eps, layer):
        self.left = Attention(mc["left"], w, p + "left.", eps, layer, qk_norm=False, learned_sink=True, rot_values=True)
        self.right = GatedDeltaRule(mc["right"], w, p + "right.", eps)
        self.ls, self.rs = float(mc["left_scale"]), float(mc["right_scale"])

    def step(self, h, pos, caches):
        return self.ls * self.left.step(h, pos, caches) + self.rs * self.right.step(h, pos, caches)


def feed_forward(h, w, p):
    return w[p + "down"] @ (silu(w[p + "gate"] @ h) * (w[p + "up"] @ h))


# ------------------------------------------------------------------------------------- the model
class Oracle:
    """One sequence's run through the model, token by token."""

    def __init__(self, cfg: dict, weights: dict):
        self.cfg = cfg
        self.w = {k: np.asarray(v, dtype=np.float64) for k, v in weights.items()}
        self.eps = float(cfg["norm"]["eps"])
        self.pos = 0
        self.caches: dict = {}
        self.mixers = []
        for i, l in enumerate(cfg["layers"]):
            p = f"l{i}.mix."
            if l["type"] == "mamba2":
                m = Mamba2(l["mixer"], self.w, p, self.eps)
            elif l["type"] == "attention":
                m = Attention(l["mixer"], self.w, p, self.eps, i, qk_norm=True, learned_sink=False, rot_values=False)
            elif l["type"] == "parallel":
                m = Parallel(l["mixer"], self.w, p, self.eps, i)
            else:
                raise ValueError(l["type"])
            self.mixers.append(m)

    def norm(self, x, name):
        return rms_norm(x, self.eps) * self.w[name]

    def step(self, token: int):
        w = self.w
        x = w["embed"][token] * float(self.cfg["embedding"]["scale"])
        streams = []
        for i, l in enumerate(self.cfg["layers"]):
            p = f"l{i}."
            x = x + self.norm(self.mixers[i].step(self.norm(x, p + "norm1"), self.pos, self.caches), p + "norm1b")
            if l.get("mlp"):
                x = x + self.norm(feed_forward(self.norm(x, p + "norm2"), w, p + "mlp."), p + "norm2b")
            streams.append(x.copy())
        self.pos += 1
        return w["head"] @ self.norm(x, "final.norm"), np.stack(streams)

    def run(self, tokens):
        """(logits [T, vocab], streams [layers, T, width]) of a whole sequence."""
        outs = [self.step(int(t)) for t in tokens]
        return np.stack([o[0] for o in outs]), np.stack([o[1] for o in outs], axis=1)
