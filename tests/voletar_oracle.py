"""Plain, slow oracle of the Voletar design, one function per mechanism, written token by token from
the design's equations in float64.  It shares no code with mxserve: the tests compare the engine
(paged cache, state slots, chunked steps, HIP kernels) against it.

Notation: W is the model width, h the input of a mixer (the normed residual), per-head tensors are
laid out head by head.  `w` maps tensor names ("l0.mix.q", ...) to float64 arrays.
"""
from __future__ import annotations

import math

import numpy as np


def rms(x: np.ndarray, eps: float) -> np.ndarray:
    """x over its root mean square, eps inside the root (last axis)."""
    return x / np.sqrt(np.mean(x * x, axis=-1, keepdims=True) + eps)


def silu(z):
    return z / (1.0 + np.exp(-z))


def sigmoid(z):
    return 1.0 / (1.0 + np.exp(-z))


def logsigmoid(z):
    return -np.logaddexp(0.0, -z)


def lightning_mixer(h: np.ndarray, w: dict, p: str, mc: dict, eps: float) -> np.ndarray:
    """Linear attention with a fixed per-head decay: S_t = a S_(t-1) + k_t v_t^T, o_t = S_t^T q_t."""
    T = h.shape[0]
    H, D, V = mc["heads"], mc["dim"], mc["vdim"]
    q = silu(h @ w[p + "q"].T).reshape(T, H, D)
    k = silu(h @ w[p + "k"].T).reshape(T, H, D)
    v = silu(h @ w[p + "v"].T).reshape(T, H, V)
    o = np.zeros((T, H, V))
    for hd in range(H):
        a = float(mc["decay"][hd])
        S = np.zeros((D, V))
        for t in range(T):
            S = a * S + np.outer(k[t, hd], v[t, hd])
            o[t, hd] = S.T @ q[t, hd]
    y = rms(o.reshape(T, H * V), eps) * w[p + "norm"]
    y = y * sigmoid(h @ w[p + "g"].T)
    return y @ w[p + "o"].T


def window_attention(h: np.ndarray, w: dict, p: str, mc: dict) -> np.ndarray:
    """Softmax attention without positions: query i sees key j <= i when i - j < size or j < keep_first."""
    T = h.shape[0]
    H, G, D, V = mc["heads"], mc["kv_heads"], mc["dim"], mc["vdim"]
    size, keep = mc["mask"]["size"], mc["mask"]["keep_first"]
    q = (h @ w[p + "q"].T).reshape(T, H, D)
    k = (h @ w[p + "k"].T).reshape(T, G, D)
    v = (h @ w[p + "v"].T).reshape(T, G, V)
    o = np.zeros((T, H, V))
    for i in range(T):
        js = [j for j in range(i + 1) if i - j < size or j < keep]
        for hd in range(H):
            g = hd // (H // G)
            s = np.array([q[i, hd] @ k[j, g] for j in js]) * mc["scale"]
            e = np.exp(s - s.max())
            pr = e / e.sum()
            o[i, hd] = sum(pr[n] * v[j, g] for n, j in enumerate(js))
    return o.reshape(T, H * V) @ w[p + "o"].T


def mlstm_mixer(h: np.ndarray, w: dict, p: str, mc: dict, eps: float) -> np.ndarray:
    """Matrix memory with exponential gates and a running maximum m (m_0 = 0)."""
    T = h.shape[0]
    H, D, V, cap = mc["heads"], mc["dim"], mc["vdim"], mc["gate_cap"]
    q = (h @ w[p + "q"].T).reshape(T, H, D) * D ** -0.5
    k = (h @ w[p + "k"].T).reshape(T, H, D)
    v = (h @ w[p + "v"].T).reshape(T, H, V)
    ig = cap * np.tanh((h @ w[p + "i"].T + w[p + "i.b"]) / cap)
    fg = logsigmoid(cap * np.tanh((h @ w[p + "f"].T + w[p + "f.b"]) / cap))
    o = np.zeros((T, H, V))
    for hd in range(H):
        S, n, m = np.zeros((D, V)), np.zeros(D), 0.0
        for t in range(T):
            m_new = max(fg[t, hd] + m, ig[t, hd])
            fa, ia = math.exp(fg[t, hd] + m - m_new), math.exp(ig[t, hd] - m_new)
            S = fa * S + ia * np.outer(k[t, hd], v[t, hd])
            n = fa * n + ia * k[t, hd]
            m = m_new
            den = max(abs(n @ q[t, hd]), math.exp(-m)) + 1e-6
            o[t, hd] = (S.T @ q[t, hd]) / den
    y = rms(o, eps).reshape(T, H * V) * w[p + "norm"]
    y = y * sigmoid(h @ w[p + "g"].T)
    return y @ w[p + "o"].T


def parallel_mixer(h: np.ndarray, w: dict, p: str, mc: dict, eps: float) -> np.ndarray:
    """Window attention beside the matrix memory; each output normed over the width, then averaged."""
    a = window_attention(h, w, p + "left.", mc["left"])
    b = mlstm_mixer(h, w, p + "right.", mc["right"], eps)
    return 0.5 * (rms(a, eps) * w[p + "left.out"] + rms(b, eps) * w[p + "right.out"])


def dense_ff(h: np.ndarray, w: dict, p: str) -> np.ndarray:
    return np.square(np.maximum(h @ w[p + "up"].T, 0.0)) @ w[p + "down"].T


def layer(x: np.ndarray, w: dict, i: int, lc: dict, eps: float) -> np.ndarray:
    p = f"l{i}."
    h = rms(x, eps) * w[p + "norm1"]
    if lc["type"] == "lightning":
        x = x + lightning_mixer(h, w, p + "mix.", lc["mixer"], eps)
    elif lc["type"] == "parallel":
        x = x + parallel_mixer(h, w, p + "mix.", lc["mixer"], eps)
    else:
        raise ValueError(lc["type"])
    if lc.get("mlp") is not None:
        x = x + dense_ff(rms(x, eps) * w[p + "norm2"], w, p + "mlp.")
    return x


def layer_runs(cfg: dict) -> list:
    """(layer, pass) in execution order; pass is None outside the loop."""
    n = len(cfg["layers"])
    loop = cfg.get("loop")
    if not loop:
        return [(i, None) for i in range(n)]
    runs = [(i, None) for i in range(loop["start"])]
    for t in range(loop["times"]):
        runs += [(i, t) for i in range(loop["start"], loop["stop"])]
    return runs + [(i, None) for i in range(loop["stop"], n)]


def forward(cfg: dict, w: dict, tokens, trace: list | None = None) -> np.ndarray:
    """Logits [T, vocab] of one sequence.  `trace` collects the residual stream after every layer run."""
    eps = cfg["norm"]["eps"]
    x0 = w["embed"][np.asarray(tokens)]
    x = x0
    loop = cfg.get("loop")
    for i, t in layer_runs(cfg):
        if t is not None and i == loop["start"]:
            x = np.concatenate([x, x0], axis=-1) @ w["loop.in"].T + w["loop.step"][t]
        x = layer(x, w, i, cfg["layers"][i], eps)
        if trace is not None:
            trace.append(x.copy())
    y = (rms(x, eps) * w["final.norm"]) @ w["head"].T
    cap = cfg.get("logit_softcap")
    return cap * np.tanh(y / cap) if cap else y
