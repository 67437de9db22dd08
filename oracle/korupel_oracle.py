"""Plain NumPy statement of the Korupel decoder, one function per mechanism (float64, whole sequences, no cache).

Test infrastructure only: nothing here is imported by the product.  A model is a config dict in the checkpoint's own
spelling (``architecture``, ``width``, ``vocab``, ``residual_mult``, ``norm.eps``, ``canon.taps``, ``layers[...]``) and a dict
of arrays under the checkpoint's tensor names (``embed``, ``l<i>.norm1``, ``l<i>.mix.q``, ..., ``final.norm``, ``head``).

Notation: T tokens, W model width; for a mixer H query heads, G key/value heads, d head size, e value size.
"""
from __future__ import annotations

import numpy as np


def rms_norm(x, w, eps):
    """y = x / sqrt(mean(x^2) + eps) * w over the last axis."""
    x = np.asarray(x, np.float64)
    return x / np.sqrt((x * x).mean(-1, keepdims=True) + eps) * np.asarray(w, np.float64)


def sigmoid(z):
    return 1.0 / (1.0 + np.exp(-np.asarray(z, np.float64)))


def silu(z):
    return z * sigmoid(z)


def gelu_tanh(z):
    return 0.5 * z * (1.0 + np.tanh(np.sqrt(2.0 / np.pi) * (z + 0.044715 * z ** 3)))


def short_conv_residual(h, w):
    """h[t] + sum_j w[:, j] * h[t - taps + 1 + j] per channel, zeros before the first token.  h: [T, W], w: [W, taps]."""
    T, taps = h.shape[0], w.shape[1]
    out = h.copy()
    for t in range(T):
        for j in range(taps):
            s = t - taps + 1 + j
            if s >= 0:
                out[t] += w[:, j] * h[s]
    return out


def visible(i, j, size, keep_first):
    """Sliding window of `size` positions that also keeps the first `keep_first` positions of the sequence."""
    return j <= i and (i - j < size or j < keep_first)


def window_attention(h, P, pre, mx):
    """Softmax attention whose values are its keys, with a logarithmic distance penalty and one sigmoid gate per head."""
    H, G, d = mx["heads"], mx["kv_heads"], mx["dim"]
    size, keep = mx["mask"]["size"], mx["mask"]["keep_first"]
    T = h.shape[0]
    q = (h @ P[pre + "q"].T + P[pre + "q.b"]).reshape(T, H, d)
    k = (h @ P[pre + "k"].T + P[pre + "k.b"]).reshape(T, G, d)
    gate = sigmoid(h @ P[pre + "g"].T)                       # [T, H]
    r1, r2 = P[pre + "r1"], P[pre + "r2"]
    out = np.zeros((T, H, d))
    for hd in range(H):
        kv = hd // (H // G)
        for i in range(T):
            js = [j for j in range(i + 1) if visible(i, j, size, keep)]
            dist = np.array([i - j for j in js], np.float64)
            s = k[js, kv] @ q[i, hd] * mx["scale"] - r1[hd] * np.log1p(r2[hd] * dist)
            p = np.exp(s - s.max())
            p /= p.sum()
            out[i, hd] = (p[:, None] * k[js, kv]).sum(0) * gate[i, hd]
    return out.reshape(T, H * d) @ P[pre + "o"].T


def lightning_attention(h, P, pre, mx, eps):
    """Per head S_t = decay * S_{t-1} + k_t v_t^T, o_t = S_t^T q_t; the heads are normed together, gated and projected."""
    H, d, e = mx["heads"], mx["dim"], mx["vdim"]
    T = h.shape[0]
    q = silu(h @ P[pre + "q"].T).reshape(T, H, d)
    k = silu(h @ P[pre + "k"].T).reshape(T, H, d)
    v = silu(h @ P[pre + "v"].T).reshape(T, H, e)
    o = np.zeros((T, H, e))
    for hd in range(H):
        S = np.zeros((d, e))
        for t in range(T):
            S = mx["decay"][hd] * S + np.outer(k[t, hd], v[t, hd])
            o[t, hd] = S.T @ q[t, hd]
    y = rms_norm(o.reshape(T, H * e), P[pre + "norm"], eps) * sigmoid(h @ P[pre + "g"].T)
    return y @ P[pre + "o"].T


def dense_ff(h, P, pre):
    return (gelu_tanh(h @ P[pre + "gate"].T) * (h @ P[pre + "up"].T)) @ P[pre + "down"].T


def moe_ff(h, P, pre, mlp):
    """Sigmoid router; the `top` largest scores choose the experts and weigh them as they are (no renormalisation)."""
    E, top = mlp["router"]["experts"], mlp["router"]["top"]
    s = sigmoid(h @ P[pre + "router"].T)                     # [T, E]
    out = np.zeros((h.shape[0], P[pre + "e0.down"].shape[0]))
    for t in range(h.shape[0]):
        for ex in np.argsort(-s[t], kind="stable")[:top]:
            p = f"{pre}e{ex}."
            out[t] += s[t, ex] * ((silu(h[t] @ P[p + "gate"].T) * (h[t] @ P[p + "up"].T)) @ P[p + "down"].T)
    assert E == s.shape[1]
    return out


def forward(cfg, P, tokens, return_layers=False):
    """Logits [T, vocab] of one whole sequence (and the residual stream after every layer)."""
    P = {k: np.asarray(v, np.float64) for k, v in P.items()}
    eps, m = cfg["norm"]["eps"], cfg["residual_mult"]
    x = P["embed"][np.asarray(tokens, np.int64)]
    layers = []
    for i, ly in enumerate(cfg["layers"]):
        p = f"l{i}."
        h = short_conv_residual(rms_norm(x, P[p + "norm1"], eps), P[p + "canon1"])
        if ly["type"] == "attention":
            y = window_attention(h, P, p + "mix.", ly["mixer"])
        elif ly["type"] == "lightning":
            y = lightning_attention(h, P, p + "mix.", ly["mixer"], eps)
        else:
            raise ValueError(ly["type"])
        x = x + m * rms_norm(y, P[p + "norm1b"], eps)
        if ly.get("mlp") is not None:
            h = short_conv_residual(rms_norm(x, P[p + "norm2"], eps), P[p + "canon2"])
            y = dense_ff(h, P, p + "mlp.") if ly["mlp"]["kind"] == "dense" else moe_ff(h, P, p + "mlp.", ly["mlp"])
            x = x + m * rms_norm(y, P[p + "norm2b"], eps)
        layers.append(x.copy())
    logits = rms_norm(x, P["final.norm"], eps) @ P["head"].T
    return (logits, np.stack(layers)) if return_layers else logits


def generate(cfg, P, prompt, n_new):
    """Greedy continuation by recomputing the whole sequence for every token (lowest index wins a tie)."""
    toks = list(prompt)
    for _ in range(n_new):
        toks.append(int(np.argmax(forward(cfg, P, toks)[-1])))
    return toks
