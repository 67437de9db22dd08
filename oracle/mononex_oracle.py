"""Plain NumPy statement of the Mononex decoder, one function per mechanism (float64, whole sequences, no cache).

Test infrastructure only: nothing here is imported by the product.  A model is a config dict in the checkpoint's own
spelling (``architecture``, ``width``, ``vocab``, ``norm.eps``, ``layers[...]``) and a dict of arrays under the checkpoint's
tensor names (``embed``, ``l<i>.norm1``, ``l<i>.shift``, ``l<i>.mix.q``, ..., ``final.norm``, ``head``).

Notation: T tokens, W model width; for a mixer H query heads, G key/value heads, d key size, r rotated key size, e value
size, R latent size.
"""
from __future__ import annotations

import math

import numpy as np


def unit_rms(x, eps):
    """x / sqrt(mean(x^2) + eps) over the last axis."""
    x = np.asarray(x, np.float64)
    return x / np.sqrt((x * x).mean(-1, keepdims=True) + eps)


def norm_around_zero(x, w, eps):
    """Norm of the layers and of the output: the stored weight is the distance of the factor from one."""
    return unit_rms(x, eps) * (1.0 + np.asarray(w, np.float64))


def norm_plain(x, w, eps):
    return unit_rms(x, eps) * np.asarray(w, np.float64)


def sigmoid(z):
    return 1.0 / (1.0 + np.exp(-np.asarray(z, np.float64)))


def silu(z):
    return z * sigmoid(z)


def token_shift(h, s):
    """Row t moves towards row t - 1 by the fraction s per channel; the row before the first is zero."""
    before = np.zeros_like(h)
    before[1:] = h[:-1]
    return h + (before - h) * s


def squared_relu_ff(h, P, pre):
    return (np.maximum(h @ P[pre + "up"].T, 0.0) ** 2) @ P[pre + "down"].T


# ---- rotation -------------------------------------------------------------------------------------------------------
def rotation_tables(rot, n_pos):
    """cos / sin [n_pos, dims / 2] of the angle position * frequency, with the YaRN blend and magnitude when asked for."""
    dims, base = rot["dims"], rot["base"]
    f = np.array([base ** (-2.0 * i / dims) for i in range(dims // 2)])
    mag = 1.0
    sc = rot.get("scaling")
    if sc:
        def pair_of(turns):          # the pair index whose wavelength fits `turns` times into the original length
            return dims * math.log(sc["original"] / (2 * math.pi * turns)) / (2 * math.log(base))
        lo = max(math.floor(pair_of(sc["fast"])), 0)
        hi = min(math.ceil(pair_of(sc["slow"])), dims - 1)
        ramp = np.clip((np.arange(dims // 2) - lo) / max(hi - lo, 0.001), 0.0, 1.0)
        f = f / sc["factor"] * ramp + f * (1.0 - ramp)
        mag = 0.1 * math.log(sc["factor"]) + 1.0
    ang = np.arange(n_pos)[:, None] * f[None, :]
    return np.cos(ang) * mag, np.sin(ang) * mag


def rotate_pairs(x, cos, sin, dims):
    """x: [T, ..., n]; elements (2i, 2i + 1), 2i + 1 < dims, of row t turn by the angle of position t; the rest stay."""
    out = np.array(x, np.float64)
    shape = (x.shape[0],) + (1,) * (x.ndim - 2) + (dims // 2,)
    c, s = cos[:x.shape[0]].reshape(shape), sin[:x.shape[0]].reshape(shape)
    a, b = x[..., 0:dims:2], x[..., 1:dims:2]
    out[..., 0:dims:2] = a * c - b * s
    out[..., 1:dims:2] = b * c + a * s
    return out


# ---- mixers ---------------------------------------------------------------------------------------------------------
def same_block(i, j, size):
    """Causal, and only inside the block of `size` positions that holds i (size None: causal alone)."""
    return j <= i and (size is None or i // size == j // size)


def head_slope(h, H):
    return 2.0 ** (-8.0 * (h + 1) / H)


def keys_and_values(h, P, pre, mx):
    T = h.shape[0]
    return ((h @ P[pre + "k"].T).reshape(T, mx["kv_heads"], mx["dim"]), (h @ P[pre + "v"].T).reshape(T, mx["kv_heads"], mx["vdim"]))


def block_attention(h, P, pre, mx, k, v):
    """Softmax attention inside position blocks: score - slope * distance, a sink in the denominator, a sigmoid gate per
    output element.  k, v come from this layer's projections or from the layer it borrows them from."""
    H, G, d, e = mx["heads"], mx["kv_heads"], mx["dim"], mx["vdim"]
    T = h.shape[0]
    size = (mx.get("mask") or {}).get("size")
    q = (h @ P[pre + "q"].T).reshape(T, H, d)
    out = np.zeros((T, H, e))
    for hd in range(H):
        g = hd // (H // G)
        for i in range(T):
            js = [j for j in range(i + 1) if same_block(i, j, size)]
            s = k[js, g] @ q[i, hd] * mx["scale"] - head_slope(hd, H) * (i - np.array(js, np.float64))
            sink = P[pre + "sink"][hd]
            top = max(s.max(), sink)
            p = np.exp(s - top)
            out[i, hd] = (p[:, None] * v[js, g]).sum(0) / (p.sum() + math.exp(sink - top))
    return (out.reshape(T, H * e) * sigmoid(h @ P[pre + "g"].T)) @ P[pre + "o"].T


def latent_attention(h, P, pre, mx, eps):
    """Queries through a normed latent; per token one normed latent (keys and values of every head are products of it) and
    one rotated key part that all heads share; causal softmax; sigmoid gate per output element."""
    H, d, r, e, R = mx["heads"], mx["dim"], mx["rot_dim"], mx["vdim"], mx["kv_rank"]
    T = h.shape[0]
    q = (norm_plain(h @ P[pre + "dq"].T, P[pre + "dq.norm"], eps) @ P[pre + "uq"].T).reshape(T, H, d + r)
    low = h @ P[pre + "dkv"].T
    c = norm_plain(low[:, :R], P[pre + "dkv.norm"], eps)
    dims = mx["rot"]["dims"]
    cos, sin = rotation_tables(mx["rot"], T)
    q_plain, q_rot = q[..., :d], rotate_pairs(q[..., d:], cos, sin, dims)
    k_rot = rotate_pairs(low[:, R:], cos, sin, dims)
    k_plain = (c @ P[pre + "uk"].T).reshape(T, H, d)
    v = (c @ P[pre + "uv"].T).reshape(T, H, e)
    out = np.zeros((T, H, e))
    for hd in range(H):
        for i in range(T):
            s = (k_plain[:i + 1, hd] @ q_plain[i, hd] + k_rot[:i + 1] @ q_rot[i, hd]) * mx["scale"]
            p = np.exp(s - s.max())
            out[i, hd] = (p[:, None] * v[:i + 1, hd]).sum(0) / p.sum()
    return (out.reshape(T, H * e) * sigmoid(h @ P[pre + "g"].T)) @ P[pre + "o"].T


def gated_linear_attention(h, P, pre, mx, eps):
    """Per head S_t = diag(a_t) S_(t-1) + k_t v_t^T with a decay a_t in (0, 1) per key channel, o_t = S_t^T q_t; every head's
    output normed over its e values, times silu(gate), projected."""
    H, d, e = mx["heads"], mx["dim"], mx["vdim"]
    T = h.shape[0]
    q = (h @ P[pre + "q"].T).reshape(T, H, d) * d ** -0.5
    k = (h @ P[pre + "k"].T).reshape(T, H, d)
    v = (h @ P[pre + "v"].T).reshape(T, H, e)
    a = (sigmoid((h @ P[pre + "a1"].T) @ P[pre + "a2"].T + P[pre + "a2.b"]) ** (1.0 / mx["tau"])).reshape(T, H, d)
    o = np.zeros((T, H, e))
    for hd in range(H):
        S = np.zeros((d, e))
        for t in range(T):
            S = a[t, hd][:, None] * S + np.outer(k[t, hd], v[t, hd])
            o[t, hd] = S.T @ q[t, hd]
    o = norm_plain(o, P[pre + "norm"], eps)
    return (o.reshape(T, H * e) * silu(h @ P[pre + "g"].T)) @ P[pre + "o"].T


# ---- the model ------------------------------------------------------------------------------------------------------
def forward(cfg, P, tokens, return_layers=False):
    """Logits [T, vocab] of one whole sequence (and the residual stream after every layer)."""
    P = {k: np.asarray(v, np.float64) for k, v in P.items()}
    eps = cfg["norm"]["eps"]
    x = P["embed"][np.asarray(tokens, np.int64)]
    layers, kv = [], {}
    for i, ly in enumerate(cfg["layers"]):
        p, mx = f"l{i}.", ly["mixer"]
        h = token_shift(norm_around_zero(x, P[p + "norm1"], eps), P[p + "shift"])
        if ly["type"] == "attention":
            if mx.get("kv_from") is None:
                kv[i] = keys_and_values(h, P, p + "mix.", mx)
            y = block_attention(h, P, p + "mix.", mx, *kv[i if mx.get("kv_from") is None else mx["kv_from"]])
        elif ly["type"] == "latent_attention":
            y = latent_attention(h, P, p + "mix.", mx, eps)
        elif ly["type"] == "gla":
            y = gated_linear_attention(h, P, p + "mix.", mx, eps)
        else:
            raise ValueError(ly["type"])
        if ly.get("mlp") is not None:
            y = y + squared_relu_ff(norm_around_zero(x, P[p + "norm2"], eps), P, p + "mlp.")
        x = x + y
        layers.append(x.copy())
    logits = norm_around_zero(x, P["final.norm"], eps) @ P["head"].T
    return (logits, np.stack(layers)) if return_layers else logits


def generate(cfg, P, prompt, n_new):
    """Greedy continuation by recomputing the whole sequence for every token (lowest index wins a tie)."""
    toks = list(prompt)
    for _ in range(n_new):
        toks.append(int(np.argmax(forward(cfg, P, toks)[-1])))
    return toks
