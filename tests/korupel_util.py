"""Test helpers for the Korupel decoder: small configurations, random bfloat16-exact weights, checkpoints on disk."""
import json
import os
import struct

import numpy as np


def bf16_round(a):
    """Round-to-nearest-even to bfloat16, returned as float32 (so the oracle and the checkpoint hold the same numbers)."""
    u = np.ascontiguousarray(a, np.float32).view(np.uint32).astype(np.uint64)
    u = (u + 0x7FFF + ((u >> 16) & 1)) & 0xFFFF0000
    return u.astype(np.uint32).view(np.float32)


def layer(kind, mlp, **mx):
    return dict(type=kind, mixer=mx, mlp=mlp)


def attn(heads=2, kv_heads=1, dim=16, size=12, keep_first=2, scale=None):
    return dict(heads=heads, kv_heads=kv_heads, dim=dim, vdim=dim, scale=dim ** -0.5 if scale is None else scale,
                mask=dict(size=size, keep_first=keep_first))


def light(heads=2, dim=8, vdim=16, decay=(0.7, 0.98)):
    return dict(heads=heads, dim=dim, vdim=vdim, decay=list(decay))


DENSE = dict(kind="dense", ff=40)


def moe(experts=4, top=2, ff=24):
    return dict(kind="moe", expert=dict(ff=ff), router=dict(experts=experts, top=top))


def config(layers, vocab=61, width=48, taps=3, mult=0.4, eps=1e-6):
    return dict(architecture="Korupel", vocab=vocab, width=width, residual_mult=mult, norm=dict(eps=eps), canon=dict(taps=taps),
                layers=layers)


def small_config():
    """Four layers, every kind of mixer and feed-forward, sizes that are neither equal to each other nor powers of two."""
    return config([layer("attention", DENSE, **attn(heads=4, kv_heads=2, dim=16, size=20, keep_first=3)),
                   layer("lightning", moe(experts=5, top=2, ff=24), **light(heads=3, dim=8, vdim=24, decay=(0.5, 0.9, 0.995))),
                   layer("lightning", DENSE, **light(heads=2, dim=24, vdim=8, decay=(0.8, 0.99))),
                   layer("attention", moe(experts=3, top=3, ff=16), **attn(heads=3, kv_heads=3, dim=24, size=33, keep_first=0, scale=0.3))],
                  vocab=83, width=56, taps=5, mult=0.25, eps=2e-6)


def random_weights(cfg, seed=0):
    """name -> float32 array (bfloat16-exact), in the checkpoint's spelling and shapes."""
    rs = np.random.RandomState(seed)
    W, V, taps = cfg["width"], cfg["vocab"], cfg["canon"]["taps"]
    P = {}

    def mat(name, o, i, s=None):
        P[name] = bf16_round(rs.randn(o, i) * (s if s is not None else i ** -0.5))

    def vec(name, n, s=0.1, off=1.0):
        P[name] = bf16_round(off + s * rs.randn(n))

    mat("embed", V, W, 1.0)
    for li, ly in enumerate(cfg["layers"]):
        p = f"l{li}."
        mx = ly["mixer"]
        vec(p + "norm1", W); vec(p + "norm1b", W)
        P[p + "canon1"] = bf16_round(0.3 * rs.randn(W, taps))
        H, d = mx["heads"], mx["dim"]
        if ly["type"] == "attention":
            G = mx["kv_heads"]
            mat(p + "mix.q", H * d, W, 2.0 * W ** -0.5); vec(p + "mix.q.b", H * d, 0.3, 0.0)
            mat(p + "mix.k", G * d, W, 2.0 * W ** -0.5); vec(p + "mix.k.b", G * d, 0.3, 0.0)
            mat(p + "mix.g", H, W)
            P[p + "mix.r1"] = bf16_round(0.2 + 0.5 * rs.rand(H))
            P[p + "mix.r2"] = bf16_round(0.1 + rs.rand(H))
            mat(p + "mix.o", W, H * d)
        else:
            e = mx["vdim"]
            mat(p + "mix.q", H * d, W); mat(p + "mix.k", H * d, W); mat(p + "mix.v", H * e, W); mat(p + "mix.g", H * e, W)
            vec(p + "mix.norm", H * e)
            mat(p + "mix.o", W, H * e)
        ml = ly.get("mlp")
        if ml is not None:
            vec(p + "norm2", W); vec(p + "norm2b", W)
            P[p + "canon2"] = bf16_round(0.3 * rs.randn(W, taps))
            if ml["kind"] == "dense":
                mat(p + "mlp.gate", ml["ff"], W); mat(p + "mlp.up", ml["ff"], W); mat(p + "mlp.down", W, ml["ff"])
            else:
                ff = ml["expert"]["ff"]
                for ex in range(ml["router"]["experts"]):
                    mat(f"{p}mlp.e{ex}.gate", ff, W); mat(f"{p}mlp.e{ex}.up", ff, W); mat(f"{p}mlp.e{ex}.down", W, ff)
                mat(p + "mlp.router", ml["router"]["experts"], W, 2.0 * W ** -0.5)
    vec("final.norm", W)
    mat("head", V, W)
    return P


def write_checkpoint(path, cfg, P):
    """config.json + model.safetensors (bfloat16) in `path`."""
    os.makedirs(path, exist_ok=True)
    with open(os.path.join(path, "config.json"), "w") as f:
        json.dump(cfg, f)
    header, blobs, off = {}, [], 0
    for name, a in P.items():
        b = (np.ascontiguousarray(a, np.float32).view(np.uint32) >> 16).astype("<u2").tobytes()
        header[name] = dict(dtype="BF16", shape=list(a.shape), data_offsets=[off, off + len(b)])
        blobs.append(b)
        off += len(b)
    hj = json.dumps(header).encode()
    hj += b" " * (-len(hj) % 8)
    with open(os.path.join(path, "model.safetensors"), "wb") as f:
        f.write(struct.pack("<Q", len(hj)) + hj + b"".join(blobs))
    return path


def tokens(n, vocab, seed=0, avoid=()):
    rs = np.random.RandomState(1000 + seed)
    out = []
    while len(out) < n:
        t = int(rs.randint(vocab))
        if t not in avoid:
            out.append(t)
    return out
