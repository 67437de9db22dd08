"""Test helpers for the Mononex decoder: small configurations, random bfloat16-exact weights, checkpoints on disk."""
import numpy as np

from tests.korupel_util import bf16_round, tokens, write_checkpoint  # noqa: F401  (shared helpers, re-exported)


def layer(kind, mlp, **mx):
    return dict(type=kind, mixer=mx, mlp=mlp)


def attn(heads=4, kv_heads=2, dim=16, vdim=8, size=24, scale=None, kv_from=None):
    mx = dict(heads=heads, kv_heads=kv_heads, dim=dim, vdim=vdim, scale=dim ** -0.5 if scale is None else scale)
    if size is not None:
        mx["mask"] = dict(size=size)
    if kv_from is not None:
        mx["kv_from"] = kv_from
    return mx


def latent(heads=3, dim=8, rot_dim=12, vdim=20, kv_rank=24, q_rank=40, scale=0.2, base=10000.0, dims=None, scaling="default"):
    if scaling == "default":
        scaling = dict(factor=4.0, original=64, fast=16.0, slow=2.0)
    rot = dict(base=base, dims=rot_dim if dims is None else dims)
    if scaling is not None:
        rot["scaling"] = scaling
    return dict(heads=heads, dim=dim, rot_dim=rot_dim, vdim=vdim, kv_rank=kv_rank, q_rank=q_rank, scale=scale, rot=rot)


def gla(heads=2, dim=8, vdim=24, tau=4.0):
    return dict(heads=heads, dim=dim, vdim=vdim, tau=tau)


def dense(ff=40):
    return dict(kind="dense", ff=ff)


def config(layers, vocab=61, width=48, eps=2e-6):
    return dict(architecture="Mononex", vocab=vocab, width=width, norm=dict(eps=eps), layers=layers)


def small_config():
    """Every kind of mixer, a layer that borrows keys and values from one that is not its neighbour, a layer without a
    feed-forward; sizes that are neither equal to each other nor powers of two."""
    return config([layer("gla", dense(36), **gla(heads=3, dim=8, vdim=12, tau=2.5)),
                   layer("attention", dense(28), **attn(heads=6, kv_heads=2, dim=12, vdim=20, size=21, scale=0.3)),
                   layer("latent_attention", None, **latent()),
                   layer("attention", dense(44), **attn(heads=4, kv_heads=2, dim=12, vdim=20, size=33, scale=0.2, kv_from=1)),
                   layer("gla", None, **gla(heads=2, dim=20, vdim=8, tau=9.0)),
                   layer("latent_attention", dense(24), **latent(heads=2, dim=12, rot_dim=8, vdim=16, kv_rank=20, q_rank=28, scale=0.15,
                                                                 base=500.0, scaling=None))],
                  vocab=83, width=56)


def random_weights(cfg, seed=0, a_rank=6):
    """name -> float32 array (bfloat16-exact), in the checkpoint's spelling and shapes."""
    rs = np.random.RandomState(seed)
    W, V = cfg["width"], cfg["vocab"]
    P = {}

    def mat(name, o, i, s=None):
        P[name] = bf16_round(rs.randn(o, i) * (s if s is not None else i ** -0.5))

    def vec(name, n, s=0.1, off=0.0):
        P[name] = bf16_round(off + s * rs.randn(n))

    mat("embed", V, W, 1.0)
    for li, ly in enumerate(cfg["layers"]):
        p, mx = f"l{li}.", ly["mixer"]
        vec(p + "norm1", W)
        P[p + "shift"] = bf16_round(rs.rand(W))
        H, d, e = mx["heads"], mx["dim"], mx["vdim"]
        if ly["type"] == "attention":
            G = mx["kv_heads"]
            mat(p + "mix.q", H * d, W, 2.0 * W ** -0.5)
            if mx.get("kv_from") is None:
                mat(p + "mix.k", G * d, W, 2.0 * W ** -0.5)
                mat(p + "mix.v", G * e, W)
            vec(p + "mix.sink", H, 1.0, 0.5)
            mat(p + "mix.g", H * e, W)
            mat(p + "mix.o", W, H * e)
        elif ly["type"] == "latent_attention":
            r, R, Q = mx["rot_dim"], mx["kv_rank"], mx["q_rank"]
            mat(p + "mix.dq", Q, W); vec(p + "mix.dq.norm", Q, 0.1, 1.0)
            mat(p + "mix.uq", H * (d + r), Q, 2.0 * Q ** -0.5)
            mat(p + "mix.dkv", R + r, W, 2.0 * W ** -0.5); vec(p + "mix.dkv.norm", R, 0.1, 1.0)
            mat(p + "mix.uk", H * d, R, 2.0 * R ** -0.5)
            mat(p + "mix.uv", H * e, R)
            mat(p + "mix.g", H * e, W)
            mat(p + "mix.o", W, H * e)
        else:
            mat(p + "mix.q", H * d, W); mat(p + "mix.k", H * d, W); mat(p + "mix.v", H * e, W); mat(p + "mix.g", H * e, W)
            mat(p + "mix.a1", a_rank, W); mat(p + "mix.a2", H * d, a_rank, 2.0 * a_rank ** -0.5)
            vec(p + "mix.a2.b", H * d, 1.0, 1.0)
            vec(p + "mix.norm", e, 0.1, 1.0)
            mat(p + "mix.o", W, H * e)
        if ly.get("mlp") is not None:
            vec(p + "norm2", W)
            mat(p + "mlp.up", ly["mlp"]["ff"], W); mat(p + "mlp.down", W, ly["mlp"]["ff"])
    vec("final.norm", W)
    mat("head", V, W)
    return P
