"""CPU: the NumPy statement of the Mononex decoder (oracle/mononex_oracle.py) pinned on closed forms and on second, independent
spellings of its mechanisms -- it is the yardstick of tests/test_gpu_mononex.py."""
import math

import numpy as np

from oracle import mononex_oracle as O
from tests import mononex_util as U


def test_norms_and_token_shift():
    x = np.array([[3.0, -4.0, 0.0, 0.0]])
    assert np.allclose(O.unit_rms(x, 0.0), x / 2.5)
    assert np.allclose(O.norm_around_zero(x, np.zeros(4), 0.0), O.norm_plain(x, np.ones(4), 0.0))
    assert np.allclose(O.norm_around_zero(x, np.full(4, 0.5), 0.0), 1.5 * x / 2.5)
    assert abs(O.unit_rms(np.zeros((1, 4)), 1e-4)).max() == 0.0                      # eps sits inside the root
    h = np.arange(12.0).reshape(4, 3)
    assert np.array_equal(O.token_shift(h, np.zeros(3)), h)
    assert np.array_equal(O.token_shift(h, np.ones(3))[1:], h[:-1]) and not O.token_shift(h, np.ones(3))[0].any()
    s = np.array([0.25, 0.5, 1.0])
    assert np.allclose(O.token_shift(h, s)[2], (1 - s) * h[2] + s * h[1])


def test_rotation_depends_on_distance_only_and_yarn_blends_frequencies():
    rs = np.random.RandomState(0)
    rot = dict(base=100.0, dims=6)
    cos, sin = O.rotation_tables(rot, 50)
    assert np.allclose(cos[7, 2], math.cos(7 * 100.0 ** (-4 / 6)))
    q, k = rs.randn(8), rs.randn(8)
    rq = O.rotate_pairs(np.tile(q, (50, 1)), cos, sin, 6)
    rk = O.rotate_pairs(np.tile(k, (50, 1)), cos, sin, 6)
    assert np.allclose(rq[:, 6:], q[6:])                                             # past rot.dims nothing turns
    assert np.allclose(rq[30] @ rk[10], rq[25] @ rk[5]) and not np.allclose(rq[30] @ rk[10], rq[30] @ rk[11])
    assert np.allclose(rq[3, 0], q[0] * cos[3, 0] - q[1] * sin[3, 0]) and np.allclose(rq[3, 1], q[1] * cos[3, 0] + q[0] * sin[3, 0])
    # factor 1 changes nothing; otherwise fast pairs keep their frequency, slow pairs are stretched, between them a ramp
    c1, _ = O.rotation_tables(dict(rot, scaling=dict(factor=1.0, original=40, fast=8.0, slow=1.0)), 50)
    assert np.allclose(c1, cos)
    sc = dict(factor=4.0, original=40, fast=8.0, slow=1.0)
    rot = dict(base=10000.0, dims=16, scaling=sc)
    c4, s4 = O.rotation_tables(rot, 2)
    mag = 0.1 * math.log(4.0) + 1.0
    f = np.arctan2(s4[1], c4[1])
    plain = np.array([10000.0 ** (-2 * i / 16) for i in range(8)])
    pair = lambda t: 16 * math.log(40 / (2 * math.pi * t)) / (2 * math.log(10000.0))
    lo, hi = max(math.floor(pair(8.0)), 0), min(math.ceil(pair(1.0)), 15)
    assert 0 <= lo < hi < 8
    assert np.allclose(f[:lo + 1], plain[:lo + 1]) and np.allclose(f[hi:], plain[hi:] / 4.0)
    mid = (lo + hi) // 2
    assert plain[mid] / 4.0 < f[mid] < plain[mid] or hi - lo < 2
    assert np.allclose(np.hypot(c4[1], s4[1]), mag)


def test_block_mask_slopes_and_sink():
    assert O.same_block(9, 5, 5) and not O.same_block(10, 9, 5) and O.same_block(10, 10, 5) and not O.same_block(3, 4, 5)
    assert O.same_block(1000, 0, None)
    assert O.head_slope(0, 8) == 0.5 and O.head_slope(7, 8) == 2.0 ** -8 and O.head_slope(0, 1) == 2.0 ** -8
    cfg = U.config([U.layer("attention", None, **U.attn(heads=2, kv_heads=1, dim=4, vdim=3, size=3))], vocab=11, width=8)
    P = {k: np.asarray(v, np.float64) for k, v in U.random_weights(cfg, 0).items()}
    mx = cfg["layers"][0]["mixer"]
    h = np.random.RandomState(1).randn(7, 8)
    k, v = O.keys_and_values(h, P, "l0.mix.", mx)
    gate = O.sigmoid(h @ P["l0.mix.g"].T)
    inv_o = np.linalg.pinv(P["l0.mix.o"].T)
    heads = lambda y: ((y @ inv_o) / gate).reshape(7, 2, 3)
    # position 3 opens a block: it sees itself only, and the sink takes its share
    out = heads(O.block_attention(h, P, "l0.mix.", mx, k, v))
    for hd in range(2):
        s = (h[3] @ P["l0.mix.q"].T).reshape(2, 4)[hd] @ k[3, 0] * mx["scale"]
        assert np.allclose(out[3, hd], v[3, 0] / (1.0 + math.exp(P["l0.mix.sink"][hd] - s)))
    # a sink far below every score is no sink; one far above takes everything
    P["l0.mix.sink"] = np.full(2, -50.0)
    no_sink = heads(O.block_attention(h, P, "l0.mix.", mx, k, v))
    q = (h @ P["l0.mix.q"].T).reshape(7, 2, 4)
    s = np.array([q[5, 1] @ k[j, 0] * mx["scale"] - O.head_slope(1, 2) * (5 - j) for j in (3, 4, 5)])
    w = np.exp(s - s.max()); w /= w.sum()
    assert np.allclose(no_sink[5, 1], w @ v[3:6, 0])
    P["l0.mix.sink"] = np.full(2, 50.0)
    assert abs(O.block_attention(h, P, "l0.mix.", mx, k, v)).max() < 1e-12


def test_latent_attention_equals_the_form_that_works_on_the_cached_latent():
    cfg = U.config([U.layer("latent_attention", None, **U.latent(heads=2, dim=4, rot_dim=6, vdim=5, kv_rank=7, q_rank=9, dims=4))], vocab=11, width=8)
    P = {k: np.asarray(v, np.float64) for k, v in U.random_weights(cfg, 2).items()}
    mx, eps, pre = cfg["layers"][0]["mixer"], 1e-6, "l0.mix."
    h = np.random.RandomState(3).randn(9, 8)
    want = O.latent_attention(h, P, pre, mx, eps)
    # second spelling: q' = W_uk^T q_plain scores the latent itself; the weighted latents pass W_uv afterwards
    q = (O.norm_plain(h @ P[pre + "dq"].T, P[pre + "dq.norm"], eps) @ P[pre + "uq"].T).reshape(9, 2, 10)
    low = h @ P[pre + "dkv"].T
    c = O.norm_plain(low[:, :7], P[pre + "dkv.norm"], eps)
    cos, sin = O.rotation_tables(mx["rot"], 9)
    out = np.zeros((9, 2, 5))
    for hd in range(2):
        uk, uv = P[pre + "uk"][hd * 4:(hd + 1) * 4], P[pre + "uv"][hd * 5:(hd + 1) * 5]
        for i in range(9):
            qr = O.rotate_pairs(q[i:i + 1, hd, 4:], cos[i:i + 1], sin[i:i + 1], 4)[0]
            s = np.array([(uk.T @ q[i, hd, :4]) @ c[j] + qr @ O.rotate_pairs(low[j:j + 1, 7:], cos[j:j + 1], sin[j:j + 1], 4)[0] for j in range(i + 1)])
            w = np.exp((s - s.max()) * mx["scale"]); w /= w.sum()
            out[i, hd] = uv @ (w @ c[:i + 1])
    assert np.allclose((out.reshape(9, 10) * O.sigmoid(h @ P[pre + "g"].T)) @ P[pre + "o"].T, want)


def test_gated_linear_attention_closed_forms():
    cfg = U.config([U.layer("gla", None, **U.gla(heads=1, dim=3, vdim=2, tau=2.0))], vocab=11, width=8)
    P = {k: np.asarray(v, np.float64) for k, v in U.random_weights(cfg, 4).items()}
    mx, pre = cfg["layers"][0]["mixer"], "l0.mix."
    h = np.random.RandomState(5).randn(4, 8)
    P[pre + "norm"] = np.ones(2); P[pre + "o"] = np.eye(2, 2)
    q = h @ P[pre + "q"].T * 3 ** -0.5; k = h @ P[pre + "k"].T; v = h @ P[pre + "v"].T
    a = O.sigmoid((h @ P[pre + "a1"].T) @ P[pre + "a2"].T + P[pre + "a2.b"]) ** 0.5
    # o_t = sum_s (q_t * prod_(s < u <= t) a_u) . k_s  v_s, then unit root mean square, then silu(gate)
    o = np.zeros((4, 2))
    for t in range(4):
        for s in range(t + 1):
            o[t] += ((q[t] * np.prod(a[s + 1:t + 1], axis=0)) @ k[s]) * v[s]
    want = O.unit_rms(o, 1e-6) * O.silu(h @ P[pre + "g"].T)
    assert np.allclose(O.gated_linear_attention(h, P, pre, mx, 1e-6), want)
    # a decay of one keeps everything: plain linear attention
    P[pre + "a2"] = np.zeros_like(P[pre + "a2"]); P[pre + "a2.b"] = np.full(3, 40.0)
    o = np.array([sum((q[t] @ k[s]) * v[s] for s in range(t + 1)) for t in range(4)])
    assert np.allclose(O.gated_linear_attention(h, P, pre, mx, 1e-6), O.unit_rms(o, 1e-6) * O.silu(h @ P[pre + "g"].T))


def test_layer_is_parallel_borrowed_keys_follow_their_source_and_generation_is_greedy():
    cfg = U.small_config()
    P = U.random_weights(cfg, 6)
    toks = U.tokens(30, cfg["vocab"], 6)
    logits, layers = O.forward(cfg, P, toks, True)
    assert logits.shape == (30, cfg["vocab"]) and layers.shape == (6, 30, cfg["width"])
    # feed-forward and mixer read the same residual: zeroing the feed-forward of layer 1 changes layer 1's output by exactly its term
    Q = dict(P); Q["l1.mlp.down"] = np.zeros_like(P["l1.mlp.down"])
    _, l2 = O.forward(cfg, Q, toks, True)
    x0 = layers[0]
    ff = O.squared_relu_ff(O.norm_around_zero(x0, P["l1.norm2"], cfg["norm"]["eps"]), {k: np.asarray(v, np.float64) for k, v in P.items()}, "l1.mlp.")
    assert np.allclose(layers[1] - l2[1], ff)
    # layer 3 has no key / value tensors and moves when layer 1's keys do
    assert "l3.mix.k" not in P and "l3.mix.v" not in P
    Q = dict(P); Q["l1.mix.k"] = P["l1.mix.k"] * 1.5
    Q["l1.mix.o"] = np.zeros_like(P["l1.mix.o"])
    R = dict(P); R["l1.mix.o"] = Q["l1.mix.o"]
    _, la = O.forward(cfg, Q, toks, True); _, lb = O.forward(cfg, R, toks, True)
    assert np.allclose(la[2], lb[2]) and not np.allclose(la[3], lb[3])
    # causal: a later token leaves earlier logits alone
    other = list(toks); other[-1] = (toks[-1] + 1) % cfg["vocab"]
    assert np.allclose(O.forward(cfg, P, other)[:-1], logits[:-1])
    out = O.generate(cfg, P, toks[:5], 3)
    assert out[:5] == toks[:5] and out[5] == int(np.argmax(O.forward(cfg, P, toks[:5])[-1]))
