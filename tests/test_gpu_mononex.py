"""GPU: the Mononex decoder in the library (kernels_layered.hip, model_layered.cpp, the engine's mixed steps) against the plain
NumPy statement oracle/mononex_oracle.py, on small configurations with random weights made here.

float32 compute is the sharp comparison (TOL_F32 relative to the largest logit); bfloat16 compute is checked against the
same oracle with the rounding's own allowance, and against itself across schedules."""
import numpy as np
import pytest

from oracle import mononex_oracle as O
from tests import mononex_util as U

pytestmark = pytest.mark.gpu

TOL_F32 = 2e-4
TOL_BF16 = 6e-2


def _load(tmp_path, cfg, P, dtype="float32", **kw):
    from crane_amd.backend import Model
    kw.setdefault("max_seq_len", 512)
    kw.setdefault("max_seqs", 4)
    return Model.from_pretrained(U.write_checkpoint(str(tmp_path / "ckpt"), cfg, P), compute_dtype=dtype, **kw)


def _err(got, want):
    want = np.asarray(want, np.float64)
    return float(np.abs(np.asarray(got, np.float64) - want).max() / np.abs(want).max())


def _all(n):
    return list(range(n))


SINGLE = {
    "gated linear attention alone": U.config([U.layer("gla", None, **U.gla(heads=3, dim=8, vdim=24, tau=3.0))]),
    "gated linear attention, tau 1, one head": U.config([U.layer("gla", None, **U.gla(heads=1, dim=20, vdim=12, tau=1.0))]),
    "block attention alone": U.config([U.layer("attention", None, **U.attn(heads=4, kv_heads=2, dim=16, vdim=8, size=9))]),
    "block attention, every head its own keys, no blocks": U.config([U.layer("attention", None, **U.attn(heads=3, kv_heads=3, dim=12, vdim=20, size=None))]),
    "borrowed keys and values": U.config([U.layer("attention", None, **U.attn(heads=2, kv_heads=1, dim=8, vdim=12, size=11)),
                                          U.layer("attention", None, **U.attn(heads=3, kv_heads=1, dim=8, vdim=12, size=7, scale=0.5, kv_from=0))]),
    "latent attention alone": U.config([U.layer("latent_attention", None, **U.latent())]),
    "latent attention, part of the rotated size turns, no stretching": U.config(
        [U.layer("latent_attention", None, **U.latent(heads=1, dim=12, rot_dim=10, vdim=6, kv_rank=14, q_rank=10, dims=6, scaling=None))]),
    "feed-forward beside the mixer": U.config([U.layer("gla", U.dense(40), **U.gla())]),
}


@pytest.mark.parametrize("name", list(SINGLE))
def test_each_mechanism_alone_whole_prompt_and_layer_rows(tmp_path, name):
    cfg = SINGLE[name]
    P = U.random_weights(cfg, 1)
    toks = U.tokens(41, cfg["vocab"], 1)
    want, layers = O.forward(cfg, P, toks, True)
    m = _load(tmp_path, cfg, P)
    try:
        m.layer_capture(True)
        s = m.seq_alloc()
        got, greedy = m.step_batch([(s, toks, _all(len(toks)))])
        rows = m.layer_rows().reshape(len(cfg["layers"]), len(toks), cfg["width"])
        assert _err(rows, layers) < TOL_F32
        assert _err(got, want) < TOL_F32
        assert list(greedy) == [int(np.argmax(r)) for r in got]
    finally:
        m.close()


def test_prefill_against_token_by_token_decoding(tmp_path):
    cfg = U.small_config()
    P = U.random_weights(cfg, 2)
    toks = U.tokens(70, cfg["vocab"], 2)
    want = O.forward(cfg, P, toks)
    m = _load(tmp_path, cfg, P)
    try:
        a, b = m.seq_alloc(), m.seq_alloc()
        whole, _ = m.step_batch([(a, toks, _all(len(toks)))])
        serial = np.concatenate([m.step_batch([(b, [t], [0])])[0] for t in toks])
        assert _err(whole, want) < TOL_F32 and _err(serial, want) < TOL_F32
        assert _err(serial, whole) < TOL_F32
    finally:
        m.close()


@pytest.mark.parametrize("cuts", [[2] * 12 + [3, 5, 2, 7, 1, 1, 2, 16, 2], [64, 2, 1, 3], [1, 69], [33, 33, 4], [5, 60, 2, 2, 1]])
def test_portions_of_several_sizes_down_to_two_tokens(tmp_path, cuts):
    cfg = U.small_config()
    P = U.random_weights(cfg, 3)
    n = sum(cuts)
    toks = U.tokens(n, cfg["vocab"], 3)
    want = O.forward(cfg, P, toks)
    m = _load(tmp_path, cfg, P)
    try:
        s, at, out = m.seq_alloc(), 0, []
        for c in cuts:
            out.append(m.step_batch([(s, toks[at:at + c], _all(c))])[0])
            at += c
        assert m.seq_len(s) == n
        assert _err(np.concatenate(out), want) < TOL_F32
    finally:
        m.close()


def test_batches_of_unequal_requests_against_each_alone(tmp_path):
    cfg = U.small_config()
    P = U.random_weights(cfg, 4)
    reqs = [U.tokens(n, cfg["vocab"], 10 + i) for i, n in enumerate((67, 5, 130, 31))]
    want = [O.forward(cfg, P, t) for t in reqs]
    # per step: (request, tokens taken) -- long portions beside single decode tokens, requests joining and pausing
    plan = [[(0, 40), (1, 2)], [(0, 1), (1, 1), (2, 64)], [(2, 2), (0, 1), (3, 30)], [(1, 2), (2, 60), (3, 1), (0, 25)], [(2, 0)]]
    m = _load(tmp_path, cfg, P)
    try:
        seqs = [m.seq_alloc() for _ in reqs]
        at = [0] * len(reqs)
        got = [[] for _ in reqs]
        for step in plan:
            step = [(r, c if c else len(reqs[r]) - at[r]) for r, c in step]
            out, _ = m.step_batch([(seqs[r], reqs[r][at[r]:at[r] + c], _all(c)) for r, c in step])
            row = 0
            for r, c in step:
                got[r].append(out[row:row + c])
                row += c
                at[r] += c
        for r in range(len(reqs)):
            have = np.concatenate(got[r])
            assert _err(have, want[r][:len(have)]) < TOL_F32, r
        assert at[2] == 130 and at[0] == 67
    finally:
        m.close()


def test_pages_and_slots_that_are_freed_and_used_again(tmp_path):
    cfg = U.small_config()
    P = U.random_weights(cfg, 5)
    m = _load(tmp_path, cfg, P, max_seq_len=192, kv_pool_tokens=256, max_seqs=2)        # 4 pages of 64, 2 slots
    try:
        for rnd in range(3):
            reqs = [U.tokens(n, cfg["vocab"], 20 + 2 * rnd + i) for i, n in enumerate((100 + 7 * rnd, 90 - 11 * rnd))]
            seqs = [m.seq_alloc(), m.seq_alloc()]
            with pytest.raises(Exception):
                m.seq_alloc()                                     # both slots taken
            out, _ = m.step_batch([(seqs[0], reqs[0][:50], []), (seqs[1], reqs[1], _all(len(reqs[1])))])
            assert _err(out, O.forward(cfg, P, reqs[1])) < TOL_F32
            out, _ = m.step_batch([(seqs[0], reqs[0][50:], _all(len(reqs[0]) - 50))])
            assert _err(out, O.forward(cfg, P, reqs[0])[50:]) < TOL_F32
            assert m.active_kv_cache_bytes() > 0
            for s in seqs:
                m.seq_free(s)
            assert m.active_kv_cache_bytes() == 0
        # a step that does not fit in the pool fails and leaves the sequence as it was
        a, b = m.seq_alloc(), m.seq_alloc()
        m.step_batch([(a, U.tokens(150, cfg["vocab"], 1), None)])
        with pytest.raises(Exception):
            m.step_batch([(b, U.tokens(120, cfg["vocab"], 2), None)])
        assert m.seq_len(b) == 0 and m.seq_len(a) == 150
    finally:
        m.close()


def _planted_block(size, heads=2, kv_heads=1, dim=16, vdim=8, alpha=9.0):
    """One block-attention layer whose input is a function of the token alone (no shift), with a query token QT and a key
    token KT whose score stands out by alpha^2 * scale whatever else is visible and however far away it is."""
    cfg = U.config([U.layer("attention", None, **U.attn(heads=heads, kv_heads=kv_heads, dim=dim, vdim=vdim, size=size, scale=0.25))],
                   vocab=67, width=40)
    P = U.random_weights(cfg, 7)
    P["l0.shift"][:] = 0
    P["l0.mix.sink"][:] = 1.0
    QT, KT = 65, 66
    h = O.norm_around_zero(P["embed"].astype(np.float64), P["l0.norm1"], cfg["norm"]["eps"])
    for g in range(kv_heads):
        P["l0.mix.k"][g * dim] = U.bf16_round(alpha * h[KT] / (h[KT] @ h[KT]))
    for hd in range(heads):
        P["l0.mix.q"][hd * dim] = U.bf16_round(alpha * h[QT] / (h[QT] @ h[QT]))
    return cfg, P, QT, KT


@pytest.mark.parametrize("decoded", [False, True])
def test_planted_keys_at_both_edges_of_a_block_at_page_borders_and_far_inside(tmp_path, decoded):
    size = 70
    cfg, P, QT, KT = _planted_block(size)
    m = _load(tmp_path, cfg, P)
    try:
        # (key position, query position): first and last position of a block from its other end, the position just outside on
        # either side, keys on both sides of a page border (pages of 64 tokens) inside one block, a block's first query
        cases = [(0, 69), (69, 70), (70, 139), (69, 139), (139, 140), (127, 128), (127, 139), (128, 139), (63, 64), (63, 69), (64, 69),
                 (140, 199), (139, 199), (70, 70)]
        for kp, qp in cases:
            toks = U.tokens(200, 65, kp * 1000 + qp)
            toks[kp] = KT
            toks[qp] = QT if kp != qp else KT
            want = O.forward(cfg, P, toks)
            if kp != qp:
                plain = list(toks)
                plain[kp] = (toks[kp - 1] + 1) % 65 if kp else 1
                moved = float(np.abs(O.forward(cfg, P, plain)[qp] - want[qp]).max() / np.abs(want[qp]).max())
                assert (moved > 0.05) == O.same_block(qp, kp, size), (kp, qp, moved)   # the planted key matters exactly inside the block
            s = m.seq_alloc()
            if decoded:
                lo = max(1, qp - 2)
                m.step_batch([(s, toks[:lo], [])])
                got = np.concatenate([m.step_batch([(s, [toks[p]], [0])])[0] for p in range(lo, qp + 1)])
                assert _err(got, want[lo:qp + 1]) < TOL_F32, (kp, qp)
            else:
                got, _ = m.step_batch([(s, toks[:qp + 1], [qp - 1, qp])])
                assert _err(got, want[qp - 1:qp + 1]) < TOL_F32, (kp, qp)
            m.seq_free(s)
    finally:
        m.close()


def _planted_latent(alpha=9.0):
    """One latent-attention layer (no shift): the first unrotated key element of every head is alpha for token KT, the first
    unrotated query element alpha for token QT."""
    cfg = U.config([U.layer("latent_attention", None, **U.latent(heads=2, dim=8, rot_dim=4, vdim=12, kv_rank=16, q_rank=24, scale=0.25))],
                   vocab=67, width=40)
    P = U.random_weights(cfg, 8)
    P["l0.shift"][:] = 0
    QT, KT = 65, 66
    eps = cfg["norm"]["eps"]
    h = O.norm_around_zero(P["embed"].astype(np.float64), P["l0.norm1"], eps)
    c = O.norm_plain(h @ P["l0.mix.dkv"][:16].astype(np.float64).T, P["l0.mix.dkv.norm"], eps)
    cq = O.norm_plain(h @ P["l0.mix.dq"].astype(np.float64).T, P["l0.mix.dq.norm"], eps)
    for hd in range(2):
        P["l0.mix.uk"][hd * 8] = U.bf16_round(alpha * c[KT] / (c[KT] @ c[KT]))
        P["l0.mix.uq"][hd * 12] = U.bf16_round(alpha * cq[QT] / (cq[QT] @ cq[QT]))
    return cfg, P, QT, KT


@pytest.mark.parametrize("decoded", [False, True])
def test_a_planted_key_hundreds_of_positions_back_in_latent_attention(tmp_path, decoded):
    cfg, P, QT, KT = _planted_latent()
    m = _load(tmp_path, cfg, P)
    try:
        for kp, qp in [(0, 299), (3, 280), (63, 257), (64, 256), (191, 192)]:
            toks = U.tokens(300, 65, kp * 1000 + qp)
            toks[kp], toks[qp] = KT, QT
            want = O.forward(cfg, P, toks)
            plain = list(toks)
            plain[kp] = (toks[kp + 1] + 1) % 65
            moved = float(np.abs(O.forward(cfg, P, plain)[qp] - want[qp]).max() / np.abs(want[qp]).max())
            assert moved > 0.05, (kp, qp, moved)
            s = m.seq_alloc()
            if decoded:
                m.step_batch([(s, toks[:qp - 2], [])])
                got = np.concatenate([m.step_batch([(s, [toks[p]], [0])])[0] for p in range(qp - 2, qp + 1)])
                assert _err(got, want[qp - 2:qp + 1]) < TOL_F32, (kp, qp)
            else:
                got, _ = m.step_batch([(s, toks[:qp + 1], [qp - 1, qp])])
                assert _err(got, want[qp - 1:qp + 1]) < TOL_F32, (kp, qp)
            m.seq_free(s)
    finally:
        m.close()


def test_a_token_long_ago_still_shows_through_the_linear_state(tmp_path):
    """Decay close to one (large bias of the decay's projection): swapping token 2 moves the logits 250 tokens later, in the
    oracle and -- through a portion, a long run of single tokens and another portion -- in the library."""
    cfg = U.config([U.layer("gla", None, **U.gla(heads=2, dim=8, vdim=8, tau=16.0))], vocab=37, width=24)
    P = U.random_weights(cfg, 9)
    P["l0.mix.a2.b"][:] = 6.0
    toks = U.tokens(256, 37, 9)
    other = list(toks); other[2] = (toks[2] + 5) % 37
    want, want2 = O.forward(cfg, P, toks), O.forward(cfg, P, other)
    assert _err(want2[255], want[255]) > 3e-3
    m = _load(tmp_path, cfg, P)
    try:
        for t, w in ((toks, want), (other, want2)):
            s = m.seq_alloc()
            m.step_batch([(s, t[:40], [])])
            for p in range(40, 200):
                m.step_batch([(s, [t[p]], [])], want_logits=False)
            got, _ = m.step_batch([(s, t[200:], [54, 55])])
            assert _err(got, w[254:256]) < TOL_F32
            m.seq_free(s)
    finally:
        m.close()


def test_first_tokens_of_a_sequence(tmp_path):
    cfg = U.small_config()
    P = U.random_weights(cfg, 8)
    m = _load(tmp_path, cfg, P)
    try:
        for n in (1, 2, 3, 5):
            toks = U.tokens(n, cfg["vocab"], 40 + n)
            s = m.seq_alloc()
            got, _ = m.step_batch([(s, toks, _all(n))])
            assert _err(got, O.forward(cfg, P, toks)) < TOL_F32
            m.seq_free(s)
        # a fresh slot starts from zero state and a zero shift input although the one before it left its own behind
        toks = U.tokens(4, cfg["vocab"], 50)
        s = m.seq_alloc()
        got = np.concatenate([m.step_batch([(s, [t], [0])])[0] for t in toks])
        assert _err(got, O.forward(cfg, P, toks)) < TOL_F32
    finally:
        m.close()


def test_long_decoding_across_many_blocks(tmp_path):
    cfg = U.small_config()                                        # blocks of 21 and 33 positions
    P = U.random_weights(cfg, 9)
    toks = U.tokens(230, cfg["vocab"], 9)
    want = O.forward(cfg, P, toks)
    m = _load(tmp_path, cfg, P)
    try:
        s = m.seq_alloc()
        m.step_batch([(s, toks[:10], [])])
        got = np.concatenate([m.step_batch([(s, [t], [0])])[0] for t in toks[10:]])
        assert _err(got, want[10:]) < TOL_F32
    finally:
        m.close()


OTHER = {
    "odd sizes": U.config([U.layer("attention", U.dense(10), **U.attn(heads=6, kv_heads=2, dim=12, vdim=6, size=1, scale=1.0)),
                           U.layer("gla", None, **U.gla(heads=1, dim=20, vdim=12, tau=1.0)),
                           U.layer("latent_attention", U.dense(30), **U.latent(heads=1, dim=6, rot_dim=2, vdim=10, kv_rank=10, q_rank=6, scale=0.7,
                                                                               scaling=dict(factor=1.5, original=16, fast=4.0, slow=1.0))),
                           U.layer("attention", None, **U.attn(heads=1, kv_heads=1, dim=40, vdim=40, size=1000))],
                          vocab=37, width=30, eps=1e-5),
    "wide heads": U.config([U.layer("gla", U.dense(), **U.gla(heads=1, dim=160, vdim=72, tau=30.0)),
                            U.layer("attention", None, **U.attn(heads=2, kv_heads=2, dim=192, vdim=144, size=16)),
                            U.layer("latent_attention", None, **U.latent(heads=2, dim=40, rot_dim=24, vdim=48, kv_rank=400, q_rank=96, scale=0.05)),
                            U.layer("attention", None, **U.attn(heads=4, kv_heads=2, dim=192, vdim=144, size=50, kv_from=1))],
                           vocab=50, width=64),
    "equal sizes, borrowing from the first layer": U.config(
        [U.layer("attention", U.dense(64), **U.attn(heads=8, kv_heads=8, dim=8, vdim=8, size=5)),
         U.layer("gla", U.dense(64), **U.gla(heads=4, dim=4, vdim=4, tau=16.0)),
         U.layer("attention", U.dense(64), **U.attn(heads=8, kv_heads=8, dim=8, vdim=8, size=64, kv_from=0)),
         U.layer("attention", U.dense(64), **U.attn(heads=16, kv_heads=8, dim=8, vdim=8, size=None, kv_from=0))], vocab=128, width=64),
}


@pytest.mark.parametrize("name", list(OTHER))
def test_other_sizes_whole_portioned_and_decoded(tmp_path, name):
    cfg = OTHER[name]
    P = U.random_weights(cfg, 11, a_rank=16 if "equal" in name else 5)
    toks = U.tokens(90, cfg["vocab"], 11)
    want = O.forward(cfg, P, toks)
    m = _load(tmp_path, cfg, P)
    try:
        a, b = m.seq_alloc(), m.seq_alloc()
        whole, _ = m.step_batch([(a, toks, _all(90))])
        assert _err(whole, want) < TOL_F32
        out, at = [], 0
        for c in [7, 2, 30, 1, 1, 2, 40, 3, 1, 1, 1, 1]:
            out.append(m.step_batch([(b, toks[at:at + c], _all(c))])[0])
            at += c
        assert at == 90 and _err(np.concatenate(out), want) < TOL_F32
    finally:
        m.close()


def test_greedy_generation_through_generate_and_through_the_engine(tmp_path):
    from crane_amd.backend import GenerationConfig
    from crane_amd.engine import GenerationParams, InferenceEngine
    cfg = U.small_config()
    P = U.random_weights(cfg, 12)
    prompts = [U.tokens(n, cfg["vocab"], 60 + i) for i, n in enumerate((9, 70, 3, 25, 40))]
    lens = [12, 6, 20, 9, 15]
    want = [O.generate(cfg, P, p, n)[len(p):] for p, n in zip(prompts, lens)]
    m = _load(tmp_path, cfg, P, max_seq_len=128, kv_pool_tokens=384, max_seqs=4, prefill_chunk=48)
    try:
        assert m.generate(prompts[0], GenerationConfig.greedy(lens[0]))[len(prompts[0]):] == want[0]
        m.clear_kv_cache()
        eng = InferenceEngine(m, max_running=3)                   # 5 requests, 3 slots, 48-row steps: prompts are fed in portions
        ids = [eng.submit(p, GenerationParams.greedy(n)) for p, n in zip(prompts, lens)]
        toks, done = eng.run_until_idle()
        for rid, w in zip(ids, want):
            assert toks[rid] == w
            assert done[rid].kind == "finished" and done[rid].finish_reason == "length"
        st = eng.stats()
        assert st["completed"] == 5 and st["failed"] == 0 and st["free_pages"] == st["total_pages"]
        # sampled requests run through the same steps and the device sampler
        rid = eng.submit(prompts[3], GenerationParams(max_tokens=8, temperature=0.8, top_p=0.9, top_k=20, seed=5))
        toks, done = eng.run_until_idle()
        assert len(toks[rid]) == 8 and all(0 <= t < cfg["vocab"] for t in toks[rid])
        eng.close()
    finally:
        m.close()


def test_bfloat16_format_against_the_oracle_and_across_schedules(tmp_path):
    cfg = U.small_config()
    P = U.random_weights(cfg, 13)
    toks = U.tokens(100, cfg["vocab"], 13)
    want = O.forward(cfg, P, toks)
    m = _load(tmp_path, cfg, P, dtype="bfloat16")
    try:
        a, b = m.seq_alloc(), m.seq_alloc()
        whole, _ = m.step_batch([(a, toks, _all(100))])
        assert _err(whole, want) < TOL_BF16
        out, at = [], 0
        for c in [50, 2, 13, 1, 1, 33]:
            out.append(m.step_batch([(b, toks[at:at + c], _all(c))])[0])
            at += c
        assert _err(np.concatenate(out), want) < TOL_BF16
        assert _err(np.concatenate(out), whole) < TOL_BF16
    finally:
        m.close()


def test_fork_carries_pages_shift_inputs_and_linear_state(tmp_path):
    cfg = U.small_config()
    P = U.random_weights(cfg, 14)
    toks = U.tokens(80, cfg["vocab"], 14)
    want = O.forward(cfg, P, toks)
    m = _load(tmp_path, cfg, P)
    try:
        a = m.seq_alloc()
        m.step_batch([(a, toks[:37], [])])
        b = m.seq_fork(a)
        ga, _ = m.step_batch([(a, toks[37:], _all(43)), ])
        gb, _ = m.step_batch([(b, toks[37:], _all(43))])
        assert _err(ga, want[37:]) < TOL_F32 and _err(gb, want[37:]) < TOL_F32
        with pytest.raises(Exception):
            m.seq_truncate(a, 10)                                 # a recurrent state cannot be rewound
    finally:
        m.close()


def test_synthetic_registry_model_generates(tmp_path):
    from crane_amd import configs
    from crane_amd.backend import GenerationConfig, Model
    m = Model.synthetic(configs.get_config("tiny-mononex"), seed=3, max_seq_len=128, max_seqs=2)
    try:
        assert m.num_layers() == 5 and m.vocab_size == 320
        out = m.generate([1, 2, 3, 4, 5], GenerationConfig.greedy(6))
        assert len(out) == 11
        logits = m.forward_step([7, 8, 9], 0)[0, 0]
        assert np.isfinite(logits).all() and int(np.argmax(logits)) == m.forward_step_greedy([7, 8, 9], 0)
        assert m.decode_bytes_per_token(64) > m.weight_bytes() // 4
    finally:
        m.close()


def test_bfloat16_products_on_the_shared_gemm_and_on_the_row_kernel_agree(tmp_path):
    """Widths that fit the matrix-core GEMM of the other families (output widths that are multiples of 128): a 300-token prompt
    (shared GEMM for the products that fit), the same with the switch off (tiled kernel of this family), and token by token
    (row kernel)."""
    cfg = U.config([U.layer("attention", U.dense(256), **U.attn(heads=4, kv_heads=2, dim=32, vdim=32, size=40)),
                    U.layer("gla", U.dense(256), **U.gla(heads=2, dim=32, vdim=64, tau=8.0)),      # 416 input-projection columns: 384 + 32
                    U.layer("latent_attention", U.dense(128), **U.latent(heads=4, dim=16, rot_dim=16, vdim=32, kv_rank=32, q_rank=64)),
                    U.layer("attention", None, **U.attn(heads=4, kv_heads=2, dim=32, vdim=32, size=24, kv_from=0))], vocab=320, width=128)
    P = U.random_weights(cfg, 15, a_rank=32)
    toks = U.tokens(300, cfg["vocab"], 15)                         # 256 rows and more: wide products are split at the last whole tile
    want = O.forward(cfg, P, toks)
    m = _load(tmp_path, cfg, P, dtype="bfloat16")
    try:
        a, b, c = m.seq_alloc(), m.seq_alloc(), m.seq_alloc()
        shared, _ = m.step_batch([(a, toks, _all(300))])
        m.debug_set("lay_shared_gemm", 0)
        tiled, _ = m.step_batch([(b, toks, _all(300))])
        rows = np.concatenate([m.step_batch([(c, [t], [0])])[0] for t in toks])
        for got in (shared, tiled, rows):
            assert _err(got, want) < TOL_BF16
        assert _err(shared, tiled) < TOL_BF16 and _err(rows, tiled) < TOL_BF16
    finally:
        m.close()


@pytest.mark.parametrize("dtype,tol", [("float32", TOL_F32), ("bfloat16", TOL_BF16)])
def test_decode_steps_over_hundreds_of_keys_and_a_long_portion_in_chunks(tmp_path, dtype, tol):
    """Blocks of hundreds of positions and causal latent attention: decode steps deal the key tiles of a query tile to several
    blocks and merge them (the sink counted once); the long portion in front runs the gated linear layer parallel over chunks
    (the state in front of every chunk by a scan with that chunk's own decay)."""
    cfg = U.config([U.layer("attention", U.dense(), **U.attn(heads=4, kv_heads=2, dim=16, vdim=24, size=300)),
                    U.layer("gla", None, **U.gla(heads=2, dim=16, vdim=40, tau=6.0)),
                    U.layer("latent_attention", None, **U.latent(heads=3, dim=8, rot_dim=8, vdim=16, kv_rank=24, q_rank=32))], vocab=71, width=48)
    P = U.random_weights(cfg, 16)
    toks = U.tokens(430, cfg["vocab"], 16)
    want = O.forward(cfg, P, toks)
    m = _load(tmp_path, cfg, P, dtype=dtype)
    try:
        s = m.seq_alloc()
        first, _ = m.step_batch([(s, toks[:395], [0, 31, 32, 33, 200, 299, 300, 394])])
        assert _err(first, want[[0, 31, 32, 33, 200, 299, 300, 394]]) < tol
        got = np.concatenate([m.step_batch([(s, [t], [0])])[0] for t in toks[395:]])
        assert _err(got, want[395:]) < tol
    finally:
        m.close()


def test_a_step_larger_than_one_pass_is_cut_into_passes(tmp_path):
    """Passes of 32 rows: a 100-token portion beside a 45-token one and a single token runs as five passes; the wanted rows come
    back in the order of the items whatever pass they fell into."""
    cfg = U.small_config()
    P = U.random_weights(cfg, 17)
    reqs = [U.tokens(n, cfg["vocab"], 70 + i) for i, n in enumerate((100, 45, 9))]
    want = [O.forward(cfg, P, t) for t in reqs]
    m = _load(tmp_path, cfg, P, prefill_chunk=32)
    try:
        s = [m.seq_alloc() for _ in reqs]
        m.step_batch([(s[2], reqs[2][:8], [])])
        w0, w1 = [0, 31, 32, 63, 64, 99], [10, 44]
        got, greedy = m.step_batch([(s[0], reqs[0], w0), (s[1], reqs[1], w1), (s[2], reqs[2][8:], None)])
        ref = np.concatenate([want[0][w0], want[1][w1], want[2][8:9]])
        assert got.shape == ref.shape and _err(got, ref) < TOL_F32
        assert list(greedy) == [int(np.argmax(r)) for r in got]
        assert [m.seq_len(x) for x in s] == [100, 45, 9]
    finally:
        m.close()


def test_matrix_core_attention_of_prompt_passes(tmp_path):
    """bfloat16 format, key and value sizes that are multiples of 16: prompt passes run block attention (value pages of their own,
    block edges inside a tile, the sink, borrowed pages) and latent attention (values = the latent part of the cached rows) on the
    matrix cores.  Against the oracle, and against the same steps with the switch off."""
    cfg = U.config([U.layer("attention", U.dense(), **U.attn(heads=6, kv_heads=2, dim=32, vdim=16, size=50)),
                    U.layer("latent_attention", None, **U.latent(heads=3, dim=16, rot_dim=16, vdim=24, kv_rank=48, q_rank=40)),
                    U.layer("attention", None, **U.attn(heads=2, kv_heads=2, dim=32, vdim=16, size=7, scale=0.4, kv_from=0)),
                    U.layer("attention", None, **U.attn(heads=5, kv_heads=1, dim=16, vdim=48, size=None))], vocab=90, width=64)
    P = U.random_weights(cfg, 18)
    reqs = [U.tokens(200, cfg["vocab"], 81), U.tokens(90, cfg["vocab"], 82)]
    want = [O.forward(cfg, P, t) for t in reqs]
    m = _load(tmp_path, cfg, P, dtype="bfloat16")
    try:
        outs = []
        for on in (1, 0):
            m.debug_set("lay_attn_mfma", on)
            a, b = m.seq_alloc(), m.seq_alloc()
            g1, _ = m.step_batch([(a, reqs[0][:130], _all(130)), (b, reqs[1][:17], _all(17))])
            g2, _ = m.step_batch([(a, reqs[0][130:], _all(70)), (b, reqs[1][17:], _all(73))])
            got = [np.concatenate([g1[:130], g2[:70]]), np.concatenate([g1[130:], g2[70:]])]
            for r in range(2):
                assert _err(got[r], want[r]) < TOL_BF16, (on, r)
            outs.append(got)
            m.seq_free(a); m.seq_free(b)
        for r in range(2):
            assert _err(outs[0][r], outs[1][r]) < 3e-2
    finally:
        m.close()


def test_matrix_core_latent_attention_over_long_cached_rows(tmp_path):
    """bfloat16 format, cached rows of 192 and 288 elements (latent + rotated key part): the wide matrix-core form of prompt
    passes (the value operand gathered from the key rows), both register layouts.  Against the oracle and against the switch off."""
    cfg = U.config([U.layer("latent_attention", U.dense(), **U.latent(heads=3, dim=16, rot_dim=16, vdim=24, kv_rank=176, q_rank=40, scale=0.1)),
                    U.layer("latent_attention", None, **U.latent(heads=2, dim=8, rot_dim=16, vdim=16, kv_rank=272, q_rank=24, scale=0.1))],
                   vocab=90, width=64)
    P = U.random_weights(cfg, 19)
    reqs = [U.tokens(150, cfg["vocab"], 83), U.tokens(70, cfg["vocab"], 84)]
    want = [O.forward(cfg, P, t) for t in reqs]
    m = _load(tmp_path, cfg, P, dtype="bfloat16")
    try:
        outs = []
        for on in (1, 0):
            m.debug_set("lay_attn_mfma", on)
            a, b = m.seq_alloc(), m.seq_alloc()
            g1, _ = m.step_batch([(a, reqs[0][:100], _all(100)), (b, reqs[1][:17], _all(17))])
            g2, _ = m.step_batch([(a, reqs[0][100:], _all(50)), (b, reqs[1][17:], _all(53))])
            got = [np.concatenate([g1[:100], g2[:50]]), np.concatenate([g1[100:], g2[50:]])]
            for r in range(2):
                assert _err(got[r], want[r]) < TOL_BF16, (on, r)
            outs.append(got)
            m.seq_free(a); m.seq_free(b)
        for r in range(2):
            assert _err(outs[0][r], outs[1][r]) < 3e-2
    finally:
        m.close()


def test_gated_linear_attention_over_a_whole_pass_of_chunks(tmp_path):
    """2048 + 37 tokens, 8 heads: the first pass has 512 (chunk, head) pairs, where one block walks all value slices of its pair."""
    cfg = U.config([U.layer("gla", None, **U.gla(heads=8, dim=8, vdim=40, tau=5.0))], vocab=53, width=32)
    P = U.random_weights(cfg, 20)
    toks = U.tokens(2085, cfg["vocab"], 20)
    want = O.forward(cfg, P, toks)
    rows = [0, 31, 32, 1000, 2047, 2048, 2084]
    m = _load(tmp_path, cfg, P, max_seq_len=2112, kv_pool_tokens=2112)
    try:
        s = m.seq_alloc()
        got, _ = m.step_batch([(s, toks, rows)])
        assert _err(got, want[rows]) < TOL_F32
    finally:
        m.close()


def _drawn_config(seed):
    """A model of this design with sizes, layer order and constants drawn from the seed (widths of a few hundred)."""
    rs = np.random.RandomState(100 + seed)
    pick = lambda *xs: xs[rs.randint(len(xs))]
    width, layers, owners = pick(96, 128, 192, 256, 320), [], []
    for i in range(rs.randint(4, 8)):
        kind = pick("attention", "latent_attention", "gla")
        mlp = None if rs.rand() < 0.2 else U.dense(pick(64, 136, 384, 512))
        if kind == "attention":
            if owners and rs.rand() < 0.5:
                src = owners[rs.randint(len(owners))]
                o = layers[src]["mixer"]
                mx = U.attn(heads=o["kv_heads"] * pick(1, 2, 3), kv_heads=o["kv_heads"], dim=o["dim"], vdim=o["vdim"], size=pick(None, 17, 64, 100),
                            scale=pick(0.1, 0.25), kv_from=src)
            else:
                kvh = pick(1, 2, 4)
                mx = U.attn(heads=kvh * pick(1, 2, 4), kv_heads=kvh, dim=pick(16, 24, 32, 64), vdim=pick(16, 32, 48), size=pick(None, 30, 64, 128),
                            scale=pick(0.125, 0.2))
                owners.append(i)
        elif kind == "latent_attention":
            rot_dim = pick(8, 16, 32)
            scaling = pick(None, dict(factor=pick(2.0, 8.0), original=pick(32, 128), fast=pick(8.0, 32.0), slow=pick(1.0, 2.0)))
            mx = U.latent(heads=pick(1, 2, 4, 8), dim=pick(8, 16, 32), rot_dim=rot_dim, vdim=pick(16, 24, 32), kv_rank=pick(24, 64, 80, 128),
                          q_rank=pick(32, 96, 128), scale=pick(0.1, 0.2), base=pick(100.0, 10000.0, 1e6), dims=pick(rot_dim, rot_dim // 2), scaling=scaling)
        else:
            mx = U.gla(heads=pick(1, 2, 4), dim=pick(8, 16, 32, 64), vdim=pick(16, 32, 64, 72), tau=pick(1.0, 4.0, 16.0, 32.0))
        layers.append(U.layer(kind, mlp, **mx))
    return U.config(layers, vocab=pick(97, 256, 601), width=width, eps=pick(1e-6, 1e-5, 1e-4))


@pytest.mark.parametrize("seed", range(8))
def test_drawn_models_whole_in_portions_and_decoded_in_both_formats(tmp_path, seed):
    cfg = _drawn_config(seed)
    P = U.random_weights(cfg, 30 + seed, a_rank=(4, 16, 24)[seed % 3])
    toks = U.tokens(150, cfg["vocab"], 30 + seed)
    want = O.forward(cfg, P, toks)
    for dtype, tol in (("float32", TOL_F32), ("bfloat16", TOL_BF16)):
        m = _load(tmp_path, cfg, P, dtype=dtype)
        try:
            a, b = m.seq_alloc(), m.seq_alloc()
            whole, _ = m.step_batch([(a, toks, _all(150))])
            assert _err(whole, want) < tol, (dtype, "whole")
            out, at = [], 0
            for c in [70, 2, 33, 1, 1, 17, 1, 25]:
                out.append(m.step_batch([(b, toks[at:at + c], _all(c))])[0])
                at += c
            assert at == 150 and _err(np.concatenate(out), want) < tol, (dtype, "portions")
        finally:
            m.close()
