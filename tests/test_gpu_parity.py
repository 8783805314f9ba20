"""Parity of the HIP path (through the C-ABI) against the CPU oracle on identical seeded inputs.

Bars: gathers / index work bit-exact; fp32 activations, log-probs and attention weights within 1e-4 relative
(|got - want| <= 1e-4 * max(|want|, 1e-2), see gpu_util.assert_close)."""
import numpy as np
import pytest

import oracle_lib as o
from gpu_util import Layer, assert_close, magnitude_floor, run_lstm_step
from zoph_rnn_amd import capi, synth

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def ctx():
    c = capi.Context(0)
    yield c
    c.close()


def U(g, shape, lo=-0.08, hi=0.08):
    return synth.uniform(g, shape, lo, hi)


# ------------------------------------------------------------------------------------------------ A1 / A2 / A12
def test_vocab_prep_and_gather_bit_exact(ctx):
    g = synth.rng(1, 10)
    V, H = 97, 52
    ids = g.integers(0, V, size=300).astype(np.int32)
    ids[::7] = -1
    d_ids = ctx.array(ids)
    d_nn, d_m = ctx.empty(ids.shape, np.int32), ctx.empty(ids.shape, np.int32)
    ctx.vocab_prep(d_ids, ids.size, V, d_nn, d_m)
    ctx.sync()
    nn, m = o.vocab_prep(ids)
    assert np.array_equal(d_nn.get(), nn) and np.array_equal(d_m.get(), m)
    d_mf = ctx.empty(ids.shape, np.float32)
    ctx.vocab_prep_softmax(d_ids, ids.size, V, d_m, d_mf)
    ctx.sync()
    ids2, m2, mf2 = o.vocab_softmax(ids)
    assert np.array_equal(d_ids.get(), ids2) and np.array_equal(d_m.get(), m2) and np.array_equal(d_mf.get(), mf2)
    for Hh in (52, 51, 1000):  # 16-byte path, scalar path, full size
        W = U(g, (Hh, V))
        gids = np.array([0, V - 1, 5, 5, 0, 17] + list(g.integers(0, V, size=40)), np.int32)
        d_x = ctx.empty((Hh, gids.size))
        ctx.embed_gather(ctx.array(W), Hh, V, ctx.array(gids), gids.size, d_x)
        ctx.sync()
        assert d_x.get().tobytes() == o.embed_gather(W, gids).tobytes()


@pytest.mark.parametrize("Hh,n", [(1000, 1500), (260, 1024), (2052, 1100), (4, 2000)])
def test_gather_many_columns_bit_exact(ctx, Hh, n):
    """1024 columns and more take the one-wave-per-column kernel: column lengths below, at and above one 1024-float
    pass, duplicates, first and last column of the table."""
    g = synth.rng(23, Hh + n)
    V = 777
    W = U(g, (Hh, V))
    ids = g.integers(0, V, size=n).astype(np.int32)
    ids[:4] = [0, V - 1, 5, 5]
    d_x = ctx.empty((Hh, n))
    ctx.embed_gather(ctx.array(W), Hh, V, ctx.array(ids), n, d_x)
    ctx.sync()
    assert d_x.get().tobytes() == o.embed_gather(W, ids).tobytes()
    bad = ids.copy()
    bad[n // 2] = V + 3
    ctx.embed_gather(ctx.array(W), Hh, V, ctx.array(bad), n, d_x)
    with pytest.raises(capi.ZrError):
        ctx.sync()
    want = o.embed_gather(W, np.minimum(bad, V - 1))
    assert d_x.get().tobytes() == want.tobytes()


def test_gather_out_of_range_id_is_reported_not_fatal(ctx):
    W = np.asfortranarray(np.arange(12, dtype=np.float32).reshape(4, 3, order="F"))
    d_x = ctx.empty((4, 2))
    ctx.embed_gather(ctx.array(W), 4, 3, ctx.array(np.array([1, 7], np.int32)), 2, d_x)
    with pytest.raises(capi.ZrError) as e:
        ctx.sync()
    assert e.value.code == -4
    assert np.array_equal(d_x.get()[:, 0], W[:, 1]) and np.array_equal(d_x.get()[:, 1], W[:, 2])
    ctx.sync()  # flag cleared


def test_decoder_state_shuffles(ctx):
    g = synth.rng(2, 10)
    src = U(g, (1000, 12))
    perm = np.array([3, 3, 0, 11, 5, 5, 5, 1, 2, 10, 9, 0], np.int32)
    d_dst = ctx.empty((1000, 12))
    ctx.gather_columns(ctx.array(src), 1000, ctx.array(perm), 12, d_dst)
    ctx.sync()
    assert d_dst.get().tobytes() == o.gather_columns(src, perm).tobytes()
    ctx.broadcast_column(ctx.array(src[:, [4]]), 1000, 12, d_dst)
    ctx.sync()
    assert np.array_equal(d_dst.get(), np.repeat(src[:, [4]], 12, axis=1))
    # every state matrix of a decode step in one launch: bit-equal to one gather per matrix
    for Hh in (1000, 50, 33):  # 16-byte path, and two heights that take the scalar path
        srcs = [U(g, (Hh, 12)) for _ in range(9)]
        dsts = [ctx.empty((Hh, 12)) for _ in range(9)]
        ctx.gather_columns_multi([ctx.array(a) for a in srcs], Hh, ctx.array(perm), 12, 12, dsts)
        ctx.sync()
        for a, d in zip(srcs, dsts):
            assert d.get().tobytes() == o.gather_columns(a, perm).tobytes()
    bad = ctx.array(np.array([0, 12, 3], np.int32))  # 12 is out of range: clamped, reported at the next sync
    ctx.gather_columns_multi([ctx.array(srcs[0])], 33, bad, 12, 3, [ctx.empty((33, 3))])
    with pytest.raises(capi.ZrError):
        ctx.sync()
    ctx.sync()


# ------------------------------------------------------------------------------------------------ A3 contraction
@pytest.mark.parametrize("cfg", [0, 1, 2, 3, 4, 5, 6, 7, 8])
@pytest.mark.parametrize("M,N,K,trans", [(100, 8, 100, 0), (257, 33, 61, 0), (64, 128, 200, 1), (95, 7, 37, 1)])
def test_gemm_tiles_and_tails(ctx, cfg, M, N, K, trans):
    g = synth.rng(3, 100 * cfg + M)
    A = U(g, (K, M) if trans else (M, K), -1, 1)
    B = U(g, (K, N), -1, 1)
    want = (A.T.astype(np.float64) if trans else A.astype(np.float64)) @ B.astype(np.float64)
    dC = ctx.zeros((M, N))
    ctx.set_option(capi.ZR_OPT_GEMM_CFG, cfg)
    try:
        ctx.gemm(trans, M, N, K, ctx.array(A), A.shape[0], ctx.array(B), K, dC, M)
        ctx.sync()
    finally:
        ctx.set_option(capi.ZR_OPT_GEMM_CFG, 0)
    # operands are U(-1,1): entries near zero are sums with cancellation whose rounding noise follows the size of the
    # partial sums, so the near-zero floor follows the largest output (gpu_util.magnitude_floor)
    assert_close(dC.get(), want, floor=magnitude_floor(want), what="gemm cfg %d" % cfg)


def test_gemm_padded_leading_dimensions(ctx):
    g = synth.rng(4, 1)
    M, N, K, lda, ldb, ldc = 70, 9, 44, 75, 47, 90  # ldb not a multiple of 4 -> scalar activation loads
    A, B = U(g, (lda, K), -1, 1), U(g, (ldb, N), -1, 1)
    C0 = np.full((ldc, N), 7.0, np.float32, order="F")
    dC = ctx.array(C0)
    ctx.gemm(0, M, N, K, ctx.array(A), lda, ctx.array(B), ldb, dC, ldc)
    ctx.sync()
    got = dC.get()
    want = A[:M].astype(np.float64) @ B[:K].astype(np.float64)
    assert_close(got[:M], want, floor=magnitude_floor(want), what="padded gemm")
    assert np.all(got[M:] == 7.0)  # rows beyond M untouched


def test_gemm_full_size_attention_shape(ctx):
    g = synth.rng(5, 1)
    A, B = U(g, (1000, 1000)), U(g, (1000, 128), -1, 1)
    dC = ctx.empty((1000, 128))
    ctx.gemm(0, 1000, 128, 1000, ctx.array(A), 1000, ctx.array(B), 1000, dC, 1000)
    ctx.sync()
    assert_close(dC.get(), o.gemm_nn(A, B), what="1000x128x1000")
    ctx.gemm(1, 1000, 128, 1000, ctx.array(A), 1000, ctx.array(B), 1000, dC, 1000)
    ctx.sync()
    assert_close(dC.get(), o.gemm_tn(A, B), what="1000x128x1000 transposed")


# ------------------------------------------------------------------------------------------------ A3-A5 LSTM node
LSTM_SHAPES = [(32, 3), (100, 8), (72, 33), (250, 70)]


@pytest.mark.parametrize("H,mb", LSTM_SHAPES)
@pytest.mark.parametrize("tn,ks", [(0, 0), (1, 4), (1, 8), (2, 4), (2, 8), (4, 4)])
def test_lstm_step_fused(ctx, H, mb, tn, ks):
    g = synth.rng(6, H * 1000 + mb)
    ly = synth.lstm_layer(g, H, forget_bias_one=True)
    x, hp, cp = U(g, (H, mb), -1, 1), U(g, (H, mb), -1, 1), U(g, (H, mb), -1, 1)
    mask = (g.random(mb) > 0.2).astype(np.int32)
    layer = Layer(ctx, ly)
    ctx.set_option(capi.ZR_OPT_LSTM_TN, tn)
    ctx.set_option(capi.ZR_OPT_LSTM_KSPLIT, ks)
    try:
        got = run_lstm_step(ctx, layer, x, hp, cp, mask, want_gates=True)
    finally:
        ctx.set_option(capi.ZR_OPT_LSTM_TN, 0)
        ctx.set_option(capi.ZR_OPT_LSTM_KSPLIT, 0)
        layer.close()
    want = o.lstm_step(ly["M"], ly["Wh"], ly["b"], x, hp, cp, mask)
    for k in ("i", "f", "c_tilde", "o", "c", "h"):
        assert_close(got[k], want[k], what="%s (H=%d mb=%d tn=%d ks=%d)" % (k, H, mb, tn, ks))
    dead = mask == 0
    assert np.all(got["h"][:, dead] == 0) and np.all(got["c"][:, dead] == 0)


@pytest.mark.parametrize("fused", [1, 0])
def test_lstm_step_feed_input_clip_and_unfused(ctx, fused):
    g = synth.rng(7, fused)
    H, mb = 100, 8
    ly = synth.lstm_layer(g, H, feed_input=True)
    x, hp, ht = U(g, (H, mb), -1, 1), U(g, (H, mb), -1, 1), U(g, (H, mb), -1, 1)
    cp = U(g, (H, mb), -3, 3)
    mask = np.array([1, 1, 0, 1, 1, 1, 0, 1], np.int32)
    layer = Layer(ctx, ly)
    ctx.set_option(capi.ZR_OPT_LSTM_FUSED_EPILOGUE, fused)
    try:
        got_feed = run_lstm_step(ctx, layer, x, hp, cp, mask, htild=ht, clip=0.6, want_gates=True)
        got_plain = run_lstm_step(ctx, layer, x, hp, cp, mask)  # index 0: Q skipped although packed
    finally:
        ctx.set_option(capi.ZR_OPT_LSTM_FUSED_EPILOGUE, 1)
        layer.close()
    want_feed = o.lstm_step(ly["M"], ly["Wh"], ly["b"], x, hp, cp, mask, Q=ly["Q"], htild=ht, clip=0.6)
    want_plain = o.lstm_step(ly["M"], ly["Wh"], ly["b"], x, hp, cp, mask)
    for k in ("i", "f", "c_tilde", "o", "c", "h"):
        assert_close(got_feed[k], want_feed[k], what="feed " + k)
    assert np.all(np.abs(got_feed["c"]) <= 0.6)
    assert_close(got_plain["h"], want_plain["h"], what="plain h")
    assert_close(got_plain["c"], want_plain["c"], what="plain c")


def test_lstm_gates_kernel_closed_forms(ctx):
    """Stand-alone gate kernel on given pre-activations: zero pre-activations and saturation."""
    H, mb = 1000, 16
    g = synth.rng(8, 1)
    cp = U(g, (H, mb), -2, 2)
    zero_b = [ctx.zeros((H,)) for _ in range(4)]
    dh, dc = ctx.empty((H, mb)), ctx.empty((H, mb))
    ctx.lstm_gates(ctx.zeros((4 * H * mb,)), zero_b, ctx.array(cp), ctx.array(np.ones(mb, np.int32)), H, mb, dh, dc)
    ctx.sync()
    assert np.array_equal(dc.get(), 0.5 * cp)
    assert_close(dh.get(), 0.5 * np.tanh(0.5 * cp.astype(np.float64)), what="h at zero pre-activation")
    pre = np.concatenate([np.full(H * mb, v, np.float32) for v in (40.0, -40.0, 40.0, 40.0)])
    ctx.lstm_gates(ctx.array(pre), zero_b, ctx.array(cp), ctx.array(np.ones(mb, np.int32)), H, mb, dh, dc)
    ctx.sync()
    assert np.all(dc.get() == 1.0) and np.allclose(dh.get(), np.tanh(1.0), atol=1e-6)


def test_lstm_step_full_size_layer(ctx):
    """One layer-step at the benchmark shape (H=1000, mb=128), with and without feed-input."""
    g = synth.rng(9, 1)
    H, mb = 1000, 128
    ly = synth.lstm_layer(g, H, feed_input=True, forget_bias_one=True)
    x, hp, cp, ht = (U(g, (H, mb), -0.08, 0.08), np.tanh(U(g, (H, mb), -1, 1)) * np.float32(0.5),
                     U(g, (H, mb), -0.5, 0.5), np.tanh(U(g, (H, mb), -1, 1)))
    mask = np.ones(mb, np.int32)
    layer = Layer(ctx, ly)
    try:
        got = run_lstm_step(ctx, layer, x, hp, cp, mask)
        got_feed = run_lstm_step(ctx, layer, x, hp, cp, mask, htild=ht)
    finally:
        layer.close()
    want = o.lstm_step(ly["M"], ly["Wh"], ly["b"], x, hp, cp, mask)
    want_feed = o.lstm_step(ly["M"], ly["Wh"], ly["b"], x, hp, cp, mask, Q=ly["Q"], htild=ht)
    assert_close(got["h"], want["h"], what="h")
    assert_close(got["c"], want["c"], what="c")
    assert_close(got_feed["h"], want_feed["h"], what="h feed")
    assert_close(got_feed["c"], want_feed["c"], what="c feed")


# ------------------------------------------------------------------------------------------------ A6/A7/A11 stack
def _run_stack(ctx, cfg_layers, embed, ids, h0=None, c0=None, clip=0.0, expect_path=None):
    """expect_path: the schedule zr_lstm_stack_forward must have taken (capi.ZR_LSTM_STACK_PATH_*), asserted."""
    H, V = embed.shape
    T, mb = ids.shape
    L = len(cfg_layers)
    layers = [Layer(ctx, ly) for ly in cfg_layers]
    d_ids = ctx.array(ids.reshape(-1))
    d_nn, d_m = ctx.empty(ids.size, np.int32), ctx.empty(ids.size, np.int32)
    ctx.vocab_prep(d_ids, ids.size, V, d_nn, d_m)
    z = ctx.zeros((H, mb))
    d_h0 = [ctx.array(h0[l]) if h0 is not None else z for l in range(L)]
    d_c0 = [ctx.array(c0[l]) if c0 is not None else z for l in range(L)]
    h_all = [ctx.empty((H * mb * T,)) for _ in range(L)]
    c_all = [ctx.empty((H * mb * T,)) for _ in range(L)]
    ctx.lstm_stack_forward([ly.w for ly in layers], ctx.array(embed), V, d_nn, d_m, T, mb, d_h0, d_c0, h_all, c_all,
                           clip=clip)
    if expect_path is not None:
        assert ctx.query(capi.ZR_QUERY_LSTM_STACK_PATH) == expect_path, "zr_lstm_stack_forward took the other schedule"
    ctx.sync()
    hs = np.stack([a.get().reshape(T, mb, H).transpose(0, 2, 1) for a in h_all])
    cs = np.stack([a.get().reshape(T, mb, H).transpose(0, 2, 1) for a in c_all])
    for ly in layers:
        ly.close()
    return hs, cs


def test_stack_forward_small_with_padding(ctx):
    g = synth.rng(10, 1)
    H, mb, T, V, L = 64, 5, 7, 211, 3
    embed = U(g, (H, V))
    layers = [synth.lstm_layer(g, H, forget_bias_one=True) for _ in range(L)]
    ids = g.integers(0, V, size=(T, mb)).astype(np.int32)
    ids[:3, 1] = -1  # left padding, as the source side is laid out
    ids[:5, 4] = -1
    hs, cs = _run_stack(ctx, layers, embed, ids)
    nn, m = o.vocab_prep(ids)
    want_h, want_c = o.lstm_stack_forward(embed, layers, nn, m)
    assert_close(hs, want_h, what="stack h")
    assert_close(cs, want_c, what="stack c")
    assert np.all(hs[:, :3, :, 1] == 0) and np.all(cs[:, :5, :, 4] == 0)


def test_config1_lm_forward_logprobs_and_loss(ctx):
    """benchmark configuration 1: 1-layer LM, H=100, mb=8, T=20, V=10000; per-step full log-probs and the summed loss."""
    c = synth.config1()
    H, mb, T, V = c["H"], c["mb"], c["T"], c["V"]
    hs, _ = _run_stack(ctx, c["layers"], c["embed"], c["ids"])
    nn, m = o.vocab_prep(c["ids"])
    want_h, _ = o.lstm_stack_forward(c["embed"], c["layers"], nn, m)
    assert_close(hs, want_h, what="LM h")
    dD, dbd = ctx.array(c["D"]), ctx.array(c["b_d"])
    d_logp, d_logp64, d_scr = ctx.empty((V, mb)), ctx.empty((V, mb), np.float64), ctx.empty((V, mb))
    total, want_total = 0.0, 0.0
    for t in range(T):
        h_t = np.asfortranarray(hs[0, t])
        d_h = ctx.array(h_t)
        ctx.softmax_forward(dD, dbd, V, H, d_h, mb, capi.ZR_SOFTMAX_LOGPROB, d_logp)
        ctx.softmax_logprob_f64(dD, dbd, V, H, d_h, mb, d_logp64, d_scr)
        ctx.sync()
        want = o.softmax_logprob_f64(o.softmax_logits(c["D"], c["b_d"], np.asfortranarray(want_h[0, t])))
        assert_close(d_logp.get(), want, what="log-probs step %d" % t)
        assert_close(d_logp64.get(), want, what="f64 log-probs step %d" % t)
        tgt = c["targets"][t]
        total += ctx.softmax_loss(dD, dbd, V, H, d_h, mb, ctx.array(tgt), ctx.array(np.ones(mb, np.int32)), d_scr)
        want_total += o.softmax_loss(want, tgt, np.ones(mb, np.int32))
    assert total == pytest.approx(want_total, rel=1e-5)


# ------------------------------------------------------------------------------------------------ A8/A9 softmax
@pytest.mark.parametrize("prepared", [False, True])
@pytest.mark.parametrize("V,H,mb", [(211, 16, 6), (10000, 100, 8), (4099, 64, 33), (1003, 27, 70), (8300, 40, 128),
                                    (8400, 24, 100), (16500, 32, 192), (9000, 16, 40), (9100, 24, 64), (8250, 16, 320)])
def test_softmax_prob_and_logprob(ctx, V, H, mb, prepared):
    """prepared: the output matrix registered with zr_softmax_prepare (k-interleaved copy); same results.  The shapes
    with more than 8192 rows take the tall-matrix kernels when prepared: 64-row tiles of 128, 96 or 64 columns where
    the minibatch is a multiple of those (128; 192; 64 and 320), row ranges with 32-column pieces otherwise (100 and
    40 columns, the last column tile partly filled); the rows beyond the last full tile go to the small tiles."""
    g = synth.rng(11, V)
    D, bd, h = U(g, (V, H), -1, 1), U(g, (V,), -1, 1), U(g, (H, mb), -1, 1)
    dD, dbd, dh = ctx.array(D), ctx.array(bd), ctx.array(h)
    if prepared:
        ctx.softmax_prepare(dD, V, H)
    d_p, d_lp, d_scr = ctx.empty((V, mb)), ctx.empty((V, mb)), ctx.empty((V, mb))
    ctx.softmax_forward(dD, dbd, V, H, dh, mb, capi.ZR_SOFTMAX_PROB, d_p, d_scr)
    ctx.softmax_forward(dD, dbd, V, H, dh, mb, capi.ZR_SOFTMAX_LOGPROB, d_lp)  # in place on the logits
    ctx.sync()
    logits = o.softmax_logits(D, bd, h)
    assert_close(d_scr.get(), logits, what="logits")
    P = d_p.get()
    assert_close(P, o.softmax_dist(logits), floor=1e-7, what="probabilities")
    assert np.allclose(P.sum(axis=0, dtype=np.float64), 1.0, atol=1e-5)
    assert np.array_equal(P.argmax(axis=0), logits.argmax(axis=0))
    assert_close(d_lp.get(), o.softmax_logprob_f64(logits), what="log-probs")
    # masked loss with out-of-order targets
    tgt = g.integers(0, V, size=mb).astype(np.int32)
    mask = (g.random(mb) > 0.3).astype(np.int32)
    got = ctx.softmax_loss(dD, dbd, V, H, dh, mb, ctx.array(tgt), ctx.array(mask), d_scr)
    assert got == pytest.approx(o.softmax_loss(o.softmax_logprob_f64(logits), tgt, mask), rel=1e-5, abs=1e-6)
    if prepared:
        # re-packing after a change of D is picked up; releasing returns to the plain path
        D2 = np.asfortranarray(-D)
        dD.set(D2)
        ctx.softmax_prepare(dD, V, H)
        ctx.softmax_forward(dD, dbd, V, H, dh, mb, capi.ZR_SOFTMAX_LOGPROB, d_lp, d_scr)
        ctx.sync()
        assert_close(d_scr.get(), o.softmax_logits(D2, bd, h), what="logits after re-pack")
        ctx.softmax_release(dD)
        ctx.softmax_forward(dD, dbd, V, H, dh, mb, capi.ZR_SOFTMAX_LOGPROB, d_lp, d_scr)
        ctx.sync()
        assert_close(d_scr.get(), o.softmax_logits(D2, bd, h), what="logits after release")


def test_softmax_extreme_logits_no_overflow(ctx):
    V, H, mb = 512, 4, 3
    D = np.zeros((V, H), np.float32, order="F")
    D[:, 0] = np.where(np.arange(V) % 3 == 0, 80.0, -80.0)
    h = np.zeros((H, mb), np.float32, order="F")
    h[0, :] = [1.0, -1.0, 0.0]
    d_p = ctx.empty((V, mb))
    ctx.softmax_forward(ctx.array(D), ctx.zeros((V,)), V, H, ctx.array(h), mb, capi.ZR_SOFTMAX_PROB, d_p)
    ctx.sync()
    P = d_p.get()
    assert np.all(np.isfinite(P)) and np.allclose(P.sum(axis=0, dtype=np.float64), 1.0, atol=1e-5)
    assert np.allclose(P[:, 2], 1.0 / V)  # zero logits -> uniform


@pytest.mark.parametrize("prepared", [False, True])
def test_softmax_full_vocab_properties(ctx, prepared):
    """V=50000, H=1000, mb=128 (the benchmark shape): size-independent properties plus an exact check of a
    sampled set of columns against the oracle."""
    g = synth.rng(12, 1)
    V, H, mb = 50000, 1000, 128
    D, bd = U(g, (V, H)), U(g, (V,))
    h = np.tanh(U(g, (H, mb), -1, 1))
    dD, dbd = ctx.array(D), ctx.array(bd)
    if prepared:
        ctx.softmax_prepare(dD, V, H)
    d_p, d_scr = ctx.empty((V, mb)), ctx.empty((V, mb))
    ctx.softmax_forward(dD, dbd, V, H, ctx.array(h), mb, capi.ZR_SOFTMAX_PROB, d_p, d_scr)
    ctx.sync()
    P, logits = d_p.get(), d_scr.get()
    assert np.allclose(P.sum(axis=0, dtype=np.float64), 1.0, atol=1e-5)
    assert np.array_equal(P.argmax(axis=0), logits.argmax(axis=0))
    cols = [0, 31, 32, 77, 127]
    want_logits = o.softmax_logits(D, bd, np.asfortranarray(h[:, cols]))
    assert_close(logits[:, cols], want_logits, what="logits (sampled columns)")
    assert_close(P[:, cols], o.softmax_dist(want_logits), floor=1e-7, what="probabilities (sampled columns)")
    if prepared:
        ctx.softmax_release(dD)


@pytest.mark.parametrize("V,mb", [(50000, 12), (50000, 1), (50033, 32), (2100, 5)])
def test_softmax_at_decode_width(ctx, V, mb):
    """The output layer at the reference's own decode shape -- one sentence, minibatch = beam (src/model.hpp:491-492,553)
    -- and at a single column: with a prepared matrix and at most 32 columns the logits product is a stream of the matrix
    (every wave a pair of 32-row blocks over all of K; an odd number of blocks, a ragged last block and a vocabulary of
    less than one workgroup's share are among the shapes).  Logits, probabilities and log-probs against the oracle."""
    g = synth.rng(14, V + mb)
    H = 1000
    D, bd = U(g, (V, H)), U(g, (V,))
    h = np.tanh(U(g, (H, mb), -1, 1))
    dD, dbd, dh = ctx.array(D), ctx.array(bd), ctx.array(h)
    ctx.softmax_prepare(dD, V, H)
    d_p, d_lp, d_scr = ctx.empty((V, mb)), ctx.empty((V, mb)), ctx.empty((V, mb))
    ctx.softmax_forward(dD, dbd, V, H, dh, mb, capi.ZR_SOFTMAX_PROB, d_p, d_scr)
    ctx.softmax_forward(dD, dbd, V, H, dh, mb, capi.ZR_SOFTMAX_LOGPROB, d_lp)
    ctx.sync()
    want_logits = o.softmax_logits(D, bd, h)
    assert_close(d_scr.get(), want_logits, what="logits")
    P = d_p.get()
    assert_close(P, o.softmax_dist(want_logits), floor=1e-7, what="probabilities")
    assert np.allclose(P.sum(axis=0, dtype=np.float64), 1.0, atol=1e-5)
    assert_close(d_lp.get(), o.softmax_logprob_f64(want_logits), what="log-probs")
    ctx.softmax_release(dD)


# ------------------------------------------------------------------------------------------------ A10 attention
def _run_attention(ctx, w, hs, batch_info, h_t, mask, D, prepared=False):
    """prepared: zr_attn_prepare first (the three-launch path on snapshots of the matrices)."""
    S, H, mb = hs.shape
    tables = [ctx.array(np.asfortranarray(hs[t])) for t in range(S)]
    dw = {k: ctx.array(v) for k, v in w.items()}
    a = ctx.attn_create(H, mb, D, dw["W_a"], dw["W_p"], dw["v_p"], dw["out_bias"], dw["W_c1"], dw["W_c2"], tables)
    if prepared:
        ctx.attn_prepare(a)
    Wn = 2 * D + 1
    d_ht, d_al, d_ix, d_pt, d_cx = (ctx.empty((H, mb)), ctx.empty((mb, Wn)), ctx.empty((mb, Wn), np.int32),
                                    ctx.empty((mb,)), ctx.empty((H, mb)))
    ctx.attn_step(a, ctx.array(batch_info), ctx.array(h_t), ctx.array(mask), d_ht, d_al, d_ix, d_pt, d_cx)
    ctx.sync()
    out = {"h_tild": d_ht.get(), "alignments": d_al.get(), "indices": d_ix.get(), "p_t": d_pt.get(),
           "c_ctx": d_cx.get()}
    ctx.attn_destroy(a)
    return out


@pytest.mark.parametrize("prepared", [False, True])
@pytest.mark.parametrize("H,mb,S,D", [(64, 6, 9, 2), (100, 8, 20, 10), (52, 33, 12, 12), (30, 5, 7, 3), (1028, 70, 40, 100),
                                      (2052, 9, 6, 1), (256, 3, 300, 255),
                                      # 1024 < H <= 2048: the eight-wave register-resident kernel up to 52 window slots
                                      # (50 and exactly 52), the two-pass kernel beyond (53)
                                      (2000, 20, 50, 50), (1500, 12, 52, 30), (2048, 5, 53, 40)])
def test_attention_against_oracle(ctx, H, mb, S, D, prepared):
    g = synth.rng(13, H + S)
    w = synth.attention_weights(g, H)
    if H <= 128:  # small layers get wider matrices so that the scores spread; large ones keep the model's own range
        for k in ("W_a", "W_p", "W_c1", "W_c2"):
            w[k] = U(g, (H, H), -0.3, 0.3)
    # scores are H-term dot products: keep their spread (and with it the conditioning of the softmax) the same for
    # the large layers as for the small ones; the benchmark's own distribution is covered by the config-3 test
    hs = (g.standard_normal(size=(S, H, mb), dtype=np.float32) * np.float32(0.5 if H <= 128 else 0.1))
    lens = g.integers(1, S + 1, size=mb).astype(np.int32)
    lens[0] = S
    batch_info = np.concatenate([lens, S - lens]).astype(np.int32)
    mask = (g.random(mb) > 0.15).astype(np.int32)
    h_t = U(g, (H, mb), -1, 1)
    want = o.attention_forward(hs_table=hs, batch_info=batch_info, h_t=h_t, mask01=mask, D=D, **w)
    got = _run_attention(ctx, w, hs, batch_info, h_t, mask, D, prepared)
    assert_close(got["p_t"], want["p_t"], what="p_t")
    # the window is floor(p_t) +- D: a p_t within rounding of an integer could legitimately move it
    frac = want["p_t"] - np.floor(want["p_t"])
    safe = (frac > 1e-4) & (frac < 1 - 1e-4)
    assert safe.all(), "test inputs put p_t on an integer boundary; pick another seed"
    assert np.array_equal(got["indices"], want["indices"])
    assert_close(got["alignments"], want["alignments"], floor=1e-4, what="alignments")
    assert_close(got["c_ctx"], want["c_ctx"], what="context")
    assert_close(got["h_tild"], want["h_tild"], what="h_tild")
    assert np.all(got["h_tild"][:, mask == 0] == 0)


@pytest.mark.parametrize("H,mb,S,D", [(1000, 128, 50, 50), (64, 6, 9, 2), (200, 70, 40, 10), (1024, 33, 64, 31),
                                      (512, 12, 21, 10), (96, 1, 5, 7), (1000, 12, 50, 10), (1000, 1, 50, 10),
                                      (1000, 192, 30, 10), (256, 250, 20, 5)])
def test_attention_step_in_one_launch(ctx, H, mb, S, D):
    """The attention step as one launch (projections, per-column middle and output product handing over through device
    memory): against the oracle, against the three-launch schedule on the same inputs, and twice in a row on one
    attention object (the counters go back to zero inside the launch)."""
    g = synth.rng(17, H + S + mb)
    w = synth.attention_weights(g, H)
    hs = (g.standard_normal(size=(S, H, mb), dtype=np.float32) * np.float32(0.5 if H <= 128 else 0.1))
    lens = g.integers(1, S + 1, size=mb).astype(np.int32)
    lens[0] = S
    batch_info = np.concatenate([lens, S - lens]).astype(np.int32)
    mask = (g.random(mb) > 0.15).astype(np.int32)
    mask[0] = 1
    h_t = U(g, (H, mb), -1, 1)
    want = o.attention_forward(hs_table=hs, batch_info=batch_info, h_t=h_t, mask01=mask, D=D, **w)
    frac = want["p_t"] - np.floor(want["p_t"])
    assert ((frac > 1e-4) & (frac < 1 - 1e-4)).all(), "test inputs put p_t on an integer boundary; pick another seed"
    tables = [ctx.array(np.asfortranarray(hs[t])) for t in range(S)]
    dw = {k: ctx.array(v) for k, v in w.items()}
    a = ctx.attn_create(H, mb, D, dw["W_a"], dw["W_p"], dw["v_p"], dw["out_bias"], dw["W_c1"], dw["W_c2"], tables)
    ctx.attn_prepare(a)
    Wn = 2 * D + 1
    d_bi, d_h, d_m = ctx.array(batch_info), ctx.array(h_t), ctx.array(mask)

    def run():
        outs = (ctx.empty((H, mb)), ctx.empty((mb, Wn)), ctx.empty((mb, Wn), np.int32), ctx.empty((mb,)),
                ctx.empty((H, mb)))
        ctx.attn_step(a, d_bi, d_h, d_m, *outs)
        ctx.sync()
        return [x.get() for x in outs]

    try:
        one = run()
        assert ctx.query(capi.ZR_QUERY_ATTN_PATH) == capi.ZR_ATTN_PATH_SINGLE_LAUNCH
        again = run()
        ctx.set_option(capi.ZR_OPT_ATTN_SINGLE_LAUNCH, 1)
        three = run()
        assert ctx.query(capi.ZR_QUERY_ATTN_PATH) == capi.ZR_ATTN_PATH_THREE_LAUNCHES
    finally:
        ctx.set_option(capi.ZR_OPT_ATTN_SINGLE_LAUNCH, 0)
        ctx.attn_destroy(a)
    names = ("h_tild", "alignments", "indices", "p_t", "c_ctx")
    for name, x, y in zip(names, one, again):
        assert np.array_equal(x, y), name + " differs between two launches"
    got = dict(zip(names, one))
    assert_close(got["p_t"], want["p_t"], what="p_t")
    assert np.array_equal(got["indices"], want["indices"])
    assert_close(got["alignments"], want["alignments"], floor=1e-4, what="alignments")
    assert_close(got["c_ctx"], want["c_ctx"], what="context")
    assert_close(got["h_tild"], want["h_tild"], what="h_tild")
    assert np.all(got["h_tild"][:, mask == 0] == 0)
    other = dict(zip(names, three))
    assert np.array_equal(got["indices"], other["indices"])
    assert_close(got["h_tild"], other["h_tild"], what="h_tild, one launch against three")
    assert_close(got["c_ctx"], other["c_ctx"], what="context, one launch against three")


@pytest.mark.parametrize("mb,D", [(7, 4), (130, 50), (3, 255)])
def test_attention_viterbi_alignment_bit_exact(ctx, mb, D):
    """zr_attn_viterbi against the oracle on crafted weights: ties (first maximum wins), all-zero live columns, masked
    columns and short windows; then on the alignments of a real attention step."""
    g = synth.rng(31, mb + D)
    Wn = 2 * D + 1
    al = np.asfortranarray(g.random((mb, Wn), dtype=np.float32))
    ix = np.asfortranarray(g.integers(0, 300, size=(mb, Wn)).astype(np.int32))
    al[1, 2] = al[1, Wn - 1] = 2.0
    al[2, :] = 0.0
    al[0, :], ix[0, :] = 0.0, -1
    if mb > 5:
        al[5, 5:], ix[5, 5:] = 0.0, -1
        al[6, 70 % Wn] = al[6, 3] = 3.0  # tie across lanes: lower slot wins
    H = 8
    tables = [ctx.zeros((H, mb))]
    z = ctx.zeros((H, H))
    a = ctx.attn_create(H, mb, D, z, z, ctx.zeros((H,)), ctx.zeros((H,)), z, z, tables)
    d_out = ctx.empty((mb,), np.int32)
    ctx.attn_viterbi(a, ctx.array(al), ctx.array(ix), d_out)
    ctx.sync()
    assert d_out.get().tolist() == o.attention_viterbi(al, ix).tolist()
    ctx.attn_destroy(a)


def test_attention_viterbi_after_a_step(ctx):
    H, mb, S, D = 64, 9, 12, 3
    g = synth.rng(32, 1)
    w = synth.attention_weights(g, H)
    hs = (g.standard_normal(size=(S, H, mb), dtype=np.float32) * np.float32(0.5))
    lens = g.integers(2, S + 1, size=mb).astype(np.int32)
    bi = np.concatenate([lens, S - lens]).astype(np.int32)
    mask = np.ones(mb, np.int32)
    mask[4] = 0
    h_t = U(g, (H, mb), -1, 1)
    tables = [ctx.array(np.asfortranarray(hs[t])) for t in range(S)]
    dw = {k: ctx.array(v) for k, v in w.items()}
    a = ctx.attn_create(H, mb, D, dw["W_a"], dw["W_p"], dw["v_p"], dw["out_bias"], dw["W_c1"], dw["W_c2"], tables)
    ctx.attn_prepare(a)
    d_ht, d_out = ctx.empty((H, mb)), ctx.empty((mb,), np.int32)
    ctx.attn_step(a, ctx.array(bi), ctx.array(h_t), ctx.array(mask), d_ht)  # internal alignment / index arrays
    ctx.attn_viterbi(a, None, None, d_out)
    ctx.sync()
    want = o.attention_forward(hs_table=hs, batch_info=bi, h_t=h_t, mask01=mask, D=D, **w)
    assert d_out.get().tolist() == o.attention_viterbi(want["alignments"], want["indices"]).tolist()
    assert d_out.get()[4] == -1
    ctx.attn_destroy(a)


@pytest.mark.parametrize("prepared", [False, True])
def test_attention_negative_scores_use_zero_initialised_max(ctx, prepared):
    """All scores very negative: the reference's max starts at 0, exp underflows, the sum is 0 and the
    alignments stay 0 (a -inf initialised max would give a normalised distribution instead)."""
    H, mb, S, D = 8, 2, 5, 5
    g = synth.rng(14, 1)
    w = synth.attention_weights(g, H)
    w["W_a"] = np.asfortranarray(-200.0 * np.eye(H, dtype=np.float32))
    hs = np.ones((S, H, mb), np.float32)
    h_t = np.ones((H, mb), np.float32, order="F")
    bi = np.concatenate([np.full(mb, S, np.int32), np.zeros(mb, np.int32)])
    got = _run_attention(ctx, w, hs, bi, h_t, np.ones(mb, np.int32), D, prepared)
    want = o.attention_forward(hs_table=hs, batch_info=bi, h_t=h_t, mask01=np.ones(mb, np.int32), D=D, **w)
    assert np.all(got["alignments"] == 0) and np.all(want["alignments"] == 0)
    assert_close(got["h_tild"], want["h_tild"], what="h_tild")


def test_config3_decoder_step_reduced_vocab(ctx):
    """benchmark configuration 3 wiring at H=1000, mb=128, S=50 with D=50 ("global") and D=10: LSTM stack with
    feed-input on layer 0, attention on the top layer, softmax over a reduced vocabulary so that the oracle
    finishes in seconds (the full-vocabulary softmax is covered by test_softmax_full_vocab_properties)."""
    c = synth.decoder_config(V=2000)
    H, mb, S, L, V = c["H"], c["mb"], c["S"], c["L"], c["V"]
    mask = np.ones(mb, np.int32)
    # oracle
    x = o.embed_gather(c["embed"], c["ids"])
    below, want_states = x, []
    for l in range(L):
        ly = c["layers"][l]
        r = o.lstm_step(ly["M"], ly["Wh"], ly["b"], below, c["h_prev"][l], c["c_prev"][l], mask,
                        Q=ly.get("Q"), htild=c["h_tild_prev"] if l == 0 else None)
        want_states.append(r)
        below = r["h"]
    # HIP path
    layers = [Layer(ctx, ly) for ly in c["layers"]]
    d_x = ctx.empty((H, mb))
    ctx.embed_gather(ctx.array(c["embed"]), H, V, ctx.array(c["ids"]), mb, d_x)
    d_mask, d_ht_prev = ctx.array(mask), ctx.array(c["h_tild_prev"])
    d_below, outs = d_x, []
    for l in range(L):
        d_h, d_c = ctx.empty((H, mb)), ctx.empty((H, mb))
        ctx.lstm_step(layers[l].w, d_below, ctx.array(c["h_prev"][l]), ctx.array(c["c_prev"][l]), d_mask, mb, d_h,
                      d_c, d_htild=d_ht_prev if l == 0 else None)
        outs.append((d_h, d_c))
        d_below = d_h
    ctx.sync()
    for l in range(L):
        assert_close(outs[l][0].get(), want_states[l]["h"], what="layer %d h" % l)
        assert_close(outs[l][1].get(), want_states[l]["c"], what="layer %d c" % l)
    top_h = outs[-1][0].get()
    for D, prepared in ((50, False), (50, True), (10, False), (10, True)):
        want_att = o.attention_forward(hs_table=c["hs"], batch_info=c["batch_info"], h_t=top_h, mask01=mask, D=D,
                                       **c["attn"])
        got_att = _run_attention(ctx, c["attn"], c["hs"], c["batch_info"], top_h, mask, D, prepared)
        frac = want_att["p_t"] - np.floor(want_att["p_t"])
        safe = (frac > 1e-4) & (frac < 1 - 1e-4)
        assert np.array_equal(got_att["indices"][safe], want_att["indices"][safe])
        assert_close(got_att["alignments"][safe], want_att["alignments"][safe], floor=1e-4, what="alignments D=%d" % D)
        assert_close(got_att["h_tild"][:, safe], want_att["h_tild"][:, safe], what="h_tild D=%d" % D)
        if D == 50:  # every source position has a slot
            assert np.all((want_att["indices"][:, :S] == np.arange(S)[None, :]))
    d_lp = ctx.empty((V, mb))
    ctx.softmax_forward(ctx.array(c["D"]), ctx.array(c["b_d"]), V, H, ctx.array(got_att["h_tild"]), mb,
                        capi.ZR_SOFTMAX_LOGPROB, d_lp)
    ctx.sync()
    want_lp = o.softmax_logprob_f64(o.softmax_logits(c["D"], c["b_d"], got_att["h_tild"]))
    assert_close(d_lp.get(), want_lp, what="log-probs")
    for ly in layers:
        ly.close()


# ------------------------------------------------------------------------------------------------ error handling
def test_bad_arguments_return_errors(ctx):
    with pytest.raises(capi.ZrError) as e:
        ctx.gemm(0, 0, 4, 4, 1, 1, 1, 1, 1, 1)
    assert e.value.code == -1
    with pytest.raises(capi.ZrError):
        ctx.embed_gather(None, 8, 8, None, 4, None)
    with pytest.raises(capi.ZrError):
        ctx.lstm_step(None, 1, 1, 1, 1, 4, 1, 1)
    g = synth.rng(15, 1)
    layer = Layer(ctx, synth.lstm_layer(g, 16))
    buf = ctx.zeros((16, 4))
    with pytest.raises(capi.ZrError):  # feed-input requested on weights packed without Q
        ctx.lstm_step(layer.w, buf, buf, buf, ctx.array(np.ones(4, np.int32)), 4, ctx.empty((16, 4)), ctx.empty((16, 4)),
                      d_htild=buf)
    layer.close()


# ------------------------------------------------------------------------------------------------ split-K LSTM kernel
@pytest.mark.parametrize("H,mb", [(32, 3), (100, 8), (72, 33), (252, 70), (1000, 128), (64, 150)])
@pytest.mark.parametrize("kparts", [0, 1, 2, 3, 5])
def test_lstm_step_lds_split_kernel(ctx, H, mb, kparts):
    """The LDS / split-K kernel forced on every shape (it is picked automatically only for wide batches): odd chunk
    counts, partial row tiles, partial column tiles, several K parts, with and without the feed-input segment."""
    g = synth.rng(16, H * 1000 + mb + kparts)
    ly = synth.lstm_layer(g, H, feed_input=True, forget_bias_one=True)
    x, hp, cp, ht = U(g, (H, mb), -1, 1), U(g, (H, mb), -1, 1), U(g, (H, mb), -1, 1), U(g, (H, mb), -1, 1)
    mask = (g.random(mb) > 0.2).astype(np.int32)
    layer = Layer(ctx, ly)
    ctx.set_option(capi.ZR_OPT_LSTM_KERNEL, 2)
    ctx.set_option(capi.ZR_OPT_LSTM_KPARTS, kparts)
    try:
        got = run_lstm_step(ctx, layer, x, hp, cp, mask, want_gates=True)
        got_feed = run_lstm_step(ctx, layer, x, hp, cp, mask, htild=ht, clip=0.7)
        again = run_lstm_step(ctx, layer, x, hp, cp, mask, htild=ht, clip=0.7)
    finally:
        ctx.set_option(capi.ZR_OPT_LSTM_KERNEL, 0)
        ctx.set_option(capi.ZR_OPT_LSTM_KPARTS, 0)
        layer.close()
    want = o.lstm_step(ly["M"], ly["Wh"], ly["b"], x, hp, cp, mask)
    want_feed = o.lstm_step(ly["M"], ly["Wh"], ly["b"], x, hp, cp, mask, Q=ly["Q"], htild=ht, clip=0.7)
    for k in ("i", "f", "c_tilde", "o", "c", "h"):
        assert_close(got[k], want[k], what="%s (H=%d mb=%d kparts=%d)" % (k, H, mb, kparts))
    assert_close(got_feed["h"], want_feed["h"], what="feed h")
    assert_close(got_feed["c"], want_feed["c"], what="feed c")
    # the cross-workgroup reduction adds partials in a fixed order: bit-identical from run to run
    assert got_feed["h"].tobytes() == again["h"].tobytes() and got_feed["c"].tobytes() == again["c"].tobytes()


@pytest.mark.parametrize("H,mb", [(32, 3), (104, 8), (72, 33), (256, 70), (1000, 128), (64, 150), (1000, 192), (1000, 12)])
@pytest.mark.parametrize("kparts", [0, 2, 3, 5])
def test_lstm_step_register_kernel_split_across_workgroups(ctx, H, mb, kparts):
    """The register-streaming kernel with K divided over several workgroups per tile (H % 8 == 0): column tiles of 32,
    64 and 96, uneven K parts, partial row and column tiles, two and three weight segments; a request for more parts
    than k-groups falls back to another kernel and must still be right."""
    g = synth.rng(19, H * 1000 + mb + kparts)
    ly = synth.lstm_layer(g, H, feed_input=True, forget_bias_one=True)
    x, hp, cp, ht = U(g, (H, mb), -1, 1), U(g, (H, mb), -1, 1), U(g, (H, mb), -1, 1), U(g, (H, mb), -1, 1)
    mask = (g.random(mb) > 0.2).astype(np.int32)
    layer = Layer(ctx, ly)
    ctx.set_option(capi.ZR_OPT_LSTM_KERNEL, 3)
    ctx.set_option(capi.ZR_OPT_LSTM_KPARTS, kparts)
    try:
        got = run_lstm_step(ctx, layer, x, hp, cp, mask, want_gates=True)
        got_feed = run_lstm_step(ctx, layer, x, hp, cp, mask, htild=ht, clip=0.7)
        again = run_lstm_step(ctx, layer, x, hp, cp, mask, htild=ht, clip=0.7)
    finally:
        ctx.set_option(capi.ZR_OPT_LSTM_KERNEL, 0)
        ctx.set_option(capi.ZR_OPT_LSTM_KPARTS, 0)
        layer.close()
    want = o.lstm_step(ly["M"], ly["Wh"], ly["b"], x, hp, cp, mask)
    want_feed = o.lstm_step(ly["M"], ly["Wh"], ly["b"], x, hp, cp, mask, Q=ly["Q"], htild=ht, clip=0.7)
    for k in ("i", "f", "c_tilde", "o", "c", "h"):
        assert_close(got[k], want[k], what="%s (H=%d mb=%d kparts=%d)" % (k, H, mb, kparts))
    assert_close(got_feed["h"], want_feed["h"], what="feed h")
    assert_close(got_feed["c"], want_feed["c"], what="feed c")
    assert got_feed["h"].tobytes() == again["h"].tobytes() and got_feed["c"].tobytes() == again["c"].tobytes()


@pytest.mark.parametrize("H,mb,feed,fused", [(64, 5, False, 1), (1000, 128, True, 1), (200, 70, True, 1), (72, 33, False, 0),
                                            (36, 12, True, 1)])
def test_lstm_step_with_embedding_lookup_folded_in(ctx, H, mb, feed, fused):
    """zr_lstm_step_embed (the node reads its input columns from the embedding by token id) against the gather followed
    by zr_lstm_step -- bit for bit, the same kernel reads the same numbers -- and against the oracle; duplicate ids,
    first and last column of the embedding, a masked column; also through the two-phase path (fused = 0)."""
    g = synth.rng(29, H + mb)
    V = 977
    ly = synth.lstm_layer(g, H, feed_input=feed, forget_bias_one=True)
    embed = U(g, (H, V), -1, 1)
    ids = g.integers(0, V, size=mb).astype(np.int32)
    ids[0], ids[mb - 1] = 0, V - 1
    if mb > 3:
        ids[2] = ids[1]
    hp, cp, ht = U(g, (H, mb), -1, 1), U(g, (H, mb), -1, 1), U(g, (H, mb), -1, 1)
    mask = np.ones(mb, np.int32)
    mask[mb // 2] = 0
    layer = Layer(ctx, ly)
    d_embed, d_ids, d_mask = ctx.array(embed), ctx.array(ids), ctx.array(mask)
    d_hp, d_cp, d_ht = ctx.array(hp), ctx.array(cp), ctx.array(ht) if feed else None
    h1, c1, h2, c2, x = (ctx.empty((H, mb)) for _ in range(5))
    ctx.set_option(capi.ZR_OPT_LSTM_FUSED_EPILOGUE, fused)
    try:
        ctx.lstm_step_embed(layer.w, d_embed, V, d_ids, d_hp, d_cp, d_mask, mb, h1, c1, d_htild=d_ht, clip=0.8)
        ctx.embed_gather(d_embed, H, V, d_ids, mb, x)
        ctx.lstm_step(layer.w, x, d_hp, d_cp, d_mask, mb, h2, c2, d_htild=d_ht, clip=0.8)
        ctx.sync()
    finally:
        ctx.set_option(capi.ZR_OPT_LSTM_FUSED_EPILOGUE, 1)
        layer.close()
    assert h1.get().tobytes() == h2.get().tobytes() and c1.get().tobytes() == c2.get().tobytes()
    want = o.lstm_step(ly["M"], ly["Wh"], ly["b"], o.embed_gather(embed, ids), hp, cp, mask, Q=ly.get("Q"),
                       htild=ht if feed else None, clip=0.8)
    assert_close(h1.get(), want["h"], what="h")
    assert_close(c1.get(), want["c"], what="c")
    assert np.all(h1.get()[:, mb // 2] == 0)


def _decoder_step_case(g, H, mb, L, feed, V=977):
    layers = [synth.lstm_layer(g, H, feed_input=(feed and l == 0), forget_bias_one=True) for l in range(L)]
    embed = U(g, (H, V), -1, 1)
    ids = g.integers(0, V, size=mb).astype(np.int32)
    ids[0], ids[mb - 1] = 0, V - 1
    if mb > 3:
        ids[2] = ids[1]
    hp = [U(g, (H, mb), -1, 1) for _ in range(L)]
    cp = [U(g, (H, mb), -1, 1) for _ in range(L)]
    ht = U(g, (H, mb), -1, 1) if feed else None
    mask = np.ones(mb, np.int32)
    if mb > 1:  # (a single column stays live: a masked one would test nothing but zeros)
        mask[mb // 2] = 0
    return layers, embed, ids, hp, cp, ht, mask


def _run_decoder_step(ctx, case, V=977, clip=0.8, expect_path=None):
    layers, embed, ids, hp, cp, ht, mask = case
    H, mb = hp[0].shape
    L = len(layers)
    lys = [Layer(ctx, ly) for ly in layers]
    try:
        d_h = [ctx.zeros((H, mb)) for _ in range(L)]
        d_c = [ctx.zeros((H, mb)) for _ in range(L)]
        ctx.lstm_decoder_step([ly.w for ly in lys], ctx.array(embed), V, ctx.array(ids), [ctx.array(a) for a in hp],
                              [ctx.array(a) for a in cp], ctx.array(mask), mb, d_h, d_c,
                              d_htild=ctx.array(ht) if ht is not None else None, clip=clip)
        if expect_path is not None:
            assert ctx.query(capi.ZR_QUERY_LSTM_STACK_PATH) == expect_path
        abandoned = ctx.query(capi.ZR_QUERY_LSTM_SWEEP_ABANDONED)
        ctx.sync()
        return [a.get() for a in d_h], [a.get() for a in d_c], abandoned
    finally:
        for ly in lys:
            ly.close()


def _oracle_decoder_step(case, clip=0.8):
    layers, embed, ids, hp, cp, ht, mask = case
    hs, cs = [], []
    x = o.embed_gather(embed, ids)
    for l, ly in enumerate(layers):
        r = o.lstm_step(ly["M"], ly["Wh"], ly["b"], x, hp[l], cp[l], mask, Q=ly.get("Q") if l == 0 else None,
                        htild=ht if l == 0 else None, clip=clip)
        hs.append(r["h"])
        cs.append(r["c"])
        x = r["h"]
    return hs, cs


@pytest.mark.parametrize("H,mb,L,feed", [(64, 5, 3, True), (1000, 128, 4, True), (200, 70, 2, True), (72, 33, 1, False),
                                         (128, 128, 4, False), (256, 192, 4, True), (1000, 12, 4, True), (1000, 1, 4, True),
                                         (104, 40, 8, False), (1000, 192, 4, True), (520, 200, 3, True),
                                         (1000, 160, 4, True), (776, 250, 2, False)])
def test_decoder_step_all_layers_in_one_launch(ctx, H, mb, L, feed):
    """zr_lstm_decoder_step as ONE launch (two resident workgroups per state tile: one streams the W_h / Q products of
    every layer, the other walks up the chain of layers) against the oracle's node-by-node step and against one launch
    per layer: feed-input on layer 0, duplicate and extreme ids, a masked column, cell clipping, row and column tails,
    a batch width that is not a multiple of 8 (consumers then invalidate their caches), one to eight layers.  The last
    four shapes have more 32-column tiles than the device holds workgroup pairs for.  Three of them keep 32-column
    tiles and hand the W_h products of the upper layers, and the upper part of Q, to helper workgroups of several tiles
    each, while the chain workgroups compute the W_h products of the lower layers themselves: 192 columns of H = 1000,
    the batched beam decode, with 64 helpers of three tiles for layers 2 and 3; 200 columns of H = 520 with a last
    column tile of 8 columns, 88 helpers of two tiles or one, layers 1 and 2; 160 columns with 96 helpers of two tiles
    or one for layers 1 to 3.  The last has exactly as many 32-column tiles as the device holds workgroups and takes
    64-column tiles."""
    g = synth.rng(31, H + mb + L)
    case = _decoder_step_case(g, H, mb, L, feed)
    ctx.set_option(capi.ZR_OPT_LSTM_SWEEP, 2)
    try:
        h1, c1, gave_up = _run_decoder_step(ctx, case, expect_path=capi.ZR_LSTM_STACK_PATH_STEP_SINGLE_LAUNCH)
        ctx.set_option(capi.ZR_OPT_LSTM_SWEEP, 1)
        h2, c2, _ = _run_decoder_step(ctx, case, expect_path=capi.ZR_LSTM_STACK_PATH_STEP_PER_LAYER)
    finally:
        ctx.set_option(capi.ZR_OPT_LSTM_SWEEP, 0)
    assert gave_up == 0
    want_h, want_c = _oracle_decoder_step(case)
    for l in range(L):
        assert_close(h1[l], want_h[l], what="h of layer %d" % l)
        assert_close(c1[l], want_c[l], what="c of layer %d" % l)
        assert_close(h2[l], want_h[l], what="h of layer %d, per-layer launches" % l)
        assert_close(c2[l], want_c[l], what="c of layer %d, per-layer launches" % l)
        if mb > 1:
            assert np.all(h1[l][:, mb // 2] == 0) and np.all(c1[l][:, mb // 2] == 0)


def test_decoder_step_picks_the_single_launch_at_benchmark_size_and_repeats_bit_for_bit(ctx):
    """H = 1000, 128 columns, 4 layers with feed-input: left to itself the library takes the single launch (it fills
    the device); two runs give the same bits (the two partial sums of a tile are always added in the same order)."""
    g = synth.rng(32, 1)
    case = _decoder_step_case(g, 1000, 128, 4, True)
    h1, c1, a1 = _run_decoder_step(ctx, case, expect_path=capi.ZR_LSTM_STACK_PATH_STEP_SINGLE_LAUNCH)
    h2, c2, a2 = _run_decoder_step(ctx, case, expect_path=capi.ZR_LSTM_STACK_PATH_STEP_SINGLE_LAUNCH)
    assert a1 == 0 and a2 == 0
    for l in range(4):
        assert h1[l].tobytes() == h2[l].tobytes() and c1[l].tobytes() == c2[l].tobytes()


@pytest.mark.parametrize("H,mb,L", [(128, 40, 3), (128, 520, 3), (128, 1000, 3)])
def test_decoder_step_single_launch_abandoned_wait_is_reported(ctx, H, mb, L):
    """The waits for the layer below are told to expect one arrival more than will come and given 64 polls: the layers
    above the first give up whatever the timing, every workgroup still leaves the kernel, the query reports it, the
    unfinished outputs hold NaN, and the next step with the default settings is complete again (the last workgroup out
    of the abandoned launch returned the counters to zero).  32-column tiles in pairs, 32-column tiles with helper
    workgroups, 64-column tiles in pairs."""
    g = synth.rng(33, 1)
    case = _decoder_step_case(g, H, mb, L, True)
    ctx.set_option(capi.ZR_OPT_LSTM_SWEEP, 2)
    ctx.set_option(capi.ZR_OPT_LSTM_SWEEP_SPIN, 64)
    ctx.set_option(capi.ZR_OPT_LSTM_STEP_WAIT_EXTRA, 1)
    try:
        h1, c1, gave_up = _run_decoder_step(ctx, case, expect_path=capi.ZR_LSTM_STACK_PATH_STEP_SINGLE_LAUNCH)
        assert gave_up == 1
        # what the abandoned step did not finish holds NaN, what it did finish is right; the top layer cannot be complete
        want_h, want_c = _oracle_decoder_step(case)
        assert np.isnan(h1[-1]).any() and np.isnan(c1[-1]).any()
        for got, want in zip(h1 + c1, want_h + want_c):
            done = ~np.isnan(got)
            assert_close(np.where(done, got, 0.0), np.where(done, want, 0.0), what="finished part of an abandoned step")
        ctx.set_option(capi.ZR_OPT_LSTM_SWEEP_SPIN, 0)
        ctx.set_option(capi.ZR_OPT_LSTM_STEP_WAIT_EXTRA, 0)
        h2, c2, gave_up = _run_decoder_step(ctx, case, expect_path=capi.ZR_LSTM_STACK_PATH_STEP_SINGLE_LAUNCH)
        assert gave_up == 0
    finally:
        ctx.set_option(capi.ZR_OPT_LSTM_SWEEP, 0)
        ctx.set_option(capi.ZR_OPT_LSTM_SWEEP_SPIN, 0)
        ctx.set_option(capi.ZR_OPT_LSTM_STEP_WAIT_EXTRA, 0)
    want_h, want_c = _oracle_decoder_step(case)
    for l in range(L):
        assert_close(h2[l], want_h[l], what="h of layer %d" % l)
        assert_close(c2[l], want_c[l], what="c of layer %d" % l)


@pytest.mark.parametrize("H,mb,L,S,D,V,prepared", [(1000, 128, 4, 20, 10, 5000, True), (64, 5, 2, 9, 3, 301, True),
                                                   (1000, 128, 2, 12, 12, 2000, False), (100, 8, 1, 7, 2, 333, True),
                                                   (256, 64, 3, 30, 50, 40000, True),
                                                   # v_p at a 4-byte offset (see below)
                                                   (1000, 128, 4, 20, 10, 5000, "v_p off by 4 bytes"),
                                                   (64, 5, 2, 9, 3, 301, "v_p off by 4 bytes")])
def test_decoder_step_as_one_call_matches_the_three_calls(ctx, H, mb, L, S, D, V, prepared):
    """zr_decoder_step (forward_prop_target as one call, hand-overs kept in the matrix cores' layout) against
    zr_lstm_decoder_step + zr_attn_step + zr_softmax_forward on the same inputs: the same kernels read the same numbers,
    so every output is the same bit for bit -- with and without the prepared snapshots, with an LSTM stack that takes
    the single launch and one that does not, with a layer size the packed layout does not cover.  With v_p misaligned
    the attention step cannot run on its snapshots and writes no k-interleaved h~: the output layer must then read the
    plain one."""
    g = synth.rng(35, H + mb + L)
    case = _decoder_step_case(g, H, mb, L, True, V=V)
    layers, embed, ids, hp, cp, ht, mask = case
    w = synth.attention_weights(g, H)
    hs = (g.standard_normal(size=(S, H, mb), dtype=np.float32) * np.float32(0.1))
    lens = g.integers(1, S + 1, size=mb).astype(np.int32)
    binfo = np.concatenate([lens, S - lens]).astype(np.int32)
    Dm, bd = U(g, (V, H)), U(g, (V,))
    lys = [Layer(ctx, ly) for ly in layers]
    tables = [ctx.array(np.asfortranarray(hs[t])) for t in range(S)]
    dw = {k: ctx.array(v) for k, v in w.items()}
    v_p = dw["v_p"]
    if prepared == "v_p off by 4 bytes":
        d_vp_shifted = ctx.array(np.concatenate([np.zeros(1, np.float32), w["v_p"].reshape(-1)]))
        v_p = d_vp_shifted.at(1)
    a = ctx.attn_create(H, mb, D, dw["W_a"], dw["W_p"], v_p, dw["out_bias"], dw["W_c1"], dw["W_c2"], tables)
    dD, dbd = ctx.array(Dm), ctx.array(bd)
    if prepared:
        ctx.attn_prepare(a)
        ctx.softmax_prepare(dD, V, H)
    try:
        d_embed, d_ids, d_mask, d_bi = ctx.array(embed), ctx.array(ids), ctx.array(mask), ctx.array(binfo)
        d_hp, d_cp, d_htp = [ctx.array(x) for x in hp], [ctx.array(x) for x in cp], ctx.array(ht)
        outs = []
        for one_call in (False, True):
            d_h = [ctx.zeros((H, mb)) for _ in range(L)]
            d_c = [ctx.zeros((H, mb)) for _ in range(L)]
            d_ht, d_p = ctx.zeros((H, mb)), ctx.zeros((V, mb))
            if one_call:
                ctx.decoder_step([ly.w for ly in lys], d_embed, V, d_ids, d_hp, d_cp, d_mask, mb, d_h, d_c, a, d_bi, d_ht, dD,
                                 dbd, V, capi.ZR_SOFTMAX_PROB, d_p, d_htild_prev=d_htp, clip=0.8)
            else:
                ctx.lstm_decoder_step([ly.w for ly in lys], d_embed, V, d_ids, d_hp, d_cp, d_mask, mb, d_h, d_c,
                                      d_htild=d_htp, clip=0.8)
                ctx.attn_step(a, d_bi, d_h[L - 1], d_mask, d_ht)
                ctx.softmax_forward(dD, dbd, V, H, d_ht, mb, capi.ZR_SOFTMAX_PROB, d_p)
            ctx.sync()
            outs.append([x.get() for x in d_h + d_c + [d_ht, d_p]])
        for x, y in zip(*outs):
            assert x.tobytes() == y.tobytes()
        want_h, _ = _oracle_decoder_step(case)
        assert_close(outs[1][L - 1], want_h[L - 1], what="top h")
        att = o.attention_forward(hs_table=hs, batch_info=binfo, h_t=want_h[L - 1], mask01=mask, D=D, **w)
        assert_close(outs[1][2 * L], att["h_tild"], what="h_tild")
        cols = np.array([0, mb // 2, mb - 1])
        want_p = o.softmax_dist(o.softmax_logits(Dm, bd, np.asfortranarray(att["h_tild"][:, cols])))
        assert_close(outs[1][2 * L + 1][:, cols], want_p, floor=1e-7, what="probabilities (sampled columns)")
    finally:
        if prepared:
            ctx.softmax_release(dD)
        ctx.attn_destroy(a)
        for ly in lys:
            ly.close()


def test_decoder_step_as_one_call_without_attention(ctx):
    """zr_decoder_step with no attention layer: the output distribution is taken from the top layer's h_t; log-probability
    mode; against the separate calls bit for bit."""
    g = synth.rng(36, 1)
    H, mb, L, V = 128, 40, 2, 777
    case = _decoder_step_case(g, H, mb, L, False, V=V)
    layers, embed, ids, hp, cp, _, mask = case
    Dm, bd = U(g, (V, H)), U(g, (V,))
    lys = [Layer(ctx, ly) for ly in layers]
    try:
        d_embed, d_ids, d_mask = ctx.array(embed), ctx.array(ids), ctx.array(mask)
        d_hp, d_cp = [ctx.array(x) for x in hp], [ctx.array(x) for x in cp]
        dD, dbd = ctx.array(Dm), ctx.array(bd)
        outs = []
        for one_call in (False, True):
            d_h = [ctx.zeros((H, mb)) for _ in range(L)]
            d_c = [ctx.zeros((H, mb)) for _ in range(L)]
            d_p = ctx.zeros((V, mb))
            if one_call:
                ctx.decoder_step([ly.w for ly in lys], d_embed, V, d_ids, d_hp, d_cp, d_mask, mb, d_h, d_c, None, None, None,
                                 dD, dbd, V, capi.ZR_SOFTMAX_LOGPROB, d_p, clip=0.8)
            else:
                ctx.lstm_decoder_step([ly.w for ly in lys], d_embed, V, d_ids, d_hp, d_cp, d_mask, mb, d_h, d_c, clip=0.8)
                ctx.softmax_forward(dD, dbd, V, H, d_h[L - 1], mb, capi.ZR_SOFTMAX_LOGPROB, d_p)
            ctx.sync()
            outs.append([x.get() for x in d_h + d_c + [d_p]])
        for x, y in zip(*outs):
            assert x.tobytes() == y.tobytes()
        want_h, _ = _oracle_decoder_step(case)
        want_lp = o.softmax_logprob_f64(o.softmax_logits(Dm, bd, want_h[L - 1]))
        assert_close(outs[1][2 * L], want_lp, what="log-probabilities")
    finally:
        for ly in lys:
            ly.close()


def test_stack_forward_with_split_kernel_forced(ctx):
    g = synth.rng(17, 1)
    H, mb, T, V, L = 64, 5, 7, 211, 3
    embed = U(g, (H, V))
    layers = [synth.lstm_layer(g, H, forget_bias_one=True) for _ in range(L)]
    ids = g.integers(0, V, size=(T, mb)).astype(np.int32)
    ids[:3, 1] = -1
    ctx.set_option(capi.ZR_OPT_LSTM_KERNEL, 2)
    try:
        hs, cs = _run_stack(ctx, layers, embed, ids)
    finally:
        ctx.set_option(capi.ZR_OPT_LSTM_KERNEL, 0)
    nn, m = o.vocab_prep(ids)
    want_h, want_c = o.lstm_stack_forward(embed, layers, nn, m)
    assert_close(hs, want_h, what="stack h")
    assert_close(cs, want_c, what="stack c")


@pytest.mark.parametrize("H,mb,T,L", [(64, 5, 7, 3), (104, 40, 9, 4), (256, 70, 6, 2), (1000, 128, 5, 4),
                                      (72, 33, 12, 1), (512, 128, 4, 8), (8, 1, 3, 2), (32, 2, 1, 1), (40, 9, 1, 5)])
def test_stack_forward_whole_sweep_launch(ctx, H, mb, T, L):
    """The single-launch sweep (workgroups hand h to each other through device memory) against the oracle and against
    one launch per diagonal: column and row tails, one to eight layers, initial states, padding, cell clipping."""
    g = synth.rng(19, H + mb)
    V = 311
    embed = U(g, (H, V))
    layers = [synth.lstm_layer(g, H, forget_bias_one=True) for _ in range(L)]
    ids = g.integers(0, V, size=(T, mb)).astype(np.int32)
    if mb > 1:
        ids[:2, 1] = -1
    ids[: T - 1, mb - 1] = -1
    h0 = [np.tanh(U(g, (H, mb), -1, 1)) for _ in range(L)]
    c0 = [U(g, (H, mb), -0.5, 0.5) for _ in range(L)]
    out = {}
    for mode in (2, 1):
        ctx.set_option(capi.ZR_OPT_LSTM_SWEEP, mode)
        try:
            path = capi.ZR_LSTM_STACK_PATH_SWEEP if mode == 2 else capi.ZR_LSTM_STACK_PATH_DIAGONALS
            out[mode] = _run_stack(ctx, layers, embed, ids, h0=h0, c0=c0, clip=0.9, expect_path=path)
            again = _run_stack(ctx, layers, embed, ids, h0=h0, c0=c0, clip=0.9, expect_path=path) if mode == 2 else None
        finally:
            ctx.set_option(capi.ZR_OPT_LSTM_SWEEP, 0)
        if again is not None:  # fixed summation order: the same bits on every run
            assert again[0].tobytes() == out[2][0].tobytes() and again[1].tobytes() == out[2][1].tobytes()
    nn, m = o.vocab_prep(ids)
    want_h, want_c = o.lstm_stack_forward(embed, layers, nn, m, h0=h0, c0=c0, clip=0.9)
    for mode in (2, 1):
        assert_close(out[mode][0], want_h, what="stack h (sweep option %d)" % mode)
        assert_close(out[mode][1], want_c, what="stack c (sweep option %d)" % mode)
    assert mb == 1 or np.all(out[2][0][:, : min(2, T), :, 1] == 0)
    assert np.all(out[2][1][:, : T - 1, :, mb - 1] == 0)


def test_whole_sweep_launch_keeps_gates_for_training(ctx):
    """zr_lstm_stack_forward_train through the single-launch sweep: every node's four gate activations, h and c against
    the oracle's node-by-node forward pass."""
    g = synth.rng(22, 1)
    H, mb, T, V, L = 96, 24, 5, 131, 2
    embed = U(g, (H, V))
    layers_np = [synth.lstm_layer(g, H, forget_bias_one=True) for _ in range(L)]
    ids = g.integers(0, V, size=(T, mb)).astype(np.int32)
    ids[:2, 3] = -1
    n = H * mb
    layers = [Layer(ctx, ly) for ly in layers_np]
    d_nn, d_m = ctx.empty(ids.size, np.int32), ctx.empty(ids.size, np.int32)
    ctx.vocab_prep(ctx.array(ids.reshape(-1)), ids.size, V, d_nn, d_m)
    z = ctx.zeros((H, mb))
    h_all = [ctx.empty((n * T,)) for _ in range(L)]
    c_all = [ctx.empty((n * T,)) for _ in range(L)]
    g_all = [ctx.empty((4 * n * T,)) for _ in range(L)]
    ctx.set_option(capi.ZR_OPT_LSTM_SWEEP, 2)
    try:
        ctx.lstm_stack_forward_train([ly.w for ly in layers], ctx.array(embed), V, d_nn, d_m, T, mb, [z] * L, [z] * L,
                                     h_all, c_all, g_all)
        assert ctx.query(capi.ZR_QUERY_LSTM_STACK_PATH) == capi.ZR_LSTM_STACK_PATH_SWEEP
        ctx.sync()
    finally:
        ctx.set_option(capi.ZR_OPT_LSTM_SWEEP, 0)
    nn, m = o.vocab_prep(ids)
    zero = np.zeros((H, mb), np.float32)
    below = None
    for l, ly in enumerate(layers_np):
        hp, cp = zero, zero
        outs = []
        got_h = h_all[l].get().reshape(T, mb, H).transpose(0, 2, 1)
        got_c = c_all[l].get().reshape(T, mb, H).transpose(0, 2, 1)
        got_g = g_all[l].get().reshape(T, 4, mb, H).transpose(0, 1, 3, 2)
        for t in range(T):
            x = np.asfortranarray(embed[:, nn[t]]) if l == 0 else below[t]
            want = o.lstm_step(ly["M"], ly["Wh"], ly["b"], x, hp, cp, m[t])
            for gi, k in enumerate(("i", "f", "c_tilde", "o")):
                assert_close(got_g[t, gi], want[k], what="gate %s layer %d step %d" % (k, l, t))
            assert_close(got_h[t], want["h"], what="h layer %d step %d" % (l, t))
            assert_close(got_c[t], want["c"], what="c layer %d step %d" % (l, t))
            hp, cp = want["h"], want["c"]
            outs.append(want["h"])
        below = outs
    for ly in layers:
        ly.close()


def test_whole_sweep_launch_back_to_back_with_different_inputs(ctx):
    """Sweeps of the same shape with different token ids and initial states, queued back to back through the same
    hand-over buffers with nothing but the counter-clearing fill between them (the whole hand-over buffer, 1.5 MB, stays
    cache resident): a later sweep must not see anything of an earlier one (mb % 8 == 0: the consumers do not
    invalidate their caches inside the launch)."""
    H, mb, T, V, L = 256, 64, 6, 211, 4
    g = synth.rng(21, 1)
    embed = U(g, (H, V))
    layers_np = [synth.lstm_layer(g, H, forget_bias_one=True) for _ in range(L)]
    layers = [Layer(ctx, ly) for ly in layers_np]
    d_embed = ctx.array(embed)
    n = H * mb
    runs = []
    for seed in range(4):
        ids = g.integers(0, V, size=(T, mb)).astype(np.int32)
        h0 = [np.tanh(U(g, (H, mb), -1, 1)) for _ in range(L)]
        c0 = [U(g, (H, mb), -0.5, 0.5) for _ in range(L)]
        d_nn, d_m = ctx.empty(ids.size, np.int32), ctx.empty(ids.size, np.int32)
        ctx.vocab_prep(ctx.array(ids.reshape(-1)), ids.size, V, d_nn, d_m)
        runs.append(dict(ids=ids, h0=h0, c0=c0, d_nn=d_nn, d_m=d_m, d_h0=[ctx.array(a) for a in h0],
                         d_c0=[ctx.array(a) for a in c0], h_all=[ctx.empty((n * T,)) for _ in range(L)],
                         c_all=[ctx.empty((n * T,)) for _ in range(L)]))
    ctx.sync()
    ctx.set_option(capi.ZR_OPT_LSTM_SWEEP, 2)
    try:
        for r in runs:  # queued without a synchronisation or any other work in between
            ctx.lstm_stack_forward([ly.w for ly in layers], d_embed, V, r["d_nn"], r["d_m"], T, mb, r["d_h0"], r["d_c0"],
                                   r["h_all"], r["c_all"])
            assert ctx.query(capi.ZR_QUERY_LSTM_STACK_PATH) == capi.ZR_LSTM_STACK_PATH_SWEEP
        ctx.sync()
    finally:
        ctx.set_option(capi.ZR_OPT_LSTM_SWEEP, 0)
    for i, r in enumerate(runs):
        nn, m = o.vocab_prep(r["ids"])
        want_h, want_c = o.lstm_stack_forward(embed, layers_np, nn, m, h0=r["h0"], c0=r["c0"])
        hs = np.stack([a.get().reshape(T, mb, H).transpose(0, 2, 1) for a in r["h_all"]])
        cs = np.stack([a.get().reshape(T, mb, H).transpose(0, 2, 1) for a in r["c_all"]])
        assert_close(hs, want_h, what="stack h (run %d)" % i)
        assert_close(cs, want_c, what="stack c (run %d)" % i)
    for ly in layers:
        ly.close()


@pytest.mark.parametrize("H,mb,T,L", [(200, 70, 20, 3), (256, 64, 12, 4)])
def test_whole_sweep_launch_many_repetitions_identical(ctx, H, mb, T, L):
    """The same sweep 400 times in a row: the order of the sums is fixed, so whatever the timing of the hand-overs
    between workgroups, every repetition gives the first one's bits (checked every 50 launches), the first one agrees
    with the oracle, and no wait is ever abandoned (zr_ctx_sync would report it).  mb = 70 takes the waits that
    invalidate the caches, mb = 64 the ones that do not."""
    g = synth.rng(23, H + mb)
    V = 257
    embed = U(g, (H, V))
    layers_np = [synth.lstm_layer(g, H, forget_bias_one=True) for _ in range(L)]
    layers = [Layer(ctx, ly) for ly in layers_np]
    ids = g.integers(0, V, size=(T, mb)).astype(np.int32)
    ids[:3, 2] = -1
    d_embed = ctx.array(embed)
    d_nn, d_m = ctx.empty(ids.size, np.int32), ctx.empty(ids.size, np.int32)
    ctx.vocab_prep(ctx.array(ids.reshape(-1)), ids.size, V, d_nn, d_m)
    z = ctx.zeros((H, mb))
    h_all = [ctx.empty((H * mb * T,)) for _ in range(L)]
    c_all = [ctx.empty((H * mb * T,)) for _ in range(L)]
    first = None
    ctx.set_option(capi.ZR_OPT_LSTM_SWEEP, 2)
    try:
        for i in range(400):
            ctx.lstm_stack_forward([ly.w for ly in layers], d_embed, V, d_nn, d_m, T, mb, [z] * L, [z] * L, h_all, c_all)
            assert ctx.query(capi.ZR_QUERY_LSTM_STACK_PATH) == capi.ZR_LSTM_STACK_PATH_SWEEP
            if i % 50 == 0 or i == 399:
                ctx.sync()
                got = [a.get().tobytes() for a in h_all + c_all]
                if first is None:
                    first = got
                    nn, m = o.vocab_prep(ids)
                    want_h, want_c = o.lstm_stack_forward(embed, layers_np, nn, m)
                    hs = np.stack([a.get().reshape(T, mb, H).transpose(0, 2, 1) for a in h_all])
                    cs = np.stack([a.get().reshape(T, mb, H).transpose(0, 2, 1) for a in c_all])
                    assert_close(hs, want_h, what="stack h")
                    assert_close(cs, want_c, what="stack c")
                assert got == first, "repetition %d differs from the first" % i
    finally:
        ctx.set_option(capi.ZR_OPT_LSTM_SWEEP, 0)
    for ly in layers:
        ly.close()


def test_whole_sweep_launch_abandoned_wait_is_reported(ctx):
    """With a single poll per wait the upper layers give up at once: every workgroup still leaves the kernel, and
    zr_ctx_sync reports the incomplete sweep; the next sweep with the default limit is complete again."""
    g = synth.rng(20, 1)
    H, mb, T, V, L = 128, 40, 6, 97, 3
    embed = U(g, (H, V))
    layers = [synth.lstm_layer(g, H) for _ in range(L)]
    ids = g.integers(0, V, size=(T, mb)).astype(np.int32)
    ctx.set_option(capi.ZR_OPT_LSTM_SWEEP, 2)
    ctx.set_option(capi.ZR_OPT_LSTM_SWEEP_SPIN, 1)
    try:
        with pytest.raises(capi.ZrError, match="gave up waiting"):
            _run_stack(ctx, layers, embed, ids, expect_path=capi.ZR_LSTM_STACK_PATH_SWEEP)
        # the same through the query, which also shows what the abandoned sweep left behind: NaN in every output, so
        # that nothing queued behind it can mistake stale memory for a result
        H_, mb_ = H, mb
        lys = [Layer(ctx, ly) for ly in layers]
        d_nn, d_m = ctx.empty(ids.size, np.int32), ctx.empty(ids.size, np.int32)
        ctx.vocab_prep(ctx.array(ids.reshape(-1)), ids.size, V, d_nn, d_m)
        z = ctx.zeros((H_, mb_))
        h_all = [ctx.zeros((H_ * mb_ * T,)) for _ in range(L)]
        c_all = [ctx.zeros((H_ * mb_ * T,)) for _ in range(L)]
        ctx.lstm_stack_forward([ly.w for ly in lys], ctx.array(embed), V, d_nn, d_m, T, mb_, [z] * L, [z] * L, h_all, c_all)
        assert ctx.query(capi.ZR_QUERY_LSTM_SWEEP_ABANDONED) == 1
        assert ctx.query(capi.ZR_QUERY_LSTM_SWEEP_ABANDONED) == 0  # the look clears the flag
        ctx.sync()  # ... so the synchronisation has nothing left to report
        assert all(np.all(np.isnan(a.get())) for a in h_all + c_all)
        for ly in lys:
            ly.close()
        ctx.set_option(capi.ZR_OPT_LSTM_SWEEP_SPIN, 0)
        hs, cs = _run_stack(ctx, layers, embed, ids, expect_path=capi.ZR_LSTM_STACK_PATH_SWEEP)
        assert ctx.query(capi.ZR_QUERY_LSTM_SWEEP_ABANDONED) == 0
    finally:
        ctx.set_option(capi.ZR_OPT_LSTM_SWEEP, 0)
        ctx.set_option(capi.ZR_OPT_LSTM_SWEEP_SPIN, 0)
    nn, m = o.vocab_prep(ids)
    want_h, want_c = o.lstm_stack_forward(embed, layers, nn, m)
    assert_close(hs, want_h, what="stack h")
    assert_close(cs, want_c, what="stack c")


def test_config2_encoder_at_benchmark_size_both_schedules(ctx):
    """Benchmark configuration 2 exactly as bench.py runs it (synth.encoder_config: H=1000, mb=128, T=50, L=4, V=50000,
    Zipf(1.1) ids, zero initial state): the schedule the library picks by itself must be the single-launch sweep, and
    both it and one launch per diagonal are compared with the oracle (double accumulation) on every h and c of all 200
    nodes."""
    c = synth.encoder_config()
    H, mb, T, L, V = c["H"], c["mb"], c["T"], c["L"], c["V"]
    assert (H, mb, T, L, V) == (1000, 128, 50, 4, 50000)
    nn, m = o.vocab_prep(c["ids"])
    want_h, want_c = o.lstm_stack_forward(c["embed"], c["layers"], nn, m)
    # the library's own choice (option 0) is what the benchmark times
    auto_h, auto_c = _run_stack(ctx, c["layers"], c["embed"], c["ids"], expect_path=capi.ZR_LSTM_STACK_PATH_SWEEP)
    assert_close(auto_h, want_h, what="config 2 h (schedule picked by the library)")
    assert_close(auto_c, want_c, what="config 2 c (schedule picked by the library)")
    ctx.set_option(capi.ZR_OPT_LSTM_SWEEP, 1)
    try:
        diag_h, diag_c = _run_stack(ctx, c["layers"], c["embed"], c["ids"], expect_path=capi.ZR_LSTM_STACK_PATH_DIAGONALS)
    finally:
        ctx.set_option(capi.ZR_OPT_LSTM_SWEEP, 0)
    assert_close(diag_h, want_h, what="config 2 h (one launch per diagonal)")
    assert_close(diag_c, want_c, what="config 2 c (one launch per diagonal)")
    # size-independent properties at full size: |h| < 1, the last step's h of the top layer is what the encoder hands on
    assert np.all(np.abs(auto_h) < 1.0) and np.all(np.isfinite(auto_c))
    # Zipf ids repeat: columns that read the same token at t = 0 leave layer 0 identical (zero initial state)
    ids0 = c["ids"][0]
    dup = [np.nonzero(ids0 == v)[0] for v in np.unique(ids0)]
    dup = [d for d in dup if len(d) > 1]
    assert dup, "Zipf(1.1) ids at 128 columns always repeat"
    for d in dup[:5]:
        assert np.array_equal(auto_h[0, 0][:, d[0]], auto_h[0, 0][:, d[1]])


@pytest.mark.parametrize("V,H,mb", [(4100, 100, 128), (5000, 72, 192), (4096, 36, 256), (6004, 1000, 100), (4360, 64, 300)])
def test_softmax_large_vocab_lds_gemm_shapes(ctx, V, H, mb):
    """Shapes that take the LDS-shared-weights GEMM (M >= 4096, N >= 96): row tails (V % 32 != 0), K tails
    (H % 32 != 0, H % 8 != 0), 4-, 6- and 8-wave workgroups, more than one column tile."""
    g = synth.rng(18, V + mb)
    D, bd, h = U(g, (V, H), -0.5, 0.5), U(g, (V,), -1, 1), U(g, (H, mb), -1, 1)
    d_lp, d_scr = ctx.empty((V, mb)), ctx.empty((V, mb))
    ctx.softmax_forward(ctx.array(D), ctx.array(bd), V, H, ctx.array(h), mb, capi.ZR_SOFTMAX_LOGPROB, d_lp, d_scr)
    ctx.sync()
    logits = o.softmax_logits(D, bd, h)
    assert_close(d_scr.get(), logits, floor=magnitude_floor(logits), what="logits")
    assert_close(d_lp.get(), o.softmax_logprob_f64(logits), what="log-probs")
    dC = ctx.empty((V, mb))
    ctx.gemm(0, V, mb, H, ctx.array(D), V, ctx.array(h), H, dC, V)
    ctx.sync()
    plain = o.gemm_nn(D, h)
    assert_close(dC.get(), plain, floor=magnitude_floor(plain), what="plain gemm")
