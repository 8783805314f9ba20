"""Training backward on the GPU (stacked LSTM + output layer) against the oracle, whose backward restatement is
pinned by torch autograd in tests/test_oracle_backward_pins.py.  fp32 tolerance: 1e-4 relative with an absolute
floor scaled to the size of the sums involved (stated per check)."""
import numpy as np
import pytest

import oracle_lib as o
from gpu_util import Layer, assert_close
from zoph_rnn_amd import capi, synth

pytestmark = pytest.mark.gpu
U = synth.uniform


@pytest.fixture(scope="module")
def ctx():
    c = capi.Context(0)
    yield c
    c.close()


class TrainLayer(Layer):
    def __init__(self, ctx, ly):
        super().__init__(ctx, ly)
        self.t = ctx.lstm_train_create(self.M, self.Wh, self.H)

    def close(self):
        self.ctx.lstm_train_destroy(self.t)
        super().close()


def _unstack(ctx, d_stack, H):
    outs = [ctx.empty((H, H)) for _ in range(4)]
    ctx.unstack_gates(d_stack, H, outs)
    ctx.sync()
    return [a.get() for a in outs]


def _gpu_stack_backward(ctx, embed, layers_np, ids, h0, c0, err_top, err_hT, err_cT, cell_clip=0.0, err_clip=0.0):
    H, V = embed.shape
    T, mb = ids.shape
    L = len(layers_np)
    n = H * mb
    layers = [TrainLayer(ctx, ly) for ly in layers_np]
    d_embed = ctx.array(embed)
    d_nn, d_m = ctx.empty(ids.size, np.int32), ctx.empty(ids.size, np.int32)
    ctx.vocab_prep(ctx.array(ids.reshape(-1)), ids.size, V, d_nn, d_m)
    d_h0, d_c0 = [ctx.array(a) for a in h0], [ctx.array(a) for a in c0]
    h_all = [ctx.empty((n * T,)) for _ in range(L)]
    c_all = [ctx.empty((n * T,)) for _ in range(L)]
    g_all = [ctx.empty((4 * n * T,)) for _ in range(L)]
    ctx.lstm_stack_forward_train([ly.w for ly in layers], d_embed, V, d_nn, d_m, T, mb, d_h0, d_c0, h_all, c_all, g_all,
                                 clip=cell_clip)
    d_err_top = ctx.array(np.concatenate([np.asfortranarray(e).reshape(-1, order="F") for e in err_top]))
    dg_all = [ctx.empty((4 * n * T,)) for _ in range(L)]
    eh0, ec0 = [ctx.empty((H, mb)) for _ in range(L)], [ctx.empty((H, mb)) for _ in range(L)]
    d_below0 = ctx.empty((n * T,))
    ctx.lstm_stack_backward([ly.t for ly in layers], T, mb, d_m, d_c0, c_all, g_all, d_err_top, dg_all, eh0, ec0,
                            err_hT=[ctx.array(a) for a in err_hT] if err_hT else None,
                            err_cT=[ctx.array(a) for a in err_cT] if err_cT else None, d_err_below0=d_below0,
                            err_clip=err_clip)
    # weight gradients, layer by layer
    x_all = ctx.empty((n * T,))
    ctx.embed_gather(d_embed, H, V, d_nn, T * mb, x_all)
    grads = []
    for l in range(L):
        dM, dWh, db = ctx.empty((4 * H, H)), ctx.empty((4 * H, H)), ctx.empty((4 * H,))
        ctx.lstm_weight_gradients(H, T, mb, dg_all[l], x_all if l == 0 else h_all[l - 1], d_h0[l], h_all[l], dM, dWh, db)
        grads.append({"dM": _unstack(ctx, dM, H), "dWh": _unstack(ctx, dWh, H), "db": list(db.get().reshape(4, H))})
    d_dW = ctx.zeros((H, V))
    ctx.embed_gradient(H, V, d_below0, d_nn, d_m, T * mb, d_dW)
    ctx.sync()
    out = (grads, d_dW.get(), [a.get() for a in eh0], [a.get() for a in ec0])
    for ly in layers:
        ly.close()
    return out


@pytest.mark.parametrize("L,H,mb,T,V,pad,tail", [(1, 32, 8, 5, 40, False, False), (3, 48, 33, 7, 90, True, True),
                                                 (2, 100, 20, 6, 150, True, True), (4, 64, 130, 4, 200, True, False),
                                                 # the layer shape the training benchmark runs (4 layers of H = 1000,
                                                 # 128 columns): full anti-diagonals of four nodes go through the
                                                 # grouped k-interleaved product and the grouped gate-derivative kernel
                                                 # at the benchmark's tile shapes; a short sweep and a small vocabulary
                                                 # keep the oracle in seconds
                                                 (4, 1000, 128, 5, 600, True, True)])
def test_stack_backward_and_gradients(ctx, L, H, mb, T, V, pad, tail):
    g = synth.rng(111, L * 1000 + H + mb)
    embed = U(g, (H, V), -0.5, 0.5)
    layers = [synth.lstm_layer(g, H) for _ in range(L)]
    for ly in layers:
        if H > 128:
            break  # a model-sized layer keeps the model's own U(-0.08, 0.08): wider matrices would saturate every gate
        ly["M"] = [U(g, (H, H), -0.2, 0.2) for _ in range(4)]
        ly["Wh"] = [U(g, (H, H), -0.2, 0.2) for _ in range(4)]
    ids = g.integers(0, V, size=(T, mb)).astype(np.int32)
    if pad:
        ids[:2, 1] = -1
        ids[T - 2:, 2] = -1
        ids[:, 5] = -1  # a fully padded column
    nn, mask = o.vocab_prep(ids)
    h0 = [U(g, (H, mb), -0.5, 0.5) for _ in range(L)]
    c0 = [U(g, (H, mb), -0.5, 0.5) for _ in range(L)]
    err_top = [U(g, (H, mb), -1, 1) for _ in range(T)]
    err_hT = [U(g, (H, mb), -1, 1) for _ in range(L)] if tail else None
    err_cT = [U(g, (H, mb), -1, 1) for _ in range(L)] if tail else None
    want_g, want_e, want_eh0, want_ec0 = o.lstm_stack_backward(embed, layers, nn, mask, err_top, h0, c0, err_hT, err_cT)
    got_g, got_e, got_eh0, got_ec0 = _gpu_stack_backward(ctx, embed, layers, ids, h0, c0, err_top, err_hT, err_cT)
    # errors are sums of up to 4H products of size ~0.2 x ~1: floor 0.05 as for the forward activations;
    # weight gradients are sums over T*mb samples of products of size ~1: floor scaled with sqrt(T*mb)
    wfloor = 0.05 * np.sqrt(T * mb)
    for l in range(L):
        assert_close(got_eh0[l], want_eh0[l], what="err_h0 layer %d" % l)
        assert_close(got_ec0[l], want_ec0[l], what="err_c0 layer %d" % l)
        for q in range(4):
            assert_close(got_g[l]["dM"][q], want_g[l]["dM"][q], floor=wfloor, what="dM layer %d gate %d" % (l, q))
            assert_close(got_g[l]["dWh"][q], want_g[l]["dWh"][q], floor=wfloor, what="dWh layer %d gate %d" % (l, q))
            assert_close(got_g[l]["db"][q], want_g[l]["db"][q], floor=wfloor, what="db layer %d gate %d" % (l, q))
    assert_close(got_e, want_e, floor=0.05 * np.sqrt(T), what="embedding gradient")
    used = set(int(v) for v in ids[ids >= 0])
    unused = [v for v in range(V) if v not in used]
    assert np.all(got_e[:, unused] == 0)


@pytest.mark.parametrize("L,H,mb,T,V", [(1, 32, 8, 5, 40), (3, 48, 33, 7, 90)])
def test_stack_backward_with_cell_and_error_clamps(ctx, L, H, mb, T, V):
    """zr_lstm_stack_backward_clamped behind a forward sweep with the cell clamp (the reference's --clip-cell): both
    thresholds low enough to act on a good share of the values (the oracle's gradients with and without them differ
    by far more than the tolerance)."""
    g = synth.rng(117, L * 1000 + H + mb)
    embed = U(g, (H, V), -0.5, 0.5)
    layers = [synth.lstm_layer(g, H) for _ in range(L)]
    for ly in layers:
        ly["M"] = [U(g, (H, H), -0.3, 0.3) for _ in range(4)]
        ly["Wh"] = [U(g, (H, H), -0.3, 0.3) for _ in range(4)]
    ids = g.integers(0, V, size=(T, mb)).astype(np.int32)
    ids[:2, 1] = -1
    nn, mask = o.vocab_prep(ids)
    h0 = [U(g, (H, mb), -0.5, 0.5) for _ in range(L)]
    c0 = [U(g, (H, mb), -0.9, 0.9) for _ in range(L)]
    err_top = [U(g, (H, mb), -1, 1) for _ in range(T)]
    cell_clip, err_clip = 0.4, 0.15
    want_g, want_e, want_eh0, want_ec0 = o.lstm_stack_backward(embed, layers, nn, mask, err_top, h0, c0,
                                                               cell_clip=cell_clip, err_clip=err_clip)
    plain_g = o.lstm_stack_backward(embed, layers, nn, mask, err_top, h0, c0)[0]
    assert np.abs(plain_g[0]["dWh"][0] - want_g[0]["dWh"][0]).max() > 0.1 * np.abs(want_g[0]["dWh"][0]).max()
    got_g, got_e, got_eh0, got_ec0 = _gpu_stack_backward(ctx, embed, layers, ids, h0, c0, err_top, None, None,
                                                         cell_clip=cell_clip, err_clip=err_clip)
    wfloor = 0.05 * np.sqrt(T * mb)
    for l in range(L):
        assert_close(got_eh0[l], want_eh0[l], what="err_h0 layer %d" % l)
        assert np.abs(got_eh0[l]).max() <= err_clip
        assert_close(got_ec0[l], want_ec0[l], what="err_c0 layer %d" % l)
        for q in range(4):
            assert_close(got_g[l]["dM"][q], want_g[l]["dM"][q], floor=wfloor, what="dM layer %d gate %d" % (l, q))
            assert_close(got_g[l]["dWh"][q], want_g[l]["dWh"][q], floor=wfloor, what="dWh layer %d gate %d" % (l, q))
            assert_close(got_g[l]["db"][q], want_g[l]["db"][q], floor=wfloor, what="db layer %d gate %d" % (l, q))
    assert_close(got_e, want_e, floor=0.05 * np.sqrt(T), what="embedding gradient")


@pytest.mark.parametrize("V,H,n", [(211, 16, 6), (1003, 48, 70), (5000, 64, 160), (1000, 32, 1056), (1003, 40, 1030)])
def test_softmax_backward(ctx, V, H, n):
    g = synth.rng(112, V)
    D, bd, h = U(g, (V, H), -0.5, 0.5), U(g, (V,), -1, 1), U(g, (H, n), -1, 1)
    target = g.integers(0, V, size=n).astype(np.int32)
    mask = (g.random(n) > 0.2).astype(np.int32)
    d_scr, d_eh, d_dD, d_db = ctx.empty((V, n)), ctx.empty((H, n)), ctx.empty((V, H)), ctx.empty((V,))
    ctx.softmax_backward(ctx.array(D), ctx.array(bd), V, H, ctx.array(h), n, ctx.array(target), ctx.array(mask), d_scr,
                         d_eh, d_dD, d_db)
    ctx.sync()
    want_eh, want_dD, want_db = o.softmax_backward(D, bd, h, target, mask)
    assert_close(d_eh.get(), want_eh, what="err_h")
    assert_close(d_dD.get(), want_dD, floor=0.05 * np.sqrt(n), what="dD")
    assert_close(d_db.get(), want_db, floor=0.05 * np.sqrt(n), what="db")
    assert np.all(d_eh.get()[:, mask == 0] == 0)
    # the variant that also returns the log-likelihood of the columns, formed from the float probabilities
    loss = ctx.softmax_backward_loss(ctx.array(D), ctx.array(bd), V, H, ctx.array(h), n, ctx.array(target),
                                     ctx.array(mask), d_scr, d_eh, d_dD, d_db)
    want_loss = o.softmax_loss(o.softmax_logprob_f64(o.softmax_logits(D, bd, h)), target, mask)
    assert loss == pytest.approx(want_loss, rel=1e-5, abs=1e-5)
    assert_close(d_dD.get(), want_dD, floor=0.05 * np.sqrt(n), what="dD (loss variant)")


@pytest.mark.parametrize("n,clip", [(1000, 0.0), (100000, 5.0), (100000, 1e6), (37, 0.5)])
def test_sgd_update(ctx, n, clip):
    g = synth.rng(113, n)
    W, G = U(g, (n,), -1, 1), U(g, (n,), -3, 3)
    scale, lr = 1.0 / 8, 0.7
    dW = ctx.array(W)
    ctx.sgd_update(dW, ctx.array(G), n, scale, clip, lr)
    ctx.sync()
    gs = G.astype(np.float64) * scale
    norm = np.sqrt((gs * gs).sum())
    coef = clip / norm if (clip > 0 and norm > clip) else 1.0
    want = W + lr * coef * gs
    assert np.allclose(dW.get(), want, rtol=1e-5, atol=1e-6)
    if clip > 0 and norm > clip:
        assert np.sqrt((((dW.get() - W) / lr) ** 2).sum()) == pytest.approx(clip, rel=1e-4)


@pytest.mark.parametrize("threshold", [0.5, 1e6])
def test_sgd_update_whole_model_clip(ctx, threshold):
    """--whole-clip-gradients (norm_clip_GPU_v2_p1 / _p2, src/custom_kernels.h:1083-1135, src/model.hpp:1850-1892): the
    squared norms of all scaled gradients are summed, and every gradient is shrunk by threshold / that norm when it is
    larger.  Three gradients of different sizes (one not a multiple of four, one empty), checked against numpy in
    float64: the accumulated sum, then each update."""
    from zoph_rnn_amd import capi
    g = synth.rng(114, 3)
    sizes = [70001, 37, 0, 4096]
    Ws = [U(g, (n,), -1, 1) for n in sizes]
    Gs = [U(g, (n,), -3, 3) for n in sizes]
    scale, lr = 1.0 / 16, 0.3
    d_ss = ctx.array(np.array([123.0]))  # stale content: the first call resets
    dGs = [ctx.array(G) if G.size else None for G in Gs]
    for i, (G, dG) in enumerate(zip(Gs, dGs)):
        ctx.grad_sumsq_accumulate(dG, G.size, scale, d_ss, reset=(i == 0))
    ctx.sync()
    want_ss = sum(((G.astype(np.float64) * scale) ** 2).sum() for G in Gs)
    assert d_ss.get()[0] == pytest.approx(want_ss, rel=1e-12)
    norm = np.sqrt(want_ss)
    coef = threshold / norm if norm > threshold else 1.0
    assert (coef < 1.0) == (threshold < 1.0)
    for W, G, dG in zip(Ws, Gs, dGs):
        if not G.size:
            continue
        dW = ctx.array(W)
        ctx.sgd_update_clipped(dW, dG, G.size, scale, capi.ZR_CLIP_WHOLE_NORM, threshold, d_ss, lr)
        ctx.sync()
        assert np.allclose(dW.get(), W + lr * coef * scale * G.astype(np.float64), rtol=1e-5, atol=1e-6)
    # reset with nothing to add clears the accumulator
    ctx.grad_sumsq_accumulate(None, 0, 1.0, d_ss, reset=True)
    ctx.sync()
    assert d_ss.get()[0] == 0.0
    # a gradient that does not start on a 16-byte boundary (the vector path must not be taken)
    G = U(g, (1001,), -2, 2)
    dG = ctx.array(G)
    ctx.grad_sumsq_accumulate(dG.at(1), 1000, 0.5, d_ss, reset=True)
    ctx.sync()
    assert d_ss.get()[0] == pytest.approx(((G[1:].astype(np.float64) * 0.5) ** 2).sum(), rel=1e-12)


def test_sgd_update_element_clip(ctx):
    """--ind-clip-gradients (clip_mat_kernel, src/custom_kernels.h:2220-2231): every element of the scaled gradient is
    clamped to +-threshold, whatever the norm.  Elements on both sides of both bounds, and exactly on them."""
    from zoph_rnn_amd import capi
    g = synth.rng(115, 1)
    n, thr, scale, lr = 5003, 0.1, 0.25, 0.7
    W, G = U(g, (n,), -1, 1), U(g, (n,), -1, 1)
    G[:4] = np.array([thr, -thr, 2 * thr, -2 * thr], np.float32) / scale
    dW = ctx.array(W)
    ctx.sgd_update_clipped(dW, ctx.array(G), n, scale, capi.ZR_CLIP_ELEMENT, thr, None, lr)
    ctx.sync()
    gs = np.clip(G * np.float32(scale), -np.float32(thr), np.float32(thr))
    assert (np.abs(G * scale) > thr).sum() > n // 4 and (np.abs(G * scale) < thr).sum() > n // 4
    assert np.allclose(dW.get(), W + np.float32(lr) * gs, rtol=1e-6, atol=1e-7)
    # mode 0: no clipping at all
    dW = ctx.array(W)
    ctx.sgd_update_clipped(dW, ctx.array(G), n, scale, capi.ZR_CLIP_NONE, 0.0, None, lr)
    ctx.sync()
    assert np.allclose(dW.get(), W + lr * scale * G.astype(np.float64), rtol=1e-5, atol=1e-6)


def test_clip_inplace(ctx):
    """clip_mat_kernel (src/custom_kernels.h:2220-2231): values beyond +-threshold are set to it, a NaN stays."""
    g = synth.rng(116, 1)
    x = U(g, (10007,), -3, 3)
    x[:5] = np.array([1.5, -1.5, np.nan, np.inf, -np.inf], np.float32)
    d = ctx.array(x)
    ctx.clip_inplace(d, x.size, 1.5)
    ctx.sync()
    got = d.get()
    assert np.isnan(got[2]) and got[3] == 1.5 and got[4] == -1.5
    keep = np.ones(x.size, bool)
    keep[2] = False
    assert np.array_equal(got[keep], np.clip(x[keep], -1.5, 1.5))


def test_sgd_update_clipped_rejects_bad_arguments(ctx):
    from zoph_rnn_amd import capi
    dW, dG = ctx.zeros((8,)), ctx.zeros((8,))
    with pytest.raises(RuntimeError):
        ctx.sgd_update_clipped(dW, dG, 8, 1.0, 7, 1.0, None, 0.1)
    with pytest.raises(RuntimeError):  # whole-model clipping needs the accumulated sum
        ctx.sgd_update_clipped(dW, dG, 8, 1.0, capi.ZR_CLIP_WHOLE_NORM, 1.0, None, 0.1)
    with pytest.raises(RuntimeError):
        ctx.sgd_update_clipped(dW, dG, 8, 1.0, capi.ZR_CLIP_ELEMENT, 0.0, None, 0.1)


def test_language_model_training_step_gradients(ctx):
    """benchmark configuration 1 shape (1-layer LM, H=100, minibatch 8, T=20, V=10000): the full gradient of the summed
    log-likelihood -- output layer, LSTM matrices and biases, embedding -- from one forward/backward pass."""
    c = synth.config1()
    H, mb, T, V = c["H"], c["mb"], c["T"], c["V"]
    L = len(c["layers"])
    n = H * mb
    ids, tgt_ids = c["ids"], c["targets"]
    nn, mask = o.vocab_prep(ids)
    # oracle: forward, per-step loss-layer backward (accumulated), then back-propagation through time
    hs, _ = o.lstm_stack_forward(c["embed"], c["layers"], nn, mask)
    dD = np.zeros((V, H), np.float64, order="F")
    db = np.zeros(V, np.float64)
    err_top = []
    for t in range(T):
        e, dD, db = o.softmax_backward(c["D"], c["b_d"], np.asfortranarray(hs[L - 1, t]), tgt_ids[t], np.ones(mb, np.int32),
                                       dD, db)
        err_top.append(e)
    want_g, want_e, _, _ = o.lstm_stack_backward(c["embed"], c["layers"], nn, mask, err_top)
    # GPU
    layers = [TrainLayer(ctx, ly) for ly in c["layers"]]
    d_embed = ctx.array(c["embed"])
    d_nn, d_m = ctx.empty(ids.size, np.int32), ctx.empty(ids.size, np.int32)
    ctx.vocab_prep(ctx.array(ids.reshape(-1)), ids.size, V, d_nn, d_m)
    z = ctx.zeros((H, mb))
    h_all, c_all, g_all = ([ctx.empty((n * T,)) for _ in range(L)] for _ in range(3))
    g_all = [ctx.empty((4 * n * T,)) for _ in range(L)]
    ctx.lstm_stack_forward_train([ly.w for ly in layers], d_embed, V, d_nn, d_m, T, mb, [z] * L, [z] * L, h_all, c_all,
                                 g_all)
    dDg, dbg = ctx.empty((V, H)), ctx.empty((V,))
    d_err_top, d_scr = ctx.empty((n * T,)), ctx.empty((V, T * mb))
    ones = ctx.array(np.ones(T * mb, np.int32))
    ctx.softmax_backward(ctx.array(c["D"]), ctx.array(c["b_d"]), V, H, h_all[L - 1], T * mb,
                         ctx.array(tgt_ids.reshape(-1).astype(np.int32)), ones, d_scr, d_err_top, dDg, dbg)
    dg_all = [ctx.empty((4 * n * T,)) for _ in range(L)]
    eh0, ec0 = [ctx.empty((H, mb)) for _ in range(L)], [ctx.empty((H, mb)) for _ in range(L)]
    d_below0 = ctx.empty((n * T,))
    ctx.lstm_stack_backward([ly.t for ly in layers], T, mb, d_m, [z] * L, c_all, g_all, d_err_top, dg_all, eh0, ec0,
                            d_err_below0=d_below0)
    x_all = ctx.empty((n * T,))
    ctx.embed_gather(d_embed, H, V, d_nn, T * mb, x_all)
    dM, dWh, dbl = ctx.empty((4 * H, H)), ctx.empty((4 * H, H)), ctx.empty((4 * H,))
    ctx.lstm_weight_gradients(H, T, mb, dg_all[0], x_all, z, h_all[0], dM, dWh, dbl)
    d_dW = ctx.zeros((H, V))
    ctx.embed_gradient(H, V, d_below0, d_nn, d_m, T * mb, d_dW)
    ctx.sync()
    fl = 0.05 * np.sqrt(T * mb)
    assert_close(dDg.get(), dD, floor=fl * 0.1, what="dD")
    assert_close(dbg.get(), db, floor=fl * 0.1, what="db_d")
    gM, gWh = _unstack(ctx, dM, H), _unstack(ctx, dWh, H)
    for q in range(4):
        assert_close(gM[q], want_g[0]["dM"][q], floor=fl * 0.1, what="dM gate %d" % q)
        assert_close(gWh[q], want_g[0]["dWh"][q], floor=fl * 0.1, what="dWh gate %d" % q)
        assert_close(dbl.get().reshape(4, H)[q], want_g[0]["db"][q], floor=fl * 0.1, what="db gate %d" % q)
    assert_close(d_dW.get(), want_e, floor=0.05, what="embedding gradient")
    for ly in layers:
        ly.close()


@pytest.mark.parametrize("L,H,mb,T,V,adjacent", [(2, 48, 9, 5, 60, True), (3, 64, 40, 4, 80, False)])
def test_node_by_node_backward_matches_oracle(ctx, L, H, mb, T, V, adjacent):
    """The reference's own schedule through the node-level entry points: per node the error step
    (zr_lstm_node_backward), then its gradient accumulation (zr_lstm_node_gradients), newest step first and top layer
    first.  adjacent: the two error outputs share one buffer (the single batched product) or not (scratch + copies)."""
    g = synth.rng(114, L * 100 + mb)
    embed = U(g, (H, V), -0.5, 0.5)
    layers_np = [synth.lstm_layer(g, H) for _ in range(L)]
    for ly in layers_np:
        ly["M"] = [U(g, (H, H), -0.2, 0.2) for _ in range(4)]
        ly["Wh"] = [U(g, (H, H), -0.2, 0.2) for _ in range(4)]
    ids = g.integers(0, V, size=(T, mb)).astype(np.int32)
    ids[:2, 1] = -1
    ids[T - 1:, 2] = -1
    nn, mask = o.vocab_prep(ids)
    h0 = [U(g, (H, mb), -0.5, 0.5) for _ in range(L)]
    c0 = [U(g, (H, mb), -0.5, 0.5) for _ in range(L)]
    err_top = [U(g, (H, mb), -1, 1) for _ in range(T)]
    want_g, want_e, want_eh0, want_ec0 = o.lstm_stack_backward(embed, layers_np, nn, mask, err_top, h0, c0)
    n = H * mb
    layers = [TrainLayer(ctx, ly) for ly in layers_np]
    d_embed = ctx.array(embed)
    d_nn, d_m = ctx.empty(ids.size, np.int32), ctx.empty(ids.size, np.int32)
    ctx.vocab_prep(ctx.array(ids.reshape(-1)), ids.size, V, d_nn, d_m)
    d_h0, d_c0 = [ctx.array(a) for a in h0], [ctx.array(a) for a in c0]
    h_all = [ctx.empty((n * T,)) for _ in range(L)]
    c_all = [ctx.empty((n * T,)) for _ in range(L)]
    g_all = [ctx.empty((4 * n * T,)) for _ in range(L)]
    ctx.lstm_stack_forward_train([ly.w for ly in layers], d_embed, V, d_nn, d_m, T, mb, d_h0, d_c0, h_all, c_all, g_all)
    x_all = ctx.empty((n * T,))
    ctx.embed_gather(d_embed, H, V, d_nn, T * mb, x_all)
    d_top = [ctx.array(e) for e in err_top]
    f4 = np.dtype(np.float32).itemsize
    dM = [ctx.zeros((4 * H, H)) for _ in range(L)]
    dWh = [ctx.zeros((4 * H, H)) for _ in range(L)]
    db = [ctx.zeros((4 * H,)) for _ in range(L)]
    d_dW = ctx.zeros((H, V))
    dg = ctx.empty((4 * H, mb))
    if adjacent:
        pair = [ctx.zeros((2 * n,)) for _ in range(L)]  # (error to h_{t-1}, error to below) per layer
        eh = [p.ptr for p in pair]
        below = [p.ptr + n * f4 for p in pair]
    else:
        eh_a, below_a = [ctx.zeros((n,)) for _ in range(L)], [ctx.zeros((n,)) for _ in range(L)]
        eh, below = [a.ptr for a in eh_a], [a.ptr for a in below_a]
    ec = [ctx.zeros((n,)) for _ in range(L)]
    for t in range(T - 1, -1, -1):
        for l in range(L - 1, -1, -1):
            gt = g_all[l].ptr + t * 4 * n * f4
            gates = [gt + k * n * f4 for k in range(4)]
            c_t = c_all[l].ptr + t * n * f4
            c_prev = d_c0[l].ptr if t == 0 else c_all[l].ptr + (t - 1) * n * f4
            h_prev = d_h0[l].ptr if t == 0 else h_all[l].ptr + (t - 1) * n * f4
            above = d_top[t].ptr if l == L - 1 else below[l + 1]
            last = t == T - 1
            ctx.lstm_node_backward(layers[l].t, mb, gates, c_t, c_prev, d_m.ptr + t * mb * 4, above,
                                   None if last else eh[l], None if last else ec[l], dg, eh[l], ec[l], below[l])
            d_in = x_all.ptr + t * n * f4 if l == 0 else h_all[l - 1].ptr + t * n * f4
            ctx.lstm_node_gradients(H, mb, dg, d_in, h_prev, dM[l], dWh[l], db[l])
            if l == 0:
                ctx.embed_gradient(H, V, below[0], d_nn.ptr + t * mb * 4, d_m.ptr + t * mb * 4, mb, d_dW)
    ctx.sync()
    wfloor = 0.05 * np.sqrt(T * mb)
    got = lambda p: ctx_get(ctx, p, (H, mb))
    for l in range(L):
        assert_close(got(eh[l]), want_eh0[l], what="err_h0 layer %d" % l)
        assert_close(ec[l].get().reshape(H, mb, order="F"), want_ec0[l], what="err_c0 layer %d" % l)
        gM, gWh, gb = _unstack(ctx, dM[l], H), _unstack(ctx, dWh[l], H), db[l].get().reshape(4, H)
        for q in range(4):
            assert_close(gM[q], want_g[l]["dM"][q], floor=wfloor, what="dM layer %d gate %d" % (l, q))
            assert_close(gWh[q], want_g[l]["dWh"][q], floor=wfloor, what="dWh layer %d gate %d" % (l, q))
            assert_close(gb[q], want_g[l]["db"][q], floor=wfloor, what="db layer %d gate %d" % (l, q))
    assert_close(d_dW.get(), want_e, floor=0.05 * np.sqrt(T), what="embedding gradient")
    for ly in layers:
        ly.close()


def ctx_get(ctx, ptr, shape):
    """Device memory at a raw address as a column-major host array."""
    import ctypes
    flat = np.empty(int(np.prod(shape)), np.float32)
    rc = capi.load().zr_d2h(ctx.h, flat.ctypes.data_as(ctypes.c_void_p), ctypes.c_void_p(int(ptr)),
                            ctypes.c_size_t(flat.nbytes))
    assert rc == 0
    return flat.reshape(shape, order="F")


@pytest.mark.parametrize("V,H,mb,T", [(301, 32, 7, 4), (2000, 64, 48, 3)])
def test_softmax_backward_step_by_step_accumulates(ctx, V, H, mb, T):
    """One zr_softmax_backward_accumulate call per time step adds up to the all-columns call and to the oracle."""
    g = synth.rng(115, V)
    D, bd = U(g, (V, H), -0.5, 0.5), U(g, (V,), -1, 1)
    hs = [U(g, (H, mb), -1, 1) for _ in range(T)]
    tg = [g.integers(0, V, size=mb).astype(np.int32) for _ in range(T)]
    mk = [(g.random(mb) > 0.2).astype(np.int32) for _ in range(T)]
    dD, db = np.zeros((V, H), np.float64, order="F"), np.zeros(V, np.float64)
    want_e = []
    for t in range(T):
        e, dD, db = o.softmax_backward(D, bd, hs[t], tg[t], mk[t], dD, db)
        want_e.append(e)
    d_D, d_b = ctx.array(D), ctx.array(bd)
    d_dD, d_db, d_scr = ctx.zeros((V, H)), ctx.zeros((V,)), ctx.empty((V, mb))
    for t in range(T):
        d_e = ctx.empty((H, mb))
        ctx.softmax_backward(d_D, d_b, V, H, ctx.array(hs[t]), mb, ctx.array(tg[t]), ctx.array(mk[t]), d_scr, d_e, d_dD,
                             d_db, accumulate=True)
        ctx.sync()
        assert_close(d_e.get(), want_e[t], what="err_h step %d" % t)
    assert_close(d_dD.get(), dD, floor=0.05 * np.sqrt(T * mb), what="dD")
    assert_close(d_db.get(), db, floor=0.05 * np.sqrt(T * mb), what="db")


@pytest.mark.parametrize("H,mb,S,D", [(64, 6, 9, 2), (100, 8, 20, 10), (52, 33, 12, 12), (30, 5, 7, 3), (300, 70, 40, 50),
                                      (1000, 16, 30, 10)])
def test_attention_backward_against_oracle(ctx, H, mb, S, D):
    """zr_attn_backward (attention_node::back_prop) against the oracle, whose restatement is pinned by torch autograd:
    the error of h_t, the error added to every source state, and the six weight gradients, all accumulated on top of
    non-zero starting values; short sources, windows cut at both ends, masked columns, row tails."""
    g = synth.rng(41, H + S)
    w = synth.attention_weights(g, H)
    if H <= 128:
        for k in ("W_a", "W_p", "W_c1", "W_c2"):
            w[k] = U(g, (H, H), -0.3, 0.3)
    hs = (g.standard_normal(size=(S, H, mb), dtype=np.float32) * np.float32(0.5 if H <= 128 else 0.1))
    lens = g.integers(1, S + 1, size=mb).astype(np.int32)
    lens[0] = S
    batch_info = np.concatenate([lens, S - lens]).astype(np.int32)
    mask = (g.random(mb) > 0.15).astype(np.int32)
    mask[0] = 1
    h_t = U(g, (H, mb), -1, 1)
    err = U(g, (H, mb), -1, 1)
    fwd = o.attention_forward(hs_table=hs, batch_info=batch_info, h_t=h_t, mask01=mask, D=D, **w)
    g0 = {k: np.asfortranarray(U(g, (H, H), -0.5, 0.5)) for k in ("W_a", "W_p", "W_c1", "W_c2")}
    g0["v_p"], g0["bias"] = U(g, (H,), -0.5, 0.5), U(g, (H,), -0.5, 0.5)
    ehs0 = (g.standard_normal(size=(S, H, mb), dtype=np.float32) * np.float32(0.5))
    want_eh, want_ehs, want_g = o.attention_backward(w["W_a"], w["W_p"], w["v_p"], w["W_c1"], w["W_c2"], hs, batch_info,
                                                     h_t, mask, fwd, err, D,
                                                     grads={k: v.copy(order="F") for k, v in g0.items()}, err_hs=ehs0)
    # the library's own forward outputs feed its backward, as in training
    tables = [ctx.array(np.asfortranarray(hs[t])) for t in range(S)]
    etables = [ctx.array(np.asfortranarray(ehs0[t])) for t in range(S)]
    dw = {k: ctx.array(v) for k, v in w.items()}
    a = ctx.attn_create(H, mb, D, dw["W_a"], dw["W_p"], dw["v_p"], dw["out_bias"], dw["W_c1"], dw["W_c2"], tables)
    ctx.attn_set_error_tables(a, etables)
    Wn = 2 * D + 1
    d_ht, d_al, d_ix, d_pt, d_cx = (ctx.empty((H, mb)), ctx.empty((mb, Wn)), ctx.empty((mb, Wn), np.int32),
                                    ctx.empty((mb,)), ctx.empty((H, mb)))
    d_bi, d_h, d_m = ctx.array(batch_info), ctx.array(h_t), ctx.array(mask)
    ctx.attn_step(a, d_bi, d_h, d_m, d_ht, d_al, d_ix, d_pt, d_cx)
    d_g = [ctx.array(g0[k]) for k in ("W_a", "W_p", "v_p", "bias", "W_c1", "W_c2")]
    d_err, d_eh = ctx.array(err), ctx.empty((H, mb))
    ctx.attn_backward(a, d_bi, d_h, d_m, d_ht, d_al, d_ix, d_pt, d_cx, d_err, d_eh, d_g)
    ctx.sync()
    assert np.array_equal(d_ix.get(), fwd["indices"])
    assert_close(d_eh.get(), want_eh, what="error of h_t")
    for t in range(S):
        assert_close(etables[t].get(), want_ehs[t], what="error of source state %d" % t)
    for d, k in zip(d_g, ("W_a", "W_p", "v_p", "bias", "W_c1", "W_c2")):
        assert_close(d.get().reshape(want_g[k].shape, order="F"), want_g[k], what="gradient of " + k)
    assert np.all(d_eh.get()[:, mask == 0] == 0)
    # in place: the error of h_t may overwrite the error of h~ (the reference copies it there, :654)
    for d, k in zip(d_g, ("W_a", "W_p", "v_p", "bias", "W_c1", "W_c2")):
        d.set(g0[k])
    ctx.attn_backward(a, d_bi, d_h, d_m, d_ht, d_al, d_ix, d_pt, d_cx, d_err, d_err, d_g)
    ctx.sync()
    assert d_err.get().tobytes() == d_eh.get().tobytes()
    ctx.attn_destroy(a)


@pytest.mark.parametrize("n,rate", [(1000, 0.8), (70001, 0.3), (5, 1.0)])
def test_dropout_apply_bit_exact_and_uniform_fill(ctx, n, rate):
    """dropout_kernel on given uniform numbers: bit for bit the oracle's; the library's own uniform numbers lie in
    (0, 1], repeat for the same (seed, call) and differ for another call, with the mean and keep fraction of a uniform
    sample."""
    g = synth.rng(43, n)
    x = U(g, (n,), -2, 2)
    u = g.random(n, dtype=np.float32)
    d_x, d_u = ctx.array(x), ctx.array(u)
    ctx.dropout_apply(d_u, rate, d_x, n)
    ctx.sync()
    assert np.array_equal(d_x.get(), o.dropout(u, rate, x))
    a, b, c = ctx.empty((n,)), ctx.empty((n,)), ctx.empty((n,))
    ctx.uniform_fill(1234, 7, a, n)
    ctx.uniform_fill(1234, 7, b, n)
    ctx.uniform_fill(1234, 8, c, n)
    ctx.sync()
    ua, uc = a.get(), c.get()
    assert ua.tobytes() == b.get().tobytes() and not np.array_equal(ua, uc)
    assert ua.min() > 0 and ua.max() <= 1
    if n >= 1000:
        assert abs(ua.mean() - 0.5) < 4 * 0.2887 / np.sqrt(n)
        assert abs((ua < 0.3).mean() - 0.3) < 4 * np.sqrt(0.21 / n)
        assert abs(np.corrcoef(ua[:-1], ua[1:])[0, 1]) < 5 / np.sqrt(n)


@pytest.mark.parametrize("H,mb", [(48, 9), (100, 33), (1000, 16)])
def test_lstm_feed_backward_against_oracle(ctx, H, mb):
    g = synth.rng(44, H)
    Q = [U(g, (H, H), -0.3, 0.3) for _ in range(4)]
    ht = U(g, (H, mb), -1, 1)
    dg = U(g, (4 * H, mb), -1, 1)
    dQ0 = U(g, (4 * H, H), -0.5, 0.5)
    want_err, want_dQ = o.lstm_feed_backward(Q, dg, ht, dQ=[np.asfortranarray(dQ0[k * H:(k + 1) * H]) for k in range(4)])
    d_err, d_dQ = ctx.empty((H, mb)), ctx.array(dQ0)
    ctx.lstm_feed_backward([ctx.array(q) for q in Q], H, mb, ctx.array(dg), ctx.array(ht), d_err, d_dQ)
    ctx.sync()
    assert_close(d_err.get(), want_err, what="error of h~")
    got = d_dQ.get()
    for k in range(4):
        assert_close(got[k * H:(k + 1) * H], want_dQ[k], what="gradient of Q[%d]" % k)
