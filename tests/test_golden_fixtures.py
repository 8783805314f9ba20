"""Golden fixtures (tests/golden/*.npz, written by tests/golden/make_fixtures.py from the CPU oracle).

The reference holds no expected outputs for this path, so the fixtures freeze the oracle: the CPU test regenerates every
fixture and compares it with the committed file, the GPU tests run the HIP path on the committed inputs and compare with
the committed outputs (fp32 results within 1e-4 relative, floor 0.05 as everywhere; ids, window indices, words and
back-pointers exact)."""
import importlib.util
import os

import numpy as np
import pytest

HERE = os.path.dirname(os.path.abspath(__file__))
GOLDEN = os.path.join(HERE, "golden")


def _load(name):
    with np.load(os.path.join(GOLDEN, name + ".npz"), allow_pickle=False) as z:
        return {k: z[k] for k in z.files}


def _generator():
    spec = importlib.util.spec_from_file_location("make_fixtures", os.path.join(GOLDEN, "make_fixtures.py"))
    mod = importlib.util.module_from_spec(spec)
    spec.loader.exec_module(mod)
    return mod


@pytest.mark.parametrize("name", ["lstm_two_layers", "attention_local_p", "softmax_output_layer", "beam_one_sentence",
                                  "beam_viterbi_one_sentence", "lstm_stack_backward_clamped"])
def test_oracle_reproduces_the_committed_fixture(name):
    want = _load(name)
    got = _generator().FIXTURES[name]()
    assert sorted(got) == sorted(want)
    for k, w in want.items():
        g = np.asarray(got[k])
        assert g.shape == w.shape and g.dtype == w.dtype, (name, k, g.shape, w.shape, g.dtype, w.dtype)
        if np.issubdtype(w.dtype, np.integer):
            assert np.array_equal(g, w), (name, k)
        else:
            # the oracle accumulates in double in a fixed order; the slack covers a different libm on another machine
            assert np.allclose(g, w, rtol=1e-6, atol=1e-7), (name, k, float(np.abs(g - w).max()))


# ------------------------------------------------------------------------------------------------------- GPU side
@pytest.fixture(scope="module")
def ctx():
    from zoph_rnn_amd import capi
    c = capi.Context(0)
    yield c
    c.close()


@pytest.mark.gpu
def test_gpu_lstm_layers_match_the_fixture(ctx):
    from gpu_util import Layer, assert_close
    f = _load("lstm_two_layers")
    H, mb = f["l0_hprev"].shape
    V = f["embed"].shape[1]
    lys, layers = [], []
    for l in range(2):
        ly = {"M": [f["l%d_M%d" % (l, g)] for g in range(4)], "Wh": [f["l%d_Wh%d" % (l, g)] for g in range(4)],
              "b": [f["l%d_b%d" % (l, g)] for g in range(4)]}
        if "l%d_Q0" % l in f:
            ly["Q"] = [f["l%d_Q%d" % (l, g)] for g in range(4)]
        lys.append(ly)
        layers.append(Layer(ctx, ly))
    try:
        d_h = [ctx.zeros((H, mb)) for _ in range(2)]
        d_c = [ctx.zeros((H, mb)) for _ in range(2)]
        ctx.lstm_decoder_step([ly.w for ly in layers], ctx.array(f["embed"]), V, ctx.array(f["ids"]),
                              [ctx.array(f["l%d_hprev" % l]) for l in range(2)],
                              [ctx.array(f["l%d_cprev" % l]) for l in range(2)], ctx.array(f["mask"]), mb, d_h, d_c,
                              d_htild=ctx.array(f["l0_htild"]), clip=float(f["clip"]))
        ctx.sync()
        for l in range(2):
            assert_close(d_h[l].get(), f["l%d_h" % l], what="h of layer %d" % l)
            assert_close(d_c[l].get(), f["l%d_c" % l], what="c of layer %d" % l)
            assert np.all(d_h[l].get()[:, f["mask"] == 0] == 0)
    finally:
        for ly in layers:
            ly.close()


@pytest.mark.gpu
@pytest.mark.parametrize("prepared", [False, True])
def test_gpu_attention_matches_the_fixture(ctx, prepared):
    from gpu_util import assert_close
    f = _load("attention_local_p")
    S, H, mb = f["hs"].shape
    D = int(f["D"])
    Wn = 2 * D + 1
    tables = [ctx.array(np.asfortranarray(f["hs"][t])) for t in range(S)]
    dw = {k: ctx.array(f[k]) for k in ("W_a", "W_p", "v_p", "out_bias", "W_c1", "W_c2")}
    a = ctx.attn_create(H, mb, D, dw["W_a"], dw["W_p"], dw["v_p"], dw["out_bias"], dw["W_c1"], dw["W_c2"], tables)
    if prepared:
        ctx.attn_prepare(a)
    d_ht, d_al, d_ix, d_pt, d_cx = (ctx.empty((H, mb)), ctx.empty((mb, Wn)), ctx.empty((mb, Wn), np.int32),
                                    ctx.empty((mb,)), ctx.empty((H, mb)))
    ctx.attn_step(a, ctx.array(f["batch_info"]), ctx.array(f["h_t"]), ctx.array(f["mask"]), d_ht, d_al, d_ix, d_pt, d_cx)
    ctx.sync()
    assert np.array_equal(d_ix.get(), f["out_indices"])
    assert_close(d_pt.get(), f["out_p_t"], what="p_t")
    assert_close(d_al.get(), f["out_alignments"], floor=1e-4, what="alignments")
    assert_close(d_cx.get(), f["out_c_ctx"], what="context")
    assert_close(d_ht.get(), f["out_h_tild"], what="h_tild")
    ctx.attn_destroy(a)


@pytest.mark.gpu
def test_gpu_output_layer_matches_the_fixture(ctx):
    from gpu_util import assert_close
    from zoph_rnn_amd import capi
    f = _load("softmax_output_layer")
    V, H = f["D"].shape
    mb = f["h"].shape[1]
    dD, dbd, dh = ctx.array(f["D"]), ctx.array(f["b_d"]), ctx.array(f["h"])
    d_p, d_lp, d_scr = ctx.empty((V, mb)), ctx.empty((V, mb)), ctx.empty((V, mb))
    ctx.softmax_forward(dD, dbd, V, H, dh, mb, capi.ZR_SOFTMAX_PROB, d_p, d_scr)
    ctx.softmax_forward(dD, dbd, V, H, dh, mb, capi.ZR_SOFTMAX_LOGPROB, d_lp)
    ctx.sync()
    assert_close(d_scr.get(), f["logits"], what="logits")
    assert_close(d_p.get(), f["prob"], floor=1e-7, what="probabilities")
    assert_close(d_lp.get(), f["logprob"], what="log-probabilities")
    got = ctx.softmax_loss(dD, dbd, V, H, dh, mb, ctx.array(f["target"]), ctx.array(f["mask"]), d_scr)
    assert got == pytest.approx(float(f["loss"]), rel=1e-5, abs=1e-6)


@pytest.mark.gpu
def test_gpu_beam_matches_the_fixture(ctx):
    f = _load("beam_one_sentence")
    beam, max_len = int(f["beam"]), int(f["max_len"])
    steps, V = f["prob"].shape[0] - 1, f["prob"].shape[1]
    b = ctx.beam_create(beam, V, 1, max_len, float(f["penalty"]))
    d_words, d_back = ctx.empty(beam, np.int32), ctx.empty(beam, np.int32)
    for index in range(steps):
        ctx.beam_expand(b, ctx.array(np.asfortranarray(f["prob"][index])), index, d_words, d_back)
        ctx.sync()
        assert np.array_equal(d_words.get(), f["words"][index]), index
        assert np.array_equal(d_back.get(), f["backptr"][index]), index
        sc, w2 = ctx.beam_state(b, 0, beam)
        live = f["words"][index] != -1
        assert np.allclose(sc[live], f["scores"][index][live], rtol=1e-4, atol=1e-5)
    ctx.beam_finish(b, ctx.array(np.asfortranarray(f["prob"][steps])))
    ctx.sync()
    got, n = ctx.beam_hypotheses(b, 0, cap=len(f["hyp_scores"]) + 4, max_len=max_len)
    assert n == len(f["hyp_scores"])
    for i, (gw, gs) in enumerate(got):
        want = f["hyp_words"][i]
        assert np.array_equal(gw, want[want != -1])
        assert gs == pytest.approx(float(f["hyp_scores"][i]), rel=1e-4, abs=1e-5)
    ctx.beam_destroy(b)


@pytest.mark.gpu
def test_gpu_beam_viterbi_alignments_match_the_fixture(ctx):
    f = _load("beam_viterbi_one_sentence")
    beam, max_len = int(f["beam"]), int(f["max_len"])
    steps, V = f["prob"].shape[0] - 1, f["prob"].shape[1]
    b = ctx.beam_create(beam, V, 1, max_len, float(f["penalty"]))
    d_vit = ctx.empty(beam, np.int32)
    ctx.beam_set_viterbi(b, True, d_vit)
    d_words, d_back = ctx.empty(beam, np.int32), ctx.empty(beam, np.int32)
    for index in range(steps):
        d_vit.set(f["viterbi"][index])
        ctx.beam_expand(b, ctx.array(np.asfortranarray(f["prob"][index])), index, d_words, d_back)
    d_vit.set(f["viterbi"][steps])
    ctx.beam_finish(b, ctx.array(np.asfortranarray(f["prob"][steps])))
    ctx.sync()
    n_want = f["hyp_words"].shape[0]
    got, n = ctx.beam_hypotheses(b, 0, cap=n_want + 4, max_len=max_len)
    vit, nv = ctx.beam_hypotheses_viterbi(b, 0, cap=n_want + 4, max_len=max_len)
    assert n == nv == n_want
    for i in range(n_want):
        ln = int(f["hyp_len"][i])
        assert np.array_equal(got[i][0], f["hyp_words"][i, :ln])
        assert np.array_equal(vit[i, :ln], f["hyp_viterbi"][i, :ln])
    ctx.beam_destroy(b)
