"""Beam search on the device against the oracle's restatement of the reference decoder (std::priority_queue
based, one sentence at a time).  Word ids and back-pointers must be bit-exact; scores within 1e-4 relative.
Inputs are tie-free random distributions (exact ties follow libstdc++'s heap order in the reference, which
the device path does not reproduce) plus one tie case whose outcome does not depend on that order."""
import numpy as np
import pytest

import oracle_lib as o
from zoph_rnn_amd import capi, synth

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def ctx():
    c = capi.Context(0)
    yield c
    c.close()


def _random_dist(g, V, cols, peaky=2.0, eof_boost=0.0):
    logits = g.standard_normal(size=(V, cols)) * peaky
    logits[1, :] += eof_boost
    e = np.exp(logits - logits.max(axis=0))
    return np.asfortranarray((e / e.sum(axis=0)).astype(np.float32))


def _decode_both(ctx, V, beam, n_sent, steps, max_len, penalty, seed, eof_boost, viterbi=None):
    """viterbi: None (not tracked), "given" (random alignments per column and step) or "absent" (tracked, but no
    alignments handed over: the reference's -1)."""
    g = synth.rng(seed, 21)
    b = ctx.beam_create(beam, V, n_sent, max_len, penalty)
    d_vit = ctx.empty(n_sent * beam, np.int32) if viterbi == "given" else None
    if viterbi:
        ctx.beam_set_viterbi(b, True, d_vit)

    def alignments():
        if viterbi != "given":
            return [None] * n_sent
        v = g.integers(0, 60, size=n_sent * beam).astype(np.int32)
        d_vit.set(v)
        return [v[s * beam:(s + 1) * beam] for s in range(n_sent)]
    decs = [o.Decoder(beam, V, max_len, penalty=penalty) for _ in range(n_sent)]
    d_words, d_back = ctx.empty(n_sent * beam, np.int32), ctx.empty(n_sent * beam, np.int32)
    d_prob = ctx.empty((V, n_sent * beam))
    for index in range(steps):
        P = _random_dist(g, V, n_sent * beam, eof_boost=eof_boost)
        d_prob.set(P)
        vit = alignments()
        ctx.beam_expand(b, d_prob, index, d_words, d_back)
        ctx.sync()
        words, back = d_words.get(), d_back.get()
        for s in range(n_sent):
            decs[s].expand(P[:, s * beam:(s + 1) * beam], index, vit[s])
            st = decs[s].state()
            assert np.array_equal(words[s * beam:(s + 1) * beam], st["current_indices"]), (index, s)
            assert np.array_equal(back[s * beam:(s + 1) * beam] - s * beam, st["new_indicies_changes"]), (index, s)
            sc, w2 = ctx.beam_state(b, s, beam)
            live = st["current_indices"] != -1
            assert np.allclose(sc[live], st["scores"][live], rtol=1e-4, atol=1e-5)
            assert np.array_equal(w2, st["current_indices"])
    P = _random_dist(g, V, n_sent * beam)
    d_prob.set(P)
    vit = alignments()
    ctx.beam_finish(b, d_prob)
    ctx.sync()
    for s in range(n_sent):
        decs[s].finish(P[:, s * beam:(s + 1) * beam], vit[s])
        want = decs[s].hypotheses()
        got, n = ctx.beam_hypotheses(b, s, cap=len(want) + 8, max_len=max_len)
        assert n == len(want), (s, n, len(want))
        for (gw, gs), (ww, ws) in zip(got, want):
            assert np.array_equal(gw, ww)
            assert gs == pytest.approx(ws, rel=1e-4, abs=1e-5)
        if viterbi:
            got_v, nv = ctx.beam_hypotheses_viterbi(b, s, cap=len(want) + 8, max_len=max_len)
            want_v = decs[s].hypotheses_viterbi()
            assert nv == len(want_v)
            for gv, wv in zip(got_v, want_v):
                assert np.array_equal(gv[:len(wv)], wv), (s, gv, wv)
    if not viterbi:
        with pytest.raises(capi.ZrError):
            ctx.beam_hypotheses_viterbi(b, 0, cap=4, max_len=max_len)
    ctx.beam_destroy(b)


@pytest.mark.parametrize("V,beam,n_sent,steps", [(50, 4, 1, 6), (500, 12, 3, 8), (97, 3, 5, 10), (40, 1, 2, 5)])
def test_beam_against_reference_rules(ctx, V, beam, n_sent, steps):
    _decode_both(ctx, V, beam, n_sent, steps, max_len=steps + 4, penalty=0.0, seed=V + beam, eof_boost=0.0)


@pytest.mark.parametrize("mode", ["given", "absent"])
@pytest.mark.parametrize("V,beam,n_sent,steps,eof_boost", [(60, 5, 4, 9, 3.0), (500, 12, 3, 8, 0.0), (40, 1, 2, 5, 1.0),
                                                          (50000, 12, 4, 6, 6.0)])
def test_beam_carries_viterbi_alignments(ctx, V, beam, n_sent, steps, eof_boost, mode):
    """The alignment histories of all finished hypotheses (those ended by an <EOF> candidate inside expand and those
    ended by the forced finish), bit-exact against the oracle's decoder; words, scores and back-pointers as without."""
    _decode_both(ctx, V, beam, n_sent, steps, max_len=steps + 4, penalty=0.2, seed=3 * V + beam, eof_boost=eof_boost,
                 viterbi=mode)


def test_beam_viterbi_tracking_must_start_before_the_first_step(ctx):
    """Alignments of steps already taken cannot be made up: switching the tracking on after an expand is refused, and
    so are alignments handed over with the tracking off; switching it off and on again before a sentence is fine."""
    V, beam = 50, 3
    g = synth.rng(5, 21)
    b = ctx.beam_create(beam, V, 1, 8, 0.0)
    d_words, d_back = ctx.empty(beam, np.int32), ctx.empty(beam, np.int32)
    d_vit = ctx.zeros(beam, np.int32)
    with pytest.raises(capi.ZrError):
        ctx.beam_set_viterbi(b, False, d_vit)
    ctx.beam_expand(b, ctx.array(_random_dist(g, V, beam)), 0, d_words, d_back)
    with pytest.raises(capi.ZrError):
        ctx.beam_set_viterbi(b, True, d_vit)
    ctx.beam_init(b)
    ctx.beam_set_viterbi(b, True, d_vit)
    ctx.beam_set_viterbi(b, False)
    ctx.beam_set_viterbi(b, True, None)
    ctx.beam_expand(b, ctx.array(_random_dist(g, V, beam)), 0, d_words, d_back)
    ctx.beam_finish(b, ctx.array(_random_dist(g, V, beam)))
    ctx.sync()
    vit, n = ctx.beam_hypotheses_viterbi(b, 0, cap=16, max_len=8)
    assert n >= 1 and np.all(vit[:, 0] == -20) and np.all(vit[:, 1] == -1)
    ctx.beam_destroy(b)


def test_beam_with_frequent_eof_and_penalty(ctx):
    """<EOF> made likely: hypotheses finish inside expand without consuming beam slots; a word penalty is added."""
    _decode_both(ctx, 60, 5, 4, 7, max_len=12, penalty=0.3, seed=7, eof_boost=4.0)


def test_beam_batching_does_not_change_a_sentence(ctx):
    """16 sentences decoded together give, per sentence, what a single-sentence decode gives."""
    V, beam, n_sent, steps, max_len = 300, 12, 16, 5, 10
    g = synth.rng(31, 21)
    Ps = [_random_dist(g, V, n_sent * beam) for _ in range(steps)]
    d_words, d_back = ctx.empty(n_sent * beam, np.int32), ctx.empty(n_sent * beam, np.int32)
    big = ctx.beam_create(beam, V, n_sent, max_len)
    hist = []
    for index, P in enumerate(Ps):
        ctx.beam_expand(big, ctx.array(P), index, d_words, d_back)
        ctx.sync()
        hist.append((d_words.get().copy(), d_back.get().copy()))
    d_w1, d_b1 = ctx.empty(beam, np.int32), ctx.empty(beam, np.int32)
    for s in (0, 7, 15):
        one = ctx.beam_create(beam, V, 1, max_len)
        for index, P in enumerate(Ps):
            ctx.beam_expand(one, ctx.array(np.asfortranarray(P[:, s * beam:(s + 1) * beam])), index, d_w1, d_b1)
            ctx.sync()
            assert np.array_equal(d_w1.get(), hist[index][0][s * beam:(s + 1) * beam])
            assert np.array_equal(d_b1.get(), hist[index][1][s * beam:(s + 1) * beam] - s * beam)
        ctx.beam_destroy(one)
    ctx.beam_destroy(big)


def test_beam_all_equal_probabilities(ctx):
    """All probabilities equal: the kept words are 0..beam; <START> is skipped, <EOF> finishes, the remaining
    slots are filled and the last one falls into the empty-heap branch -- a result that does not depend on the
    order among the tied entries apart from which of the two equal survivors comes first."""
    V, beam = 12, 3
    b = ctx.beam_create(beam, V, 1, 6)
    d_words, d_back = ctx.empty(beam, np.int32), ctx.empty(beam, np.int32)
    ctx.beam_expand(b, ctx.array(np.full((V, beam), 0.125, np.float32, order="F")), 0, d_words, d_back)
    ctx.sync()
    w = d_words.get()
    assert sorted(w[:2].tolist()) == [2, 3] and w[2] == -1
    hyps, n = ctx.beam_hypotheses(b, 0, cap=4, max_len=6)
    assert n == 1 and hyps[0][0].tolist() == [0, 1]
    ctx.beam_destroy(b)


def test_beam_full_vocab_shape(ctx):
    """V=50000, beam 12, 16 sentences (192 columns): selection equals a full sort of every column."""
    V, beam, n_sent = 50000, 12, 16
    g = synth.rng(41, 21)
    P = _random_dist(g, V, n_sent * beam, peaky=3.0)
    b = ctx.beam_create(beam, V, n_sent, 8)
    d_words, d_back = ctx.empty(n_sent * beam, np.int32), ctx.empty(n_sent * beam, np.int32)
    d_prob = ctx.array(P)
    for index in range(2):
        ctx.beam_expand(b, d_prob, index, d_words, d_back)
        ctx.sync()
        words, back = d_words.get(), d_back.get()
        for s in (0, 5, 15):
            dec = o.Decoder(beam, V, 8)
            for i2 in range(index + 1):
                dec.expand(P[:, s * beam:(s + 1) * beam], i2)
            st = dec.state()
            assert np.array_equal(words[s * beam:(s + 1) * beam], st["current_indices"])
            assert np.array_equal(back[s * beam:(s + 1) * beam] - s * beam, st["new_indicies_changes"])
    ctx.beam_destroy(b)


def _expand_given(ctx, Ps, beam, n_sent, max_len):
    """beam_expand over the given distributions against the oracle decoder, word ids and back-pointers bit-exact."""
    V = Ps[0].shape[0]
    b = ctx.beam_create(beam, V, n_sent, max_len, 0.0)
    decs = [o.Decoder(beam, V, max_len) for _ in range(n_sent)]
    d_words, d_back = ctx.empty(n_sent * beam, np.int32), ctx.empty(n_sent * beam, np.int32)
    for index, P in enumerate(Ps):
        ctx.beam_expand(b, ctx.array(P), index, d_words, d_back)
        ctx.sync()
        words, back = d_words.get(), d_back.get()
        for s in range(n_sent):
            decs[s].expand(P[:, s * beam:(s + 1) * beam], index)
            st = decs[s].state()
            assert np.array_equal(words[s * beam:(s + 1) * beam], st["current_indices"]), (index, s)
            assert np.array_equal(back[s * beam:(s + 1) * beam] - s * beam, st["new_indicies_changes"]), (index, s)
    ctx.beam_destroy(b)


@pytest.mark.parametrize("V", [20000, 8192 * 3 + 5, 600000])
def test_beam_all_equal_probabilities_large_vocab(ctx, V):
    """Every word equally probable, over several chunks of the selection kernel (and, at 600 000 words, over its large
    chunks): the probability-only bound of the first stage lets every element through, the candidate list overflows
    and the exact bound takes over.  Equal probabilities rank by lower word id, so the beam + 1 kept words are
    0..beam: <START> is skipped, <EOF> finishes a hypothesis, words 2..beam survive and the last slot stays empty."""
    beam = 12
    b = ctx.beam_create(beam, V, 1, 6)
    d_words, d_back = ctx.empty(beam, np.int32), ctx.empty(beam, np.int32)
    ctx.beam_expand(b, ctx.array(np.full((V, beam), np.float32(1.0 / V), np.float32, order="F")), 0, d_words, d_back)
    ctx.sync()
    w = d_words.get()
    assert sorted(w[:beam - 1].tolist()) == list(range(2, beam + 1)) and w[beam - 1] == -1
    hyps, n = ctx.beam_hypotheses(b, 0, cap=4, max_len=6)
    assert n == 1 and hyps[0][0].tolist() == [0, 1]
    ctx.beam_destroy(b)


@pytest.mark.parametrize("V,beam", [(40003, 12), (16384, 5), (16385, 31), (70000, 20), (8193, 12)])
def test_beam_selection_on_adversarial_layouts(ctx, V, beam):
    """Layouts chosen against the selection kernel's structure (one workgroup per 8192 or 16384 words, each thread holding
    words 4t..4t+3 of every 1024): the largest values all inside one thread's share, at chunk boundaries, in the
    ragged tail, and values that fall steadily with the word id; vocabulary sizes that are not multiples of 4 take the scalar-load path."""
    g = synth.rng(43, V)
    n_sent = 2
    cols = n_sent * beam
    # distinct small values: a random permutation of an evenly spaced grid in every column
    base = np.stack([g.permutation(V) for _ in range(cols)], axis=1) * (1e-3 / V) + 1e-4
    P = []
    a = base.copy()                                    # step 0: big values in thread 5's words of chunk 0
    idx = np.array([4 * 5 + c + 1024 * i for i in range(16) for c in range(4)])
    idx = idx[(idx > 1) & (idx < V)]
    a[idx, :] += 1.0 + g.random((idx.size, cols))
    P.append(a)
    a = base.copy()                                    # step 1: big values around chunk boundaries and the tail
    edge = np.array([v for v in (8191, 8192, 16383, 16384, 16385, 32767, 32768, V - 1, V - 2, V - 3, 2, 3)
                     if 1 < v < V and (v > 8192 or V < 16384)])  # (the 8192 boundary only in the case added for it)
    a[edge, :] += 1.0 + g.random((edge.size, cols))
    P.append(a)
    a = base.copy()                                    # step 2: values falling with the word id
    a += np.exp(-np.arange(V) / 200.0)[:, None] * (1.0 + 0.01 * np.arange(cols))[None, :]
    P.append(a)
    a = base.copy()                                    # step 3: in every wave of chunk 0, `beam` threads whose whole
    ts = [w * 64 + j for w in range(4) for j in range(beam)]   # share is large: the list built from the wave-level
    idx = np.array([4 * t + c + 1024 * i for t in ts for i in range(16) for c in range(4)])  # bound overflows
    idx = idx[(idx > 1) & (idx < V)]
    a[idx, :] = 1.0 + np.stack([g.permutation(idx.size) for _ in range(cols)], axis=1) / idx.size
    P.append(a)
    Ps = [np.asfortranarray((p / p.sum(axis=0)).astype(np.float32)) for p in P]
    for p in Ps:  # the oracle comparison needs tie-free columns at the top
        top = np.sort(p, axis=0)[-(beam + 2):]
        assert np.all(np.diff(top, axis=0) > 0)
    _expand_given(ctx, Ps, beam, n_sent, max_len=8)


@pytest.mark.parametrize("V,H,beam,n_sent,prepared", [(5000, 32, 5, 3, False), (50000, 64, 12, 16, True),
                                                      (8193, 16, 31, 2, False), (70001, 24, 7, 4, True)])
def test_beam_on_logits_equals_beam_on_probabilities(ctx, V, H, beam, n_sent, prepared):
    """ZR_SOFTMAX_LOGITS + zr_beam_expand_logits / zr_beam_finish_logits, and ZR_SOFTMAX_LOGITS_BLOCKS +
    zr_beam_expand_blocks / zr_beam_finish_blocks (one selection launch on the product's per-block pairs, which must hold
    the block maxima), against ZR_SOFTMAX_PROB + zr_beam_expand / zr_beam_finish on the same activations: the logits are the same bits, the column statistics are the column's maximum
    and its sum of exp(x - max), and every word, back-pointer, beam score and finished hypothesis is identical, scores
    to the bit (the selected entries are normalised with the expression the full matrix is normalised with).  <EOF> is
    made likely so that hypotheses finish inside the steps."""
    g = synth.rng(47, V + beam)
    cols, steps, max_len = n_sent * beam, 5, 10
    D = np.asfortranarray(g.uniform(-1, 1, size=(V, H)).astype(np.float32))
    bd = g.uniform(-1, 1, size=V).astype(np.float32)
    bd[1] += 3.0
    dD, dbd = ctx.array(D), ctx.array(bd)
    if prepared:
        ctx.softmax_prepare(dD, V, H)
    d_prob, d_scr = ctx.empty((V, cols)), ctx.empty((V, cols))
    d_lg = ctx.empty((V * cols + 2 * cols,))
    d_stats = d_lg.at(V * cols)
    ba, bb = ctx.beam_create(beam, V, n_sent, max_len, 0.1), ctx.beam_create(beam, V, n_sent, max_len, 0.1)
    bc = ctx.beam_create(beam, V, n_sent, max_len, 0.1)
    wa, ka = ctx.empty(cols, np.int32), ctx.empty(cols, np.int32)
    wb, kb = ctx.empty(cols, np.int32), ctx.empty(cols, np.int32)
    wc, kc = ctx.empty(cols, np.int32), ctx.empty(cols, np.int32)
    off, nblk = capi.softmax_blocks_offset(V, cols), capi.softmax_block_count(V)
    assert nblk == (V + 31) // 32 and off >= V * cols and off % 4 == 0
    d_lb = ctx.empty((off + 2 * nblk * cols,))
    d_blocks = d_lb.at(off)
    for index in range(steps + 1):
        h = np.asfortranarray(g.uniform(-1, 1, size=(H, cols)).astype(np.float32))
        dh = ctx.array(h)
        ctx.softmax_forward(dD, dbd, V, H, dh, cols, capi.ZR_SOFTMAX_PROB, d_prob, d_scr)
        ctx.softmax_forward(dD, dbd, V, H, dh, cols, capi.ZR_SOFTMAX_LOGITS, d_lg)
        ctx.softmax_forward(dD, dbd, V, H, dh, cols, capi.ZR_SOFTMAX_LOGITS_BLOCKS, d_lb)
        ctx.sync()
        out = d_lg.get()
        lg, stats = out[:V * cols].reshape((V, cols), order="F"), out[V * cols:].reshape(cols, 2)
        assert np.array_equal(lg, d_scr.get())
        outb = d_lb.get()
        assert np.array_equal(outb[:V * cols], out[:V * cols])
        pairs = outb[off:].reshape(cols, nblk, 2)
        pad = np.full((nblk * 32, cols), -np.inf, np.float32)
        pad[:V] = lg
        assert np.array_equal(pairs[:, :, 0], pad.reshape(nblk, 32, cols).max(axis=1).T)  # the block maxima
        assert np.array_equal(stats[:, 0], lg.max(axis=0))
        want_sum = np.exp(lg.astype(np.float64) - lg.max(axis=0).astype(np.float64)).sum(axis=0)
        assert np.allclose(stats[:, 1], want_sum, rtol=2e-6, atol=0)
        if index == steps:
            ctx.beam_finish(ba, d_prob)
            ctx.beam_finish_logits(bb, d_lg, d_stats)
            ctx.beam_finish_blocks(bc, d_lb, d_blocks)
            break
        ctx.beam_expand(ba, d_prob, index, wa, ka)
        ctx.beam_expand_logits(bb, d_lg, d_stats, index, wb, kb)
        ctx.beam_expand_blocks(bc, d_lb, d_blocks, index, wc, kc)
        ctx.sync()
        assert np.array_equal(wa.get(), wb.get()) and np.array_equal(wa.get(), wc.get()), index
        assert np.array_equal(ka.get(), kb.get()) and np.array_equal(ka.get(), kc.get()), index
        for s in range(n_sent):
            sa, xa = ctx.beam_state(ba, s, beam)
            sb, xb = ctx.beam_state(bb, s, beam)
            sc, xc = ctx.beam_state(bc, s, beam)
            assert np.array_equal(xa, xb) and np.array_equal(sa[xa != -1], sb[xb != -1]), (index, s)
            assert np.array_equal(xa, xc) and np.array_equal(sa[xa != -1], sc[xc != -1]), (index, s)
    ctx.sync()
    finished = 0
    for s in range(n_sent):
        ga, na = ctx.beam_hypotheses(ba, s, cap=256, max_len=max_len)
        gb, nb = ctx.beam_hypotheses(bb, s, cap=256, max_len=max_len)
        gc, nc = ctx.beam_hypotheses(bc, s, cap=256, max_len=max_len)
        assert na == nb and na == nc and na >= 1
        for (w1, s1), (w2, s2), (w3, s3) in zip(ga, gb, gc):
            assert np.array_equal(w1, w2) and s1 == s2 and np.array_equal(w1, w3) and s1 == s3
        finished += na
    assert finished > n_sent * beam  # some hypotheses finished inside the steps, not only at the forced end
    with pytest.raises(capi.ZrError):
        ctx.softmax_forward(dD, dbd, V, H, dh, cols, capi.ZR_SOFTMAX_LOGITS, d_lg, d_scr)
    if prepared:
        ctx.softmax_release(dD)
    ctx.beam_destroy(ba)
    ctx.beam_destroy(bb)
    ctx.beam_destroy(bc)


@pytest.mark.parametrize("K,V,cols", [(1, 37, 3), (2, 400, 12), (5, 50000, 192), (8, 1025, 1)])
def test_ensemble_average_is_the_renormalised_mean(ctx, K, V, cols):
    """zr_ensemble_average: out(:, c) = mean_k p_k(:, c) divided by its own sum (src/ensemble_factory.hpp:767-793,
    which sums the models' distributions in double, divides by their number and renormalises each column).  The
    models' columns here deliberately do not sum to one (scaled by 0.5 .. 1.5), so a kernel that skipped the
    renormalisation, or divided by a constant, fails; one column holds zeros in all models but one."""
    g = synth.rng(77, K + cols)
    ps = [np.asfortranarray(_random_dist(g, V, cols) * g.uniform(0.5, 1.5, size=(1, cols)).astype(np.float32))
          for _ in range(K)]
    if K > 1:
        for p in ps[1:]:
            p[:, 0] = 0.0
    avg = (np.sum([p.astype(np.float64) for p in ps], axis=0) / K)
    want = avg / avg.sum(axis=0)
    d_ps = [ctx.array(p) for p in ps]
    d_out = ctx.empty((V, cols))
    ctx.ensemble_average(d_ps, V, cols, d_out)
    got = d_out.get()
    np.testing.assert_allclose(got, want, rtol=3e-6, atol=1e-12)
    np.testing.assert_allclose(got.astype(np.float64).sum(axis=0), 1.0, rtol=1e-5)
    if K == 1:
        # one model: the result is that model's distribution, renormalised; in place is allowed
        ctx.ensemble_average(d_ps, V, cols, d_ps[0])
        np.testing.assert_array_equal(d_ps[0].get(), got)
    with pytest.raises(capi.ZrError):
        ctx.ensemble_average(d_ps * 17, V, cols, d_out)
    for d in d_ps + [d_out]:
        d.free()


def test_ensemble_alignment_vote_known_answer_and_brute_force(ctx):
    """zr_attn_viterbi_ensemble (src/ensemble_factory.hpp:797-834).  A hand-worked case first: model A puts 0.4375,
    0.375, 0.1875 on source positions 2, 3, 4 (its own best: 2), model B 0.375, 0.1875, 0.4375 on positions 3, 4, 5 (its
    own best: 5); the sums are 0.4375, 0.75, 0.375, 0.4375, so the vote is position 3, which neither model picks alone.
    A second column ties exactly (0.625 at positions 3 and 5): the first wins.  A third has no source position at all
    (-1).  Then random windows against the restatement in test_gpu_decode.ensemble_alignment_vote."""
    from test_gpu_decode import ensemble_alignment_vote
    f, i = np.float32, np.int32
    alA = np.asfortranarray(np.array([[0.4375, 0.375, 0.1875], [0.25, 0.5, 0.25], [0.3, 0.3, 0.4]], f))
    ixA = np.asfortranarray(np.array([[2, 3, 4], [2, 3, 4], [-1, -1, -1]], i))
    alB = np.asfortranarray(np.array([[0.375, 0.1875, 0.4375], [0.125, 0.25, 0.625], [0.5, 0.2, 0.3]], f))
    ixB = np.asfortranarray(np.array([[3, 4, 5], [3, 4, 5], [-1, -1, -1]], i))
    d = [ctx.array(x) for x in (alA, alB)], [ctx.array(x) for x in (ixA, ixB)]
    d_out = ctx.empty(3, np.int32)
    ctx.attn_viterbi_ensemble(d[0], d[1], 3, 3, 9, d_out)
    assert d_out.get().tolist() == [3, 3, -1]
    assert ensemble_alignment_vote([alA, alB], [ixA, ixB], 9).tolist() == [3, 3, -1]
    g = synth.rng(78, 5)
    for K, D, cols, longest in [(1, 2, 7, 12), (3, 10, 192, 54), (8, 50, 24, 104), (16, 3, 5, 700)]:
        W = 2 * D + 1
        als, ixs = [], []
        centre = g.integers(0, longest, size=cols)
        for k in range(K):
            c = np.clip(centre + g.integers(-2, 3, size=cols), 0, longest - 1)
            ix = c[:, None] + np.arange(-D, D + 1)[None, :]
            ix = np.where((ix < 0) | (ix >= longest - 4), -1, ix).astype(i)
            al = g.uniform(0.0, 1.0, size=(cols, W)).astype(f)
            al[ix == -1] = 0.0
            al /= np.maximum(al.sum(axis=1, keepdims=True), 1e-9)
            als.append(np.asfortranarray(al.astype(f)))
            ixs.append(np.asfortranarray(ix))
        d_al, d_ix = [ctx.array(x) for x in als], [ctx.array(x) for x in ixs]
        d_o = ctx.empty(cols, np.int32)
        ctx.attn_viterbi_ensemble(d_al, d_ix, W, cols, longest, d_o)
        want = ensemble_alignment_vote(als, ixs, longest)
        assert np.array_equal(d_o.get(), want), (K, D, cols, longest)
        if K > 1:
            own = ensemble_alignment_vote(als[:1], ixs[:1], longest)
            assert np.any(own != want), "the vote equals the first model's choice everywhere"
        for x in d_al + d_ix + [d_o]:
            x.free()
    with pytest.raises(capi.ZrError):
        ctx.attn_viterbi_ensemble(d[0], d[1], 3, 3, 9000, d_out)
    for x in d[0] + d[1] + [d_out]:
        x.free()


@pytest.mark.parametrize("V,beam,n_sent", [(50000, 12, 1), (8193, 12, 2), (40, 5, 1), (50017, 30, 1)])
def test_beam_on_blocks_with_hostile_columns(ctx, V, beam, n_sent):
    """zr_beam_expand_blocks against zr_beam_expand_logits and zr_beam_expand on logits built to stress the selection on
    block maxima: a constant column (every block reaches the bound: the exact K-pass path), thousands of copies of the
    largest value (candidate list overflows), copies of the K-th largest value spread over hundreds of blocks, the K
    largest in one block, one per block, a column of very negative numbers, the three-words-one-probability case, a last
    block of one row, a vocabulary of two blocks.  The logits are produced by the output product itself from a matrix
    that holds them and one-hot activations (exact), so the three paths see the same bits."""
    g = synth.rng(49, V + beam)
    cols, K = beam * n_sent, beam + 1
    lg = np.asfortranarray(g.uniform(-3, -2, size=(V, cols)).astype(np.float32))

    def col(i):
        return i % cols

    lg[:, col(0)] = 0.5                                                  # constant column
    many = g.choice(V, size=min(3000, V // 2), replace=False)
    lg[many, col(1)] = 1.0                                               # thousands of copies of the maximum
    top = np.float32(0.2)
    b1 = np.nextafter(top, np.float32(-1))
    b2 = np.nextafter(b1, np.float32(-1))
    lg[V - 1, col(2)], lg[3, col(2)], lg[V // 2, col(2)] = top, b1, b2   # one probability, three logits
    if V >= 64 * K:
        lg[32 * 7:32 * 7 + K, col(3)] = np.linspace(2.0, 1.0, K, dtype=np.float32)      # the K largest in one block
        lg[np.arange(K + 20) * 32 + 5, col(4)] = np.linspace(3.0, 1.0, K + 20, dtype=np.float32)  # one per block
        idx = g.choice(V, size=min(700 * 32, V) // 32, replace=False)
        lg[idx[:K - 1], col(6)] = 4.0 + np.arange(K - 1, dtype=np.float32)
        lg[idx[K - 1:], col(6)] = 1.5                                     # the K-th largest, hundreds of times
    lg[:, col(5)] = -1e30
    lg[[2 % V, (V - 1)], col(5)] = [-5.0, -6.0]
    H = cols
    dD, dbd = ctx.array(lg), ctx.array(np.zeros(V, np.float32))
    dh = ctx.array(np.asfortranarray(np.eye(H, dtype=np.float32)))
    off, nblk = capi.softmax_blocks_offset(V, cols), capi.softmax_block_count(V)
    d_prob, d_lg, d_lb = ctx.empty((V, cols)), ctx.empty((V * cols + 2 * cols,)), ctx.empty((off + 2 * nblk * cols,))
    ctx.softmax_forward(dD, dbd, V, H, dh, cols, capi.ZR_SOFTMAX_PROB, d_prob)
    ctx.softmax_forward(dD, dbd, V, H, dh, cols, capi.ZR_SOFTMAX_LOGITS, d_lg)
    ctx.softmax_forward(dD, dbd, V, H, dh, cols, capi.ZR_SOFTMAX_LOGITS_BLOCKS, d_lb)
    ctx.sync()
    assert np.array_equal(d_lg.get()[:V * cols].reshape((V, cols), order="F"), lg)  # the product reproduced the logits
    beams = [ctx.beam_create(beam, V, n_sent, 8, 0.0) for _ in range(3)]
    outs = [(ctx.empty(cols, np.int32), ctx.empty(cols, np.int32)) for _ in range(3)]
    for index in range(2):
        ctx.beam_expand(beams[0], d_prob, index, *outs[0])
        ctx.beam_expand_logits(beams[1], d_lg, d_lg.at(V * cols), index, *outs[1])
        ctx.beam_expand_blocks(beams[2], d_lb, d_lb.at(off), index, *outs[2])
        ctx.sync()
        for k in (1, 2):
            assert np.array_equal(outs[0][0].get(), outs[k][0].get()), (index, k)
            assert np.array_equal(outs[0][1].get(), outs[k][1].get()), (index, k)
            for s_ in range(n_sent):
                sa, xa = ctx.beam_state(beams[0], s_, beam)
                sk, xk = ctx.beam_state(beams[k], s_, beam)
                assert np.array_equal(xa, xk) and np.array_equal(sa[xa != -1], sk[xk != -1]), (index, k, s_)
    for b in beams:
        ctx.beam_destroy(b)


def test_beam_on_logits_ranks_words_of_equal_probability_as_the_probability_matrix_would(ctx):
    """Three words whose logits differ by one and two ulp but whose probabilities, exp(x - max) / sum, round to the same
    float.  The reference only ever sees probabilities and ranks such words by its rule for equal values (here: lower
    word id first); selection on the logits must do the same -- ranking them by logit would put the highest id first.
    Checked against the expansion of a probability matrix that holds the three equal values."""
    V, beam, n_sent = 5000, 3, 1
    cols = beam * n_sent
    g = synth.rng(48, 1)
    lg = np.asfortranarray(g.uniform(-3, -2, size=(V, cols)).astype(np.float32))
    top = np.float32(0.2)
    below1 = np.nextafter(top, np.float32(-1))
    below2 = np.nextafter(below1, np.float32(-1))
    assert top > below1 > below2
    lg[4000, 0], lg[10, 0], lg[700, 0] = top, below1, below2
    mx = lg.max(axis=0)
    sums = np.exp(lg.astype(np.float64) - mx.astype(np.float64)).sum(axis=0).astype(np.float32)
    prob = np.asfortranarray((np.exp((lg - mx).astype(np.float32)) / sums).astype(np.float32))
    assert prob[4000, 0] == prob[10, 0] == prob[700, 0]  # (exp of minus one or two ulp of 0.2 is 1 in fp32)
    flat = np.concatenate([lg.reshape(-1, order="F"), np.stack([mx, sums], axis=1).reshape(-1)]).astype(np.float32)
    d_lg = ctx.array(flat)
    d_stats = d_lg.at(V * cols)
    d_prob = ctx.array(prob)
    ba, bb = ctx.beam_create(beam, V, n_sent, 8, 0.0), ctx.beam_create(beam, V, n_sent, 8, 0.0)
    wa, ka = ctx.empty(cols, np.int32), ctx.empty(cols, np.int32)
    wb, kb = ctx.empty(cols, np.int32), ctx.empty(cols, np.int32)
    ctx.beam_expand(ba, d_prob, 0, wa, ka)
    ctx.beam_expand_logits(bb, d_lg, d_stats, 0, wb, kb)
    ctx.sync()
    assert wa.get().tolist() == [10, 700, 4000]
    assert wb.get().tolist() == [10, 700, 4000]
    sa, _ = ctx.beam_state(ba, 0, beam)
    sb, _ = ctx.beam_state(bb, 0, beam)
    assert sa[0] == sa[1] == sa[2] and np.array_equal(sa, sb)
    ctx.beam_destroy(ba)
    ctx.beam_destroy(bb)
