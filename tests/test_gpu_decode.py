"""End-to-end beam decode (benchmark configuration 4 wiring at sizes the oracle finishes in seconds): encoder, then per step
embedding gather -> LSTM stack with feed-input -> attention -> softmax -> device-side beam -> state reorder, for
several sentences side by side, against one oracle decode per sentence (the reference decodes one sentence per
pass).  Selected words and back-pointers must be identical at every step, hypotheses identical at the end."""
import numpy as np
import pytest

import oracle_lib as o
from zoph_rnn_amd import capi, driver, synth

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def ctx():
    c = capi.Context(0)
    yield c
    c.close()


def _model(g, H, Vs, Vt, L):
    m = {"src_embed": synth.uniform(g, (H, Vs), -0.5, 0.5), "tgt_embed": synth.uniform(g, (H, Vt), -0.5, 0.5),
         "src_layers": [synth.lstm_layer(g, H, forget_bias_one=True) for _ in range(L)],
         "tgt_layers": [synth.lstm_layer(g, H, feed_input=(l == 0), forget_bias_one=True) for l in range(L)],
         "attn": synth.attention_weights(g, H),
         # a peaked output distribution keeps candidate scores well separated (no near-ties for fp32 noise to flip)
         "D_soft": synth.uniform(g, (Vt, H), -3.0, 3.0), "b_soft": synth.uniform(g, (Vt,), -1.0, 1.0)}
    for ly in m["src_layers"] + m["tgt_layers"]:
        for k in ("M", "Wh"):
            ly[k] = [synth.uniform(g, (H, H), -0.3, 0.3) for _ in range(4)]
    for k in ("W_a", "W_p", "W_c1", "W_c2"):
        m["attn"][k] = synth.uniform(g, (H, H), -0.3, 0.3)
    return m


def _oracle_decode(m, src_col, src_len, S, beam, steps, D, penalty, viterbi=False, safe_out=None):
    """One sentence, minibatch = beam, following forward_prop_source / forward_prop_target / swap_decoding_states.
    viterbi: the attention layer's Viterbi alignments ride along (unk replacement); a fourth value, the alignments
    of every finished hypothesis, is returned.
    safe_out (a list): instead of failing when a step's p_t lies within 1e-4 of an integer (where fp32 rounding may
    legitimately move the attention window) or two candidate scores a step pops lie within 5e-6 of each other (where it
    (or, later in a long decode, within 1e-6 of their size) of each other (where it may swap them), the index of the
    first such step is appended (steps + 1 if there is none; the forced finish counts
    as step `steps`): a comparison is meaningful for the steps before it."""
    H, L, Vt = m["src_embed"].shape[0], len(m["src_layers"]), m["D_soft"].shape[0]
    nn, mk = o.vocab_prep(src_col.reshape(S, 1))
    hs, cs = o.lstm_stack_forward(m["src_embed"], m["src_layers"], nn, mk)
    table = np.repeat(hs[L - 1], beam, axis=2)  # (S, H, beam)
    hp = [np.repeat(np.asfortranarray(hs[l, S - 1]), beam, axis=1) for l in range(L)]
    cp = [np.repeat(np.asfortranarray(cs[l, S - 1]), beam, axis=1) for l in range(L)]
    binfo = np.concatenate([np.full(beam, src_len, np.int32), np.full(beam, S - src_len, np.int32)])
    ones = np.ones(beam, np.int32)
    dec = o.Decoder(beam, Vt, steps + 3, penalty=penalty)
    words = np.zeros(beam, np.int32)
    h_tild = None
    hist, min_gap = [], np.inf
    first_unsafe = steps + 1

    def forward(index):
        nonlocal hp, cp, h_tild
        below = o.embed_gather(m["tgt_embed"], np.maximum(words, 0))
        newh, newc = [], []
        for l in range(L):
            ly = m["tgt_layers"][l]
            feed = l == 0 and index > 0
            r = o.lstm_step(ly["M"], ly["Wh"], ly["b"], below, hp[l], cp[l], ones, Q=ly["Q"] if feed else None,
                            htild=h_tild if feed else None)
            newh.append(r["h"])
            newc.append(r["c"])
            below = r["h"]
        att = o.attention_forward(hs_table=table, batch_info=binfo, h_t=below, mask01=ones, D=D, **m["attn"])
        P = o.softmax_dist(o.softmax_logits(m["D_soft"], m["b_soft"], att["h_tild"]))
        return newh, newc, att, P

    for index in range(steps):
        newh, newc, att, P = forward(index)
        # how close the closest pair of candidate scores is among those the step can pop (the test is only meaningful
        # without near-ties there; further down the list the order of candidates has no effect on anything)
        cols = 1 if index == 0 else beam
        sc = dec.state()["scores"]
        cand = np.sort(np.concatenate([np.log(np.sort(P[:, i])[-(beam + 2):]) + sc[i] for i in range(cols)]))[::-1]
        n_hyp_before = len(dec.hypotheses())
        frac = att["p_t"] - np.floor(att["p_t"])
        if not np.all((frac > 1e-4) & (frac < 1 - 1e-4)):
            assert safe_out is not None, "p_t on an integer boundary; pick another seed"
            first_unsafe = min(first_unsafe, index)
        dec.expand(P, index, _single_model_vote(att, S) if viterbi else None)
        popped = beam + (len(dec.hypotheses()) - n_hyp_before) + 2  # survivors + <EOF> hypotheses (+ a <START>) + next
        step_gap = np.min(-np.diff(cand[:popped + 1]))
        min_gap = min(min_gap, step_gap)
        # a near-tie: either order is right to fp32 accuracy.  A score is a sum of one log-probability per step: each
        # term carries the fp32 rounding of a 1000-term logit (about 2e-5 at logits of 15; the oracle accumulates in
        # double), so two runs' scores drift apart like 2e-5 * sqrt(steps), and the sum itself is held in fp32 (as in
        # the reference), 1e-6 of its size being 4 to 8 ulp
        if safe_out is not None and step_gap <= max(5e-6, 1e-6 * float(np.abs(cand[:popped + 1]).max()),
                                                    4e-5 * np.sqrt(index + 1.0)):
            first_unsafe = min(first_unsafe, index)
        st = dec.state()
        words, back = st["current_indices"].copy(), st["new_indicies_changes"].copy()
        hist.append((words.copy(), back.copy()))
        hp = [np.asfortranarray(a[:, back]) for a in newh]
        cp = [np.asfortranarray(a[:, back]) for a in newc]
        h_tild = np.asfortranarray(att["h_tild"][:, back])
    _, _, att, P = forward(steps)
    frac = att["p_t"] - np.floor(att["p_t"])
    if safe_out is not None:
        if not np.all((frac > 1e-4) & (frac < 1 - 1e-4)):
            first_unsafe = min(first_unsafe, steps)
        safe_out.append(first_unsafe)
    dec.finish(P, _single_model_vote(att, S) if viterbi else None)
    if viterbi:
        return hist, dec.hypotheses(), min_gap, dec.hypotheses_viterbi()
    return hist, dec.hypotheses(), min_gap


def _oracle_score_of_path(m, src_col, src_len, S, D, words):
    """The log-probability of one target word sequence (<START> ... <EOF>) under the model, teacher-forced through the
    oracle one column wide: what the beam reports as that hypothesis' score whatever else was in the beam."""
    L = len(m["src_layers"])
    nn, mk = o.vocab_prep(src_col.reshape(S, 1))
    hs, cs = o.lstm_stack_forward(m["src_embed"], m["src_layers"], nn, mk)
    table = hs[L - 1]  # (S, H, 1)
    hp = [np.asfortranarray(hs[l, S - 1]) for l in range(L)]
    cp = [np.asfortranarray(cs[l, S - 1]) for l in range(L)]
    binfo = np.array([src_len, S - src_len], np.int32)
    ones = np.ones(1, np.int32)
    h_tild, score = None, np.float32(0)
    for t in range(len(words) - 1):
        below = o.embed_gather(m["tgt_embed"], np.array([words[t]], np.int32))
        for l in range(L):
            ly = m["tgt_layers"][l]
            feed = l == 0 and t > 0
            r = o.lstm_step(ly["M"], ly["Wh"], ly["b"], below, hp[l], cp[l], ones, Q=ly["Q"] if feed else None,
                            htild=h_tild if feed else None)
            hp[l], cp[l], below = r["h"], r["c"], r["h"]
        att = o.attention_forward(hs_table=table, batch_info=binfo, h_t=below, mask01=ones, D=D, **m["attn"])
        h_tild = att["h_tild"]
        P = o.softmax_dist(o.softmax_logits(m["D_soft"], m["b_soft"], h_tild))
        score = np.float32(score + np.float32(np.log(P[words[t + 1], 0])))
    return float(score)


def _single_model_vote(att, S):
    """The alignment the reference's driver hands its decoder: also for one model it is the vote of
    ensemble_factory::ensembles_models (src/ensemble_factory.hpp:797-834), which overwrites the attention layer's own
    Viterbi alignment -- the two differ where no weight of a column's window is positive (-1 instead of the first
    slot's position)."""
    return ensemble_alignment_vote([att["alignments"]], [att["indices"]], S + 4)


def ensemble_alignment_vote(aligns, indices, longest):
    """The ensemble's alignment per column (src/ensemble_factory.hpp:797-834): every model's window weights spread over
    a row of `longest` source positions (zero elsewhere, src/attention_node.hpp:236-268), the rows added in model order
    in float32, then the first position whose sum exceeds every earlier one, starting from 0 (-1 if none is positive).
    aligns, indices: per model a (columns, 2D+1) array."""
    cols, W = aligns[0].shape
    out = np.empty(cols, np.int32)
    for b in range(cols):
        total = np.zeros(longest, np.float32)
        for al, ix in zip(aligns, indices):
            row = np.zeros(longest, np.float32)
            for j in range(W):
                if ix[b, j] != -1:
                    row[ix[b, j]] = al[b, j]
            total = (total + row).astype(np.float32)
        best, pos = np.float32(0), -1
        for j in range(longest):
            if total[j] > best:
                best, pos = total[j], j
        out[b] = pos
    return out


def _oracle_ensemble_decode(ms, src_cols, S, beam, steps, D, viterbi=False):
    """One sentence through several models behind one beam (src/ensemble_factory.hpp:767-793): every model runs its
    own encoder and decoder step, the step's output distributions are averaged (sum in double, divided by the number of
    models) and each column divided by its sum, the one beam expands on that, and every model's states follow the
    same back-pointers.  Returns the finished hypotheses and the smallest gap between candidate scores a step popped.
    viterbi: the beam carries the models' alignment vote; returns in addition the finished hypotheses' alignments and
    how many (step, column) pairs had a vote different from the first model's own alignment."""
    K, Vt = len(ms), ms[0]["D_soft"].shape[0]
    vote_differs = 0

    def vote(outs):
        nonlocal vote_differs
        if not viterbi:
            return None
        v = ensemble_alignment_vote([r[2]["alignments"] for r in outs], [r[2]["indices"] for r in outs], S + 4)
        vote_differs += int(np.sum(v != o.attention_viterbi(outs[0][2]["alignments"], outs[0][2]["indices"])))
        return v

    L = len(ms[0]["src_layers"])
    ones = np.ones(beam, np.int32)
    binfo = np.concatenate([np.full(beam, S, np.int32), np.zeros(beam, np.int32)])
    st = []
    for m, col in zip(ms, src_cols):
        nn, mk = o.vocab_prep(col.reshape(S, 1))
        hs, cs = o.lstm_stack_forward(m["src_embed"], m["src_layers"], nn, mk)
        st.append({"table": np.repeat(hs[L - 1], beam, axis=2),
                   "hp": [np.repeat(np.asfortranarray(hs[l, S - 1]), beam, axis=1) for l in range(L)],
                   "cp": [np.repeat(np.asfortranarray(cs[l, S - 1]), beam, axis=1) for l in range(L)], "h_tild": None})
    dec = o.Decoder(beam, Vt, steps + 3, penalty=0.0)
    words = np.zeros(beam, np.int32)
    min_gap = np.inf

    def forward(k, index):
        m, s = ms[k], st[k]
        below = o.embed_gather(m["tgt_embed"], np.maximum(words, 0))
        newh, newc = [], []
        for l in range(L):
            ly = m["tgt_layers"][l]
            feed = l == 0 and index > 0
            r = o.lstm_step(ly["M"], ly["Wh"], ly["b"], below, s["hp"][l], s["cp"][l], ones,
                            Q=ly["Q"] if feed else None, htild=s["h_tild"] if feed else None)
            newh.append(r["h"])
            newc.append(r["c"])
            below = r["h"]
        att = o.attention_forward(hs_table=s["table"], batch_info=binfo, h_t=below, mask01=ones, D=D, **m["attn"])
        P = o.softmax_dist(o.softmax_logits(m["D_soft"], m["b_soft"], att["h_tild"]))
        return newh, newc, att, P

    def mean_dist(outs):
        avg = (np.sum([r[3].astype(np.float64) for r in outs], axis=0) / K).astype(np.float32)
        norm = avg.astype(np.float64).sum(axis=0).astype(np.float32)
        return np.asfortranarray((avg / norm[None, :]).astype(np.float32))

    for index in range(steps):
        outs = [forward(k, index) for k in range(K)]
        P = mean_dist(outs)
        cols = 1 if index == 0 else beam
        sc = dec.state()["scores"]
        cand = np.sort(np.concatenate([np.log(np.sort(P[:, i])[-(beam + 2):]) + sc[i] for i in range(cols)]))[::-1]
        n_hyp_before = len(dec.hypotheses())
        dec.expand(P, index, vote(outs))
        popped = beam + (len(dec.hypotheses()) - n_hyp_before) + 2
        min_gap = min(min_gap, np.min(-np.diff(cand[:popped + 1])))
        d = dec.state()
        words, back = d["current_indices"].copy(), d["new_indicies_changes"].copy()
        for k in range(K):
            newh, newc, att, _ = outs[k]
            st[k]["hp"] = [np.asfortranarray(a[:, back]) for a in newh]
            st[k]["cp"] = [np.asfortranarray(a[:, back]) for a in newc]
            st[k]["h_tild"] = np.asfortranarray(att["h_tild"][:, back])
    outs = [forward(k, steps) for k in range(K)]
    dec.finish(mean_dist(outs), vote(outs))
    if viterbi:
        return dec.hypotheses(), min_gap, dec.hypotheses_viterbi(), vote_differs
    return dec.hypotheses(), min_gap


@pytest.mark.parametrize("H,L,beam,n_sent,S,steps,D", [(64, 2, 4, 3, 7, 6, 3), (48, 1, 3, 2, 5, 5, 10), (100, 3, 12, 2, 9, 4, 10)])
def test_batched_beam_decode_matches_per_sentence_reference(ctx, H, L, beam, n_sent, S, steps, D):
    g = synth.rng(61, H + beam)
    Vs, Vt = 80, 400
    m = _model(g, H, Vs, Vt, L)
    lens = g.integers(max(2, S - 3), S + 1, size=n_sent).astype(np.int32)
    lens[0] = S
    src = g.integers(0, Vs, size=(S, n_sent)).astype(np.int32)
    for s in range(n_sent):
        src[:S - lens[s], s] = -1
    w = driver.Seq2SeqWeights(ctx, m["src_embed"], m["src_layers"], m["tgt_embed"], m["tgt_layers"], m["attn"],
                              m["D_soft"], m["b_soft"])
    dec = driver.BeamDecode(ctx, w, beam, n_sent, S, steps, attention_D=D, penalty=0.0)
    dec.encode(src, lens)
    for _ in range(steps):
        dec.step(record=True)
    dec.finish()
    for s in range(n_sent):
        hist, hyps, gap = _oracle_decode(m, src[:, s], int(lens[s]), S, beam, steps, D, 0.0)
        assert gap > 5e-6, "candidate scores nearly tie (gap %.2e): pick another seed" % gap
        for index in range(steps):
            gw, gb = dec.history[index]
            assert np.array_equal(gw[s * beam:(s + 1) * beam], hist[index][0]), (s, index)
            assert np.array_equal(gb[s * beam:(s + 1) * beam] - s * beam, hist[index][1]), (s, index)
        got = dec.hypotheses(s)
        assert len(got) == len(hyps)
        for (gwords, gscore), (wwords, wscore) in zip(got, hyps):
            assert np.array_equal(gwords, wwords)
            assert gscore == pytest.approx(wscore, rel=1e-4, abs=1e-4)
    dec.close()


def test_config4_beam_decode_at_full_size(ctx):
    """Benchmark configuration 4 at its real shape: 4 layers, H = 1000, beam 12 x 16 sentences = 192 live columns,
    source length 50, both vocabularies 50 000, attention window D = 50 (every source position has a slot), feed-input.
    Six decode steps and the forced finish; three of the sixteen sentences (first, middle, last: different source
    lengths) are decoded one at a time by the oracle, as the reference does, and every selected word, back-pointer
    and finished hypothesis must be identical.  LSTM and attention weights have the benchmark's U(-0.08, 0.08) range;
    the output matrix is drawn wider so that candidate scores are separated by far more than fp32 noise."""
    H, L, beam, n_sent, S, steps, D = 1000, 4, 12, 16, 50, 6, 50
    Vs = Vt = 50000
    g = synth.rng(64, 4)
    m = {"src_embed": synth.uniform(g, (H, Vs)), "tgt_embed": synth.uniform(g, (H, Vt), -0.5, 0.5),
         "src_layers": [synth.lstm_layer(g, H, forget_bias_one=True) for _ in range(L)],
         "tgt_layers": [synth.lstm_layer(g, H, feed_input=(l == 0), forget_bias_one=True) for l in range(L)],
         "attn": synth.attention_weights(g, H),
         "D_soft": synth.uniform(g, (Vt, H), -0.5, 0.5), "b_soft": synth.uniform(g, (Vt,), -1.0, 1.0)}
    lens = g.integers(S - 12, S + 1, size=n_sent).astype(np.int32)
    lens[0] = S
    src = synth.zipf_ids(g, (S, n_sent), Vs)
    for s in range(n_sent):
        src[:S - lens[s], s] = -1
    w = driver.Seq2SeqWeights(ctx, m["src_embed"], m["src_layers"], m["tgt_embed"], m["tgt_layers"], m["attn"],
                              m["D_soft"], m["b_soft"])
    dec = driver.BeamDecode(ctx, w, beam, n_sent, S, steps, attention_D=D, penalty=0.0)
    dec.encode(src, lens)
    for _ in range(steps):
        dec.step(record=True)
    dec.finish()
    checked = 0
    for s in (0, n_sent // 2, n_sent - 1):
        hist, hyps, gap = _oracle_decode(m, src[:, s], int(lens[s]), S, beam, steps, D, 0.0)
        assert gap > 5e-6, "candidate scores nearly tie (gap %.2e): pick another seed" % gap
        for index in range(steps):
            gw, gb = dec.history[index]
            assert np.array_equal(gw[s * beam:(s + 1) * beam], hist[index][0]), (s, index)
            assert np.array_equal(gb[s * beam:(s + 1) * beam] - s * beam, hist[index][1]), (s, index)
        got = dec.hypotheses(s)
        assert len(got) == len(hyps) and len(got) >= beam
        for (gwords, gscore), (wwords, wscore) in zip(got, hyps):
            assert np.array_equal(gwords, wwords)
            assert gscore == pytest.approx(wscore, rel=1e-4, abs=1e-4)
        checked += 1
    assert checked == 3
    # every sentence's words lie in the vocabulary and no beam slot died (192 live hypotheses throughout)
    for index in range(steps):
        gw, gb = dec.history[index]
        assert np.all((gw >= 2) & (gw < Vt)) and np.all((gb // beam) == np.repeat(np.arange(n_sent), beam))
    dec.close()


def test_config4_beam_decode_over_its_full_length_all_sentences(ctx):
    """Benchmark configuration 4 as stated: 4 layers, H = 1000, beam 12 x 16 sentences, source length 50, 50 000-word
    vocabularies, the reference's default attention width D = 10, decoded to the reference's stop
    min(1.5 * source length, longest_sent - 2) = 60 steps (src/ensemble_factory.hpp:637) plus the forced finish.  ALL
    sixteen sentences are decoded one at a time by the oracle and compared step by step: words, back-pointers, and at
    the end every finished hypothesis -- hypotheses that end early (the <EOF> bias is raised so that <EOF> enters the
    candidates at some steps and not at others), late ones, and the forced finish of the survivors
    (src/decoder.h:672-688).  Over 60 steps x 192 columns some step's p_t falls within fp32 rounding of an integer or
    two candidate scores nearly tie; from such a step on either continuation is right, so a sentence is compared up to
    its first such step (reported by the oracle run); enough sentences must be clean to the end."""
    H, L, beam, n_sent, S, D, longest = 1000, 4, 12, 16, 50, 10, 62
    steps = min(int(1.5 * S), longest - 2)
    assert steps == 60
    Vs = Vt = 50000
    g = synth.rng(64, 5)
    m = {"src_embed": synth.uniform(g, (H, Vs)), "tgt_embed": synth.uniform(g, (H, Vt), -0.5, 0.5),
         "src_layers": [synth.lstm_layer(g, H, forget_bias_one=True) for _ in range(L)],
         "tgt_layers": [synth.lstm_layer(g, H, feed_input=(l == 0), forget_bias_one=True) for l in range(L)],
         "attn": synth.attention_weights(g, H),
         "D_soft": synth.uniform(g, (Vt, H), -0.5, 0.5), "b_soft": synth.uniform(g, (Vt,), -1.0, 1.0)}
    m["b_soft"][1] = 10.5
    lens = g.integers(S - 12, S + 1, size=n_sent).astype(np.int32)
    lens[0] = S
    src = synth.zipf_ids(g, (S, n_sent), Vs)
    for s in range(n_sent):
        src[:S - lens[s], s] = -1
    w = driver.Seq2SeqWeights(ctx, m["src_embed"], m["src_layers"], m["tgt_embed"], m["tgt_layers"], m["attn"],
                              m["D_soft"], m["b_soft"])
    dec = driver.BeamDecode(ctx, w, beam, n_sent, S, steps, attention_D=D, penalty=0.0)
    dec.encode(src, lens)
    for _ in range(steps):
        dec.step(record=True)
    dec.finish()
    early, late, forced, compared, rescored = 0, 0, 0, 0, 0
    for s in range(n_sent):
        safe = []
        hist, hyps, _ = _oracle_decode(m, src[:, s], int(lens[s]), S, beam, steps, D, 0.0, safe_out=safe)
        upto = min(safe[0], steps)
        compared += upto
        for index in range(upto):
            gw, gb = dec.history[index]
            assert np.array_equal(gw[s * beam:(s + 1) * beam], hist[index][0]), (s, index)
            assert np.array_equal(gb[s * beam:(s + 1) * beam] - s * beam, hist[index][1]), (s, index)
        got = dec.hypotheses(s, cap=4 * beam * (steps + 2))
        # the hypotheses that finished before the first doubtful step are the oracle's, in its order
        want = [(ww, ws) for ww, ws in hyps if len(ww) - 2 < upto]
        have = [(gw_, gs) for gw_, gs in got if len(gw_) - 2 < upto]
        assert len(have) == len(want)
        for (gwords, gscore), (wwords, wscore) in zip(have, want):
            assert np.array_equal(gwords, wwords)
            assert gscore == pytest.approx(wscore, rel=1e-4, abs=2e-4)
        # whole length: words in range, <START> first and <EOF> last and nowhere else, the forced finish has produced one
        # hypothesis per surviving slot
        n_words = [len(gw_) for gw_, _ in got]
        assert sum(1 for n in n_words if n == steps + 2) == beam
        for gw_, _ in got:
            assert gw_[0] == 0 and gw_[-1] == 1 and np.all((gw_[1:-1] >= 2) & (gw_[1:-1] < Vt))
        early += sum(1 for n in n_words if n <= 12)
        late += sum(1 for n in n_words if 25 <= n < steps + 2)
        forced += sum(1 for n in n_words if n == steps + 2)
        picks = {0, len(got) - 1}
        picks.update([i for i, n in enumerate(n_words) if 25 <= n < steps + 2][:1])
        for i in sorted(picks):
            gw_, gs = got[i]
            ws = _oracle_score_of_path(m, src[:, s], int(lens[s]), S, D, gw_)
            assert gs == pytest.approx(ws, rel=2e-5, abs=2e-3), (s, i, len(gw_), gs, ws)
            rescored += 1
    for index in range(steps):
        gw, gb = dec.history[index]
        assert np.all((gw >= 2) & (gw < Vt)) and np.all((gb // beam) == np.repeat(np.arange(n_sent), beam))
    dec.close()
    # (with this seed 323 of the 960 steps are comparable one by one)
    assert compared >= 250, "only %d of %d steps were comparable" % (compared, n_sent * steps)
    assert early >= 1 and late >= 1 and forced == n_sent * beam and rescored >= 2 * n_sent, (early, late, forced, rescored)
