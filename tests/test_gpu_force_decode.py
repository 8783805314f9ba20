"""The force-decode / perplexity driver (zoph_rnn_amd/host/force_decode) end to end: a complete model file (header,
vocabulary blocks, matrices in the reference's order) and raw text in, one log-probability per minibatch out, checked
against the oracle run on the Python-integerized data.  Covers the header / vocabulary parsing, integerization,
the minibatch reader's time-major layout and batch_info, the short last minibatch, and the getError schedule."""
import numpy as np
import pytest

import model_files_util as mf
import oracle_lib as o
from test_gpu_host_layers import _write_hh, _write_ih, _write_matrix
from zoph_rnn_amd import synth

pytestmark = pytest.mark.gpu


def _time_major(rows, mb):
    """rows: list of equal-length int lists (one per sentence) -> (T, mb) array padded with -1 columns."""
    T = len(rows[0])
    a = np.full((T, mb), -1, np.int32)
    for b, r in enumerate(rows):
        a[:, b] = r
    return a


def _oracle_seq2seq(m, chunk, mb, D, longest):
    """Natural-log probability of one minibatch (list of [src, minus_two, tgt_in, tgt_out])."""
    L, H = len(m["src_layers"]), m["emb_s"].shape[0]
    src, tin, tout = (_time_major([c[k] for c in chunk], mb) for k in (0, 2, 3))
    S, T = src.shape[0], tin.shape[0]
    lens = np.array([(src[:, b] != -1).sum() if b < len(chunk) else 1 for b in range(mb)], np.int32)
    binfo = np.concatenate([lens, S - lens]).astype(np.int32)
    nn_s, m_s = o.vocab_prep(src)
    hs_src, cs_src = o.lstm_stack_forward(m["emb_s"], m["src_layers"], nn_s, m_s)
    table = np.zeros((longest, H, mb), np.float32)
    table[:S] = hs_src[L - 1]
    nn_t, m_t = o.vocab_prep(tin)
    tgt, tmask, _ = o.vocab_softmax(tout)
    hp = [np.asfortranarray(hs_src[l, S - 1]) for l in range(L)]
    cp = [np.asfortranarray(cs_src[l, S - 1]) for l in range(L)]
    h_tild_prev, total = None, 0.0
    for t in range(T):
        below = o.embed_gather(m["emb_t"], nn_t[t])
        for l in range(L):
            ly = m["tgt_layers"][l]
            feed = (l == 0 and t > 0)
            r = o.lstm_step(ly["M"], ly["Wh"], ly["b"], below, hp[l], cp[l], m_t[t], Q=ly["Q"] if feed else None,
                            htild=h_tild_prev if feed else None)
            hp[l], cp[l], below = r["h"], r["c"], r["h"]
        att = o.attention_forward(hs_table=table, batch_info=binfo, h_t=below, mask01=m_t[t], D=D, **m["attn"])
        frac = att["p_t"] - np.floor(att["p_t"])
        live = m_t[t] == 1
        assert np.all((frac[live] > 1e-4) & (frac[live] < 1 - 1e-4)), "p_t on an integer boundary; pick another seed"
        h_tild_prev = att["h_tild"]
        lp = o.softmax_logprob_f64(o.softmax_logits(m["D"], m["b_d"], att["h_tild"]))
        total += o.softmax_loss(lp, tgt[t], tmask[t])
    return total


@pytest.mark.parametrize("minibatch", [1, 3])
def test_force_decode_seq2seq_attention_feed_input(tmp_path, minibatch):
    g = synth.rng(93, minibatch)
    H, L, D, n_sent, longest = 32, 2, 4, 7, 20
    src_vocab = ["<UNK>"] + mf.make_vocab(50, "s")
    tgt_vocab = ["<START>", "<EOF>", "<UNK>"] + mf.make_vocab(60, "t")
    Vs, Vt = len(src_vocab), len(tgt_vocab)
    m = {"emb_s": synth.uniform(g, (H, Vs), -0.5, 0.5), "emb_t": synth.uniform(g, (H, Vt), -0.5, 0.5),
         "src_layers": [synth.lstm_layer(g, H, forget_bias_one=True) for _ in range(L)],
         "tgt_layers": [synth.lstm_layer(g, H, feed_input=(l == 0), forget_bias_one=True) for l in range(L)],
         "attn": synth.attention_weights(g, H), "D": synth.uniform(g, (Vt, H), -0.5, 0.5),
         "b_d": synth.uniform(g, (Vt,), -0.5, 0.5)}
    for ly in m["src_layers"] + m["tgt_layers"]:
        for k in ("M", "Wh"):
            ly[k] = [synth.uniform(g, (H, H), -0.3, 0.3) for _ in range(4)]
    for k in ("W_a", "W_p", "W_c1", "W_c2"):
        m["attn"][k] = synth.uniform(g, (H, H), -0.3, 0.3)
    model = tmp_path / "model.nn"
    with open(model, "w") as f:
        mf.write_header(f, L, H, tgt_vocab, src_vocab, True, True)
        _write_ih(f, m["src_layers"][0], m["emb_s"])
        for ly in m["src_layers"][1:]:
            _write_hh(f, ly)
        _write_ih(f, m["tgt_layers"][0], m["emb_t"])
        for i, ly in enumerate(m["tgt_layers"][1:]):
            _write_hh(f, ly, m["attn"] if i == L - 2 else None)
        _write_matrix(f, m["D"])
        _write_matrix(f, m["b_d"].reshape(-1, 1))
    src = mf.random_sentences(g, src_vocab, n_sent, 2, 9)
    tgt = mf.random_sentences(g, tgt_vocab, n_sent, 1, 8)
    sp, tp, out = tmp_path / "src.txt", tmp_path / "tgt.txt", tmp_path / "scores.txt"
    sp.write_text("".join(" ".join(s) + "\n" for s in src))
    tp.write_text("".join(" ".join(t) + "\n" for t in tgt))
    dump = tmp_path / "dump.nn"
    r = mf.run_force_decode(["--minibatch", minibatch, "--longest-sent", longest, "--attention-width", D, "--dump", dump,
                             model, sp, tp, out])
    assert r.returncode == 0, r.stderr[-2000:]
    # the dumped file is a complete model file again: same header and vocabulary lines, same numbers
    a, b = open(model).read().split("\n"), open(dump).read().split("\n")
    n_head = 1 + 3 + Vs + Vt
    assert a[:n_head] == b[:n_head]
    na = np.array(" ".join(a[n_head:]).split(), dtype=np.float64)
    nb = np.array(" ".join(b[n_head:]).split(), dtype=np.float64)
    assert na.shape == nb.shape and np.allclose(na, nb, rtol=1e-6, atol=0)
    got = [float(x) for x in out.read_text().split()]
    data = mf.integerize_pairs(src, tgt, src_vocab, tgt_vocab, minibatch)
    chunks = [data[i:i + minibatch] for i in range(0, len(data), minibatch)]
    assert len(got) == len(chunks)
    want = [_oracle_seq2seq(m, c, minibatch, D, longest) for c in chunks]
    for a, b in zip(got, want):
        assert a == pytest.approx(b, rel=1e-4, abs=1e-4)
    words = sum(len(t) + 1 for t in tgt)
    ppl = float([ln for ln in r.stdout.splitlines() if ln.startswith("Perplexity:")][0].split()[1])
    assert ppl == pytest.approx(np.exp(-sum(want) / words), rel=1e-4)


def test_force_decode_sequence_model(tmp_path):
    g = synth.rng(94, 1)
    H, L, minibatch, longest = 48, 2, 4, 16
    tgt_vocab = ["<START>", "<EOF>", "<UNK>"] + mf.make_vocab(70, "w")
    Vt = len(tgt_vocab)
    emb = synth.uniform(g, (H, Vt), -0.5, 0.5)
    layers = [synth.lstm_layer(g, H, forget_bias_one=True) for _ in range(L)]
    Dm, bd = synth.uniform(g, (Vt, H), -0.5, 0.5), synth.uniform(g, (Vt,), -0.5, 0.5)
    model = tmp_path / "lm.nn"
    with open(model, "w") as f:
        mf.write_header(f, L, H, tgt_vocab, [], False, False, lm=True)
        _write_ih(f, layers[0], emb)
        for ly in layers[1:]:
            _write_hh(f, ly)
        _write_matrix(f, Dm)
        _write_matrix(f, bd.reshape(-1, 1))
    tgt = mf.random_sentences(g, tgt_vocab, 10, 1, 10)
    tp, out = tmp_path / "tgt.txt", tmp_path / "scores.txt"
    tp.write_text("".join(" ".join(t) + "\n" for t in tgt))
    r = mf.run_force_decode(["--sequence", "--minibatch", minibatch, "--longest-sent", longest, model, tp, out])
    assert r.returncode == 0, r.stderr[-2000:]
    got = [float(x) for x in out.read_text().split()]
    data = mf.integerize_targets(tgt, tgt_vocab, minibatch)
    chunks = [data[i:i + minibatch] for i in range(0, len(data), minibatch)]
    assert len(got) == len(chunks)
    for a, c in zip(got, chunks):
        tin, tout = _time_major([x[0] for x in c], minibatch), _time_major([x[1] for x in c], minibatch)
        nn, msk = o.vocab_prep(tin)
        hs, _ = o.lstm_stack_forward(emb, layers, nn, msk)
        tg, tm, _ = o.vocab_softmax(tout)
        want = 0.0
        for t in range(tin.shape[0]):
            lp = o.softmax_logprob_f64(o.softmax_logits(Dm, bd, np.asfortranarray(hs[L - 1, t])))
            want += o.softmax_loss(lp, tg[t], tm[t])
        assert a == pytest.approx(want, rel=1e-4, abs=1e-4)
