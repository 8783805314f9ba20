"""Model-file header / vocabulary blocks and the integerization of raw text (the data formats either side of the
forward path), checked on the CPU through `force_decode --integerize-only` against an independent Python
restatement of the reference's preparation rules."""
import numpy as np
import pytest

import model_files_util as mf
from zoph_rnn_amd import synth


def _setup(tmp_path, lm=False, n=11, minibatch=4, seed=3):
    g = synth.rng(91, seed)
    src_vocab = ["<UNK>"] + mf.make_vocab(30, "s")
    tgt_vocab = ["<START>", "<EOF>", "<UNK>"] + mf.make_vocab(40, "t")
    src = mf.random_sentences(g, src_vocab, n, 1, 9)
    tgt = mf.random_sentences(g, tgt_vocab, n, 1, 8)
    model = tmp_path / "model.nn"
    with open(model, "w") as f:
        mf.write_header(f, 2, 16, tgt_vocab, src_vocab, True, True, lm=lm)
    sp, tp = tmp_path / "src.txt", tmp_path / "tgt.txt"
    sp.write_text("".join(" ".join(s) + "\n" for s in src))
    tp.write_text("".join(" ".join(t) + "\n" for t in tgt))
    return src_vocab, tgt_vocab, src, tgt, model, sp, tp


@pytest.mark.parametrize("minibatch", [1, 4])
def test_integerize_parallel_text(tmp_path, minibatch):
    sv, tv, src, tgt, model, sp, tp = _setup(tmp_path, minibatch=minibatch)
    out = tmp_path / "scores.txt"
    r = mf.run_force_decode(["--integerize-only", "--minibatch", minibatch, "--int-file", tmp_path / "d.int", model, sp,
                             tp, out])
    assert r.returncode == 0, r.stderr
    want = mf.integerize_pairs(src, tgt, sv, tv, minibatch)
    got = mf.read_int_file(tmp_path / "d.int")
    assert got == want
    assert "Sentences: %d" % len(src) in r.stdout
    assert "Total target words: %d" % sum(len(t) + 1 for t in tgt) in r.stdout
    # the rules themselves: reversed source with <UNK> = 0 for unknown words, left padding; <START> ... / ... <EOF>
    s0 = [sv.index(w) if w in sv else 0 for w in src[0]][::-1]
    assert [x for x in got[0][0] if x != -1] == s0
    assert got[0][2][0] == 0 and 1 in got[0][3]
    assert all(x in (-1, -2) for x in got[0][1])


def test_integerize_sequence_model_text(tmp_path):
    sv, tv, src, tgt, model, sp, tp = _setup(tmp_path, lm=True)
    r = mf.run_force_decode(["--sequence", "--integerize-only", "--minibatch", 3, "--int-file", tmp_path / "d.int",
                             model, tp, tmp_path / "scores.txt"])
    assert r.returncode == 0, r.stderr
    want = mf.integerize_targets(tgt, tv, 3)
    got = mf.read_int_file(tmp_path / "d.int")
    assert [g[:2] for g in got] == [[[], []]] * len(tgt)
    assert [g[2:] for g in got] == want
    # one fully padded extra step per minibatch, as the reference's `while size <= max` padding leaves
    assert all(g[2][-1] == -1 and g[3][-1] == -1 for g in got)


@pytest.mark.parametrize("header,msg", [
    ("2 16 43\n", "separator"),                     # no separator line
    ("2 16 43 31 1 1 1 0 0\n" + mf.SEP + "\n", "multi-source"),
    ("2 16\n" + mf.SEP + "\n", "fields"),
    ("2 16 43 31 1 1 0 0 0\n" + mf.SEP + "\n0 <UNK>\n" + mf.SEP + "\n0 <START>\n" + mf.SEP + "\n", "do not match"),
])
def test_malformed_model_files_are_refused(tmp_path, header, msg):
    model = tmp_path / "bad.nn"
    model.write_text(header)
    (tmp_path / "s.txt").write_text("a b\n")
    (tmp_path / "t.txt").write_text("c d\n")
    r = mf.run_force_decode(["--integerize-only", model, tmp_path / "s.txt", tmp_path / "t.txt", tmp_path / "o.txt"])
    assert r.returncode == 1
    assert msg in r.stderr


def test_too_long_sentence_is_an_error_not_a_truncation(tmp_path):
    sv, tv, src, tgt, model, sp, tp = _setup(tmp_path)
    r = mf.run_force_decode(["--integerize-only", "--longest-sent", 6, model, sp, tp, tmp_path / "o.txt"])
    assert r.returncode == 1 and "longer than longest_sent" in r.stderr


@pytest.mark.parametrize("lm,L", [(False, 2), (True, 1), (False, 1)])
def test_written_model_files_read_back_under_the_reference_scripts_layout(tmp_path, lm, L):
    """The test-suite's model writer against a second description of the format: the reference's own Python reader for
    models without attention (scripts/load_model.py), restated in model_files_util.parse_like_reference_script.  Pins
    the separator and vocabulary lines, one matrix row per line, the empty line behind every matrix and the order of
    the matrices of both layer kinds and the loss layer (gates are distinct random matrices, so a swapped pair fails)."""
    from test_gpu_host_layers import _write_hh, _write_ih, _write_matrix
    g = synth.rng(77, L + int(lm))
    H = 6
    src_vocab = ["<UNK>"] + mf.make_vocab(7, "s")
    tgt_vocab = ["<START>", "<EOF>", "<UNK>"] + mf.make_vocab(9, "t")
    Vs, Vt = len(src_vocab), len(tgt_vocab)
    m = {"emb_t": synth.uniform(g, (H, Vt)), "tgt_layers": [synth.lstm_layer(g, H, forget_bias_one=True) for _ in range(L)],
         "D": synth.uniform(g, (Vt, H)), "b_d": synth.uniform(g, (Vt,))}
    if not lm:
        m["emb_s"] = synth.uniform(g, (H, Vs))
        m["src_layers"] = [synth.lstm_layer(g, H) for _ in range(L)]
    path = tmp_path / "m.nn"
    with open(path, "w") as f:
        mf.write_header(f, L, H, tgt_vocab, src_vocab, False, False, lm=lm)
        if not lm:
            _write_ih(f, m["src_layers"][0], m["emb_s"])
            for ly in m["src_layers"][1:]:
                _write_hh(f, ly)
        _write_ih(f, m["tgt_layers"][0], m["emb_t"])
        for ly in m["tgt_layers"][1:]:
            _write_hh(f, ly)
        _write_matrix(f, m["D"])
        _write_matrix(f, m["b_d"].reshape(-1, 1))
    head, sv, tv, sl, tl, D, b = mf.parse_like_reference_script(path)
    assert head[:4] == [L, H, Vt, 0 if lm else Vs]
    assert tv == dict(enumerate(tgt_vocab))
    if lm:
        assert sv is None and sl is None
    else:
        assert sv == dict(enumerate(src_vocab))
        mf.check_layers_against_script_reading(m["src_layers"], m["emb_s"], sl)
    mf.check_layers_against_script_reading(m["tgt_layers"], m["emb_t"], tl)
    assert np.allclose(D, m["D"], rtol=1e-7, atol=0) and np.allclose(b.reshape(-1), m["b_d"], rtol=1e-7, atol=0)
