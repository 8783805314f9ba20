"""The beam-search translation driver (zoph_rnn_amd/host/beam_decode) end to end: model file and source text in,
k-best hypotheses out, against one oracle decode per sentence (the reference decodes one sentence per pass).  Covers
the C++ beam_decoder (encoder sweep, state replication, feed-input, attention, device-side beam, state reorder),
grouping by source length, the step cap min(1.5 * source length, longest_sent - 2) and the k-best selection."""
import numpy as np
import pytest

import model_files_util as mf
from test_gpu_decode import _model, _oracle_decode, _oracle_ensemble_decode
from test_gpu_host_layers import _write_hh, _write_ih, _write_matrix
from zoph_rnn_amd import synth

pytestmark = pytest.mark.gpu


def _parse_blocks(text):
    sents, cur = [], None
    lines = text.split("\n")
    i = 0
    while i < len(lines):
        ln = lines[i]
        if ln.startswith("-----"):
            cur = []
            sents.append(cur)
        elif ln.startswith("-Score:"):
            score = float(ln.split()[1])
            words = [int(x) for x in lines[i + 1].split()]
            cur.append((words, score))
            i += 1
        i += 1
    return sents


@pytest.mark.parametrize("L,beam,batch,unk", [(2, 4, 3, False), (1, 3, 8, False), (2, 4, 3, True)])
def test_beam_decode_cli_matches_per_sentence_oracle(tmp_path, L, beam, batch, unk):
    """unk: with --UNK-decode the side file must hold, per printed hypothesis, the Viterbi alignment at position j+1 for
    every <UNK> (id 2) at position j (src/decoder.h:1452-1459); the third of the target vocabulary's ids being <UNK>,
    and the random model producing it now and then, some lines are non-empty (checked)."""
    g = synth.rng(95, L + beam)
    H, D, longest, K = 64, 3, 24, 3
    src_vocab = ["<UNK>"] + mf.make_vocab(79, "s")
    tgt_vocab = ["<START>", "<EOF>", "<UNK>"] + mf.make_vocab(397, "t")
    Vs, Vt = len(src_vocab), len(tgt_vocab)
    m = _model(g, H, Vs, Vt, L)
    if unk:
        m["b_soft"][2] += 7.0  # <UNK> likely enough to show up in the hypotheses
        # window centres and scores that move from step to step, so that the alignments do
        m["attn"]["v_p"] = m["attn"]["v_p"] * 60
        m["attn"]["W_a"] = m["attn"]["W_a"] * 16
    model = tmp_path / "model.nn"
    with open(model, "w") as f:
        mf.write_header(f, L, H, tgt_vocab, src_vocab, True, True)
        _write_ih(f, m["src_layers"][0], m["src_embed"])
        for ly in m["src_layers"][1:]:
            _write_hh(f, ly)
        _write_ih(f, m["tgt_layers"][0], m["tgt_embed"], m["attn"] if L == 1 else None)
        for i, ly in enumerate(m["tgt_layers"][1:]):
            _write_hh(f, ly, m["attn"] if i == L - 2 else None)
        _write_matrix(f, m["D_soft"])
        _write_matrix(f, m["b_soft"].reshape(-1, 1))
    # sentences of three different lengths, interleaved, with unknown words
    lens = [5, 7, 5, 4, 7, 5, 4]
    src = [mf.random_sentences(g, src_vocab, 1, n, n)[0] for n in lens]
    sp, out = tmp_path / "src.txt", tmp_path / "out.txt"
    sp.write_text("".join(" ".join(s) + "\n" for s in src))
    unk_path = tmp_path / "unk.txt"
    r = mf.run_program("beam_decode", ["--beam", beam, "--batch", batch, "--longest-sent", longest, "--attention-width",
                                       D, "--num-best", K, "--print-score", "--ids"] +
                       (["--UNK-decode", unk_path] if unk else []) + [model, sp, out])
    assert r.returncode == 0, r.stderr[-2000:]
    got = _parse_blocks(out.read_text())
    assert len(got) == len(src)
    unk_lines = unk_path.read_text().split("\n")[:-1] if unk else []
    want_unk, shifted = [], 0
    smap = {w: i for i, w in enumerate(src_vocab)}
    for s, words in enumerate(src):
        ids = np.array([smap.get(w, 0) for w in words][::-1], np.int32)
        S = len(ids)
        steps = min(int(1.5 * S), longest - 2)
        res = _oracle_decode(m, ids, S, S, beam, steps, D, 0.0, viterbi=unk)
        hyps, gap = res[1], res[2]
        vits = res[3] if unk else [None] * len(hyps)
        assert gap > 5e-6, "candidate scores nearly tie (gap %.2e): pick another seed" % gap
        keep = [(w, sc, v) for (w, sc), v in zip(hyps, vits) if len(w) / S > 0.5]
        keep.sort(key=lambda t: -t[1])
        want = [(w, sc) for w, sc, _ in keep[:K]]
        for w, _, v in keep[:K]:
            want_unk.append("".join("%d " % v[j + 1] for j in range(len(w) - 1) if w[j] == 2))
            shifted += sum(1 for j in range(len(w) - 1) if w[j] == 2 and v[j] != v[j + 1])
        assert len(got[s]) == len(want), (s, len(got[s]), len(want))
        for (gw, gs), (ww, ws) in zip(got[s], want):
            assert gw == list(ww), (s, gw, list(ww))
            assert gs == pytest.approx(ws, rel=1e-4, abs=1e-4)
    if unk:
        assert unk_lines == want_unk
        assert any(ln for ln in want_unk), "no <UNK> in any hypothesis: the side file shows nothing"
        assert shifted >= 1, "every <UNK> has the same alignment before and after: position j would pass for j+1"


def _write_model(path, m, L, H, tgt_vocab, src_vocab):
    with open(path, "w") as f:
        mf.write_header(f, L, H, tgt_vocab, src_vocab, True, True)
        _write_ih(f, m["src_layers"][0], m["src_embed"])
        for ly in m["src_layers"][1:]:
            _write_hh(f, ly)
        _write_ih(f, m["tgt_layers"][0], m["tgt_embed"], m["attn"] if L == 1 else None)
        for i, ly in enumerate(m["tgt_layers"][1:]):
            _write_hh(f, ly, m["attn"] if i == L - 2 else None)
        _write_matrix(f, m["D_soft"])
        _write_matrix(f, m["b_soft"].reshape(-1, 1))


def _round_matrices_to_bf16(m):
    """Every matrix the decoder streams (LSTM, attention, output layer) rounded to bf16, so that bf16 storage is exact."""
    from gpu_util import round_bf16
    rb = lambda a: np.asfortranarray(round_bf16(a))
    for ly in m["src_layers"] + m["tgt_layers"]:
        for k in ("M", "Wh", "Q"):
            if k in ly:
                ly[k] = [rb(x) for x in ly[k]]
    for k in ("W_a", "W_p", "W_c1", "W_c2"):
        m["attn"][k] = rb(m["attn"][k])
    m["D_soft"] = rb(m["D_soft"])


@pytest.mark.parametrize("n_models,L,bf16,unk", [(2, 2, False, False), (3, 1, False, False), (2, 2, True, False),
                                                 (2, 2, False, True), (3, 1, False, True)])
def test_beam_decode_cli_ensemble_matches_per_sentence_oracle(tmp_path, n_models, L, bf16, unk):
    """A comma-separated list of model files decodes as an ensemble (src/ensemble_factory.hpp:767-793): the models'
    output distributions are averaged and renormalised at every step, one beam picks the words, every model's states
    are reordered by that beam's back-pointers.  The models differ in every weight and in their source vocabularies
    (same words, another order: each model integerizes the source text with its own mapping); an ensemble that read
    only its first model, or fed every model the first model's source ids, fails.  bf16: the members store their matrices
    as bf16 (--bf16; the matrices are bf16-representable, so the fp32 oracle on the same matrices is the bar).
    unk: with --UNK-decode the side file holds the models' alignment VOTE (src/ensemble_factory.hpp:797-834), which must
    differ from the first model's own alignment somewhere for the comparison to show anything (checked)."""
    g = synth.rng(98, n_models)
    H, D, longest, K, beam = 64, 3, 24, 3, 4
    base_src = mf.make_vocab(79, "s")
    tgt_vocab = ["<START>", "<EOF>", "<UNK>"] + mf.make_vocab(397, "t")
    ms, src_vocabs, paths = [], [], []
    for k in range(n_models):
        sv = ["<UNK>"] + [base_src[i] for i in g.permutation(len(base_src))]
        m = _model(g, H, len(sv), len(tgt_vocab), L)
        if bf16:
            _round_matrices_to_bf16(m)
        if unk:
            m["b_soft"][2] += 7.0  # <UNK> likely enough to show up; alignments that move from step to step
            m["attn"]["v_p"] = m["attn"]["v_p"] * 60
            m["attn"]["W_a"] = m["attn"]["W_a"] * 16
        p = tmp_path / ("model%d.nn" % k)
        _write_model(p, m, L, H, tgt_vocab, sv)
        ms.append(m)
        src_vocabs.append(sv)
        paths.append(str(p))
    lens = [5, 7, 5, 4, 7, 5]
    src = [mf.random_sentences(g, src_vocabs[0], 1, n, n)[0] for n in lens]
    sp, out = tmp_path / "src.txt", tmp_path / "out.txt"
    sp.write_text("".join(" ".join(s) + "\n" for s in src))
    unk_path = tmp_path / "unk.txt"
    r = mf.run_program("beam_decode", (["--bf16"] if bf16 else []) + (["--UNK-decode", unk_path] if unk else []) +
                       ["--beam", beam, "--batch", 3, "--longest-sent", longest, "--attention-width", D,
                        "--num-best", K, "--print-score", "--ids", ",".join(paths), sp, out])
    assert r.returncode == 0, r.stderr[-2000:]
    got = _parse_blocks(out.read_text())
    assert len(got) == len(src)
    smaps = [{w: i for i, w in enumerate(sv)} for sv in src_vocabs]
    differs_from_first = vote_differs = 0
    want_unk = []
    for s, words in enumerate(src):
        cols = [np.array([sm.get(w, 0) for w in words][::-1], np.int32) for sm in smaps]
        S = len(words)
        steps = min(int(1.5 * S), longest - 2)
        res = _oracle_ensemble_decode(ms, cols, S, beam, steps, D, viterbi=unk)
        hyps, gap = res[0], res[1]
        vits = res[2] if unk else [None] * len(hyps)
        vote_differs += res[3] if unk else 0
        assert gap > (5e-5 if bf16 else 5e-6), "candidate scores nearly tie (gap %.2e): pick another seed" % gap
        keep = [(w, sc, v) for (w, sc), v in zip(hyps, vits) if len(w) / S > 0.5]
        keep.sort(key=lambda t: -t[1])
        want = [(w, sc) for w, sc, _ in keep[:K]]
        for w, _, v in keep[:K]:
            want_unk.append("".join("%d " % v[j + 1] for j in range(len(w) - 1) if w[j] == 2))
        assert len(got[s]) == len(want), (s, len(got[s]), len(want))
        for (gw, gs), (ww, ws) in zip(got[s], want):
            assert gw == list(ww), (s, gw, list(ww))
            assert gs == pytest.approx(ws, rel=1e-4, abs=2e-4 if bf16 else 1e-4)
        alone = _oracle_decode(ms[0], cols[0], S, S, beam, steps, D, 0.0)[1]
        alone = sorted([(w, sc) for (w, sc) in alone if len(w) / S > 0.5], key=lambda t: -t[1])[:K]
        differs_from_first += [list(w) for w, _ in alone] != [list(w) for w, _ in want]
    assert differs_from_first >= 1, "the ensemble's output equals the first model's alone: the test shows nothing"
    if unk:
        assert unk_path.read_text().split("\n")[:-1] == want_unk
        assert any(ln for ln in want_unk), "no <UNK> in any hypothesis: the side file shows nothing"
        assert vote_differs >= 1, "the vote always equals the first model's own alignment: the test shows nothing"


def test_beam_decode_cli_ensemble_refuses_mismatched_models(tmp_path):
    g = synth.rng(99, 1)
    H, L = 48, 1
    src_vocab = ["<UNK>"] + mf.make_vocab(30, "s")
    paths = []
    for k, nt in enumerate((100, 101)):
        tgt_vocab = ["<START>", "<EOF>", "<UNK>"] + mf.make_vocab(nt, "t")
        m = _model(g, H, len(src_vocab), len(tgt_vocab), L)
        p = tmp_path / ("m%d.nn" % k)
        _write_model(p, m, L, H, tgt_vocab, src_vocab)
        paths.append(str(p))
    sp, out = tmp_path / "src.txt", tmp_path / "out.txt"
    sp.write_text("s1 s2 s3\n")
    r = mf.run_program("beam_decode", ["--beam", 3, "--batch", 2, "--longest-sent", 20, ",".join(paths), sp, out])
    assert r.returncode != 0 and "vocabular" in r.stderr


def test_beam_decode_cli_decodes_a_batch_again_after_an_abandoned_launch(tmp_path):
    """The decoder's context is put on the single-launch schedules whenever they fit, with waits that expect one arrival
    more than will come and a poll limit of 64 (every kernel still exits normally): the first decoder step's launch gives
    up, the program notices after that step, switches the context to one launch per layer and decodes the batch again.
    The output must be that of an ordinary run, and the program says how often it started over."""
    g = synth.rng(97, 1)
    H, L, beam, batch, longest, D, K = 64, 2, 4, 3, 24, 3, 2
    src_vocab = ["<UNK>"] + mf.make_vocab(60, "s")
    tgt_vocab = ["<START>", "<EOF>", "<UNK>"] + mf.make_vocab(300, "t")
    m = _model(g, H, len(src_vocab), len(tgt_vocab), L)
    model = tmp_path / "model.nn"
    _write_model(model, m, L, H, tgt_vocab, src_vocab)
    src = [mf.random_sentences(g, src_vocab, 1, n, n)[0] for n in (5, 6, 5, 5, 6)]
    sp = tmp_path / "src.txt"
    sp.write_text("".join(" ".join(s) + "\n" for s in src))
    outs = []
    for name, env in (("plain", None),
                      ("abandon", {"ZR_LSTM_SWEEP": 2, "ZR_LSTM_SWEEP_SPIN": 64, "ZR_LSTM_STEP_WAIT_EXTRA": 1})):
        out = tmp_path / (name + ".txt")
        r = mf.run_program("beam_decode", ["--beam", beam, "--batch", batch, "--longest-sent", longest,
                                           "--attention-width", D, "--num-best", K, "--print-score", "--ids", model, sp,
                                           out], env=env)
        assert r.returncode == 0, (name, r.stderr[-2000:])
        outs.append((_parse_blocks(out.read_text()), r.stdout))
    (plain, plain_log), (again, again_log) = outs
    assert "decoded again" not in plain_log
    counts = [int(ln.split(":")[1]) for ln in again_log.split("\n") if "decoded again" in ln]
    # two source lengths -> two batches of 3 and of 2 sentences; the first gives up and switches the context over for good
    assert counts == [1], again_log
    assert len(plain) == len(again) == len(src)
    for a, b in zip(plain, again):
        assert [w for w, _ in a] == [w for w, _ in b]
        for (_, sa), (_, sb) in zip(a, b):
            assert sa == pytest.approx(sb, rel=1e-4, abs=1e-4)


def test_beam_decode_cli_default_output_is_words(tmp_path):
    g = synth.rng(96, 1)
    H, L = 48, 1
    src_vocab = ["<UNK>"] + mf.make_vocab(30, "s")
    tgt_vocab = ["<START>", "<EOF>", "<UNK>"] + mf.make_vocab(100, "t")
    m = _model(g, H, len(src_vocab), len(tgt_vocab), L)
    model = tmp_path / "model.nn"
    with open(model, "w") as f:
        mf.write_header(f, L, H, tgt_vocab, src_vocab, True, True)
        _write_ih(f, m["src_layers"][0], m["src_embed"])
        _write_ih(f, m["tgt_layers"][0], m["tgt_embed"], m["attn"])
        _write_matrix(f, m["D_soft"])
        _write_matrix(f, m["b_soft"].reshape(-1, 1))
    src = mf.random_sentences(g, src_vocab, 5, 3, 6)
    sp, out = tmp_path / "src.txt", tmp_path / "out.txt"
    sp.write_text("".join(" ".join(s) + "\n" for s in src))
    r = mf.run_program("beam_decode", ["--beam", 3, "--batch", 2, "--longest-sent", 20, model, sp, out])
    assert r.returncode == 0, r.stderr[-2000:]
    lines = out.read_text().split("\n")[:-1]
    assert len(lines) == len(src)
    for ln in lines:
        assert all(w in tgt_vocab[2:] for w in ln.split())  # words, no <START> / <EOF>


def test_beam_decode_cli_with_bf16_weight_storage(tmp_path):
    """--bf16: every streamed matrix (LSTM, attention, output layer) is stored as bf16 on the device and the decode runs
    through the bf16 decoder step (the step's inputs split into bf16 terms in one launch, every LSTM node leaving its h as
    bf16 terms for the next product).  The model's matrices are bf16-representable, so the storage is exact and the
    fp32 oracle on the same matrices is the bar: same words, scores to 1e-4."""
    g = synth.rng(97, 3)
    H, L, D, longest, K, beam = 64, 2, 3, 24, 2, 4
    src_vocab = ["<UNK>"] + mf.make_vocab(79, "s")
    tgt_vocab = ["<START>", "<EOF>", "<UNK>"] + mf.make_vocab(397, "t")
    m = _model(g, H, len(src_vocab), len(tgt_vocab), L)
    _round_matrices_to_bf16(m)
    model = tmp_path / "model.nn"
    with open(model, "w") as f:
        mf.write_header(f, L, H, tgt_vocab, src_vocab, True, True)
        _write_ih(f, m["src_layers"][0], m["src_embed"])
        for ly in m["src_layers"][1:]:
            _write_hh(f, ly)
        _write_ih(f, m["tgt_layers"][0], m["tgt_embed"], None)
        for i, ly in enumerate(m["tgt_layers"][1:]):
            _write_hh(f, ly, m["attn"] if i == L - 2 else None)
        _write_matrix(f, m["D_soft"])
        _write_matrix(f, m["b_soft"].reshape(-1, 1))
    lens = [5, 7, 5, 4, 7]
    src = [mf.random_sentences(g, src_vocab, 1, n, n)[0] for n in lens]
    sp, out = tmp_path / "src.txt", tmp_path / "out.txt"
    sp.write_text("".join(" ".join(s) + "\n" for s in src))
    r = mf.run_program("beam_decode", ["--bf16", "--beam", beam, "--batch", 3, "--longest-sent", longest,
                                       "--attention-width", D, "--num-best", K, "--print-score", "--ids", model, sp, out])
    assert r.returncode == 0, r.stderr[-2000:]
    got = _parse_blocks(out.read_text())
    assert len(got) == len(src)
    smap = {w: i for i, w in enumerate(src_vocab)}
    for s, words in enumerate(src):
        ids = np.array([smap.get(w, 0) for w in words][::-1], np.int32)
        S = len(ids)
        steps = min(int(1.5 * S), longest - 2)
        _, hyps, gap = _oracle_decode(m, ids, S, S, beam, steps, D, 0.0)
        assert gap > 5e-5, "candidate scores nearly tie (gap %.2e): pick another seed" % gap
        keep = [(w, sc) for (w, sc) in hyps if len(w) / S > 0.5]
        keep.sort(key=lambda t: -t[1])
        want = keep[:K]
        assert len(got[s]) == len(want), (s, len(got[s]), len(want))
        for (gw, gs), (ww, ws) in zip(got[s], want):
            assert gw == list(ww), (s, gw, list(ww))
            assert gs == pytest.approx(ws, rel=1e-4, abs=2e-4)
