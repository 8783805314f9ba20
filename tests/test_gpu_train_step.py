"""model_trainer (zoph_rnn_amd/host/zoph_model.h) end to end through tests/host/train_step: SGD steps on minibatches
of an integerized file, the updated model file compared with the same steps computed by the oracle (forward, loss
layer backward accumulated over the time steps, stack backward, 1/minibatch scaling, per-matrix norm clipping and
the ascent update in numpy).  The oracle's backward is pinned by torch autograd in tests/test_oracle_backward_pins.py.
Tolerance: 1e-4 of the largest weight change of each matrix plus 1e-6 absolute (the file holds 8 significant digits)."""
import os
import subprocess

import numpy as np
import pytest

import model_files_util as mf
import oracle_lib as o
from test_gpu_force_decode import _time_major
from test_gpu_host_layers import _write_hh, _write_ih, _write_matrix
from zoph_rnn_amd import synth

pytestmark = pytest.mark.gpu
DRIVER = os.path.join(mf.ROOT, "tests", "host", "train_step")


def _write_model(path, m, tgt_vocab, src_vocab, lm):
    L, H = len(m["tgt_layers"]), m["emb_t"].shape[0]
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


def _read_model(path, n_head, L, H, Vs, Vt, lm):
    """The dumped file back into the dictionary layout of _write_model (same matrix order)."""
    vals = np.array(" ".join(open(path).read().split("\n")[n_head:]).split(), dtype=np.float64)
    pos = [0]

    def take(r, c):
        a = vals[pos[0]:pos[0] + r * c].reshape(r, c)
        pos[0] += r * c
        return a

    def layer(V):
        ly = {"M": [None] * 4, "Wh": [None] * 4, "b": [None] * 4}
        for g in range(4):
            ly["Wh"][g] = take(H, H)
            ly["b"][g] = take(H, 1).reshape(-1)
        emb = take(H, V) if V else None
        for g in (0, 1, 3, 2):
            ly["M"][g] = take(H, H)
        return ly, emb

    m = {}
    for side, V in (("src", Vs), ("tgt", Vt)):
        if side == "src" and lm:
            continue
        first, emb = layer(V)
        m["emb_" + side[0]] = emb
        m[side + "_layers"] = [first] + [layer(0)[0] for _ in range(L - 1)]
    m["D"] = take(Vt, H)
    m["b_d"] = take(Vt, 1).reshape(-1)
    assert pos[0] == vals.size
    return m


def _clip_update(W, grad, mb, clip, lr, clipped, mode="matrix", whole_norm=None):
    """mode "matrix": clip bounds this gradient's own norm; "whole": it bounds whole_norm, the norm of all gradients of
    the model together; "element": every element is clamped to +-clip."""
    g = np.asarray(grad, np.float64) / mb
    if mode == "element":
        clipped.append(bool((np.abs(g) > clip).any()))
        g = np.clip(g, -clip, clip)
    else:
        norm = np.sqrt((g * g).sum()) if mode == "matrix" else whole_norm
        clipped.append(bool(norm > clip))
        if norm > clip:
            g = g * (clip / norm)
    return (np.asarray(W, np.float64) + lr * g).astype(np.float32)


def _oracle_step(m, chunk, mb, lm, lr, clip, clipped, mode="matrix", norms=None, cell=None):
    """One training step on the oracle; updates m in place and returns the log-likelihood before the update."""
    L = len(m["tgt_layers"])
    if lm:
        tin, tout = _time_major([c[0] for c in chunk], mb), _time_major([c[1] for c in chunk], mb)
        h0 = c0 = None
    else:
        src, tin, tout = (_time_major([c[k] for c in chunk], mb) for k in (0, 2, 3))
        S = src.shape[0]
        nn_s, m_s = o.vocab_prep(src)
        hs_src, cs_src = o.lstm_stack_forward(m["emb_s"], m["src_layers"], nn_s, m_s, clip=cell[0] if cell else None)
        h0 = [np.asfortranarray(hs_src[l, S - 1]) for l in range(L)]
        c0 = [np.asfortranarray(cs_src[l, S - 1]) for l in range(L)]
    T = tin.shape[0]
    nn_t, m_t = o.vocab_prep(tin)
    hs, _ = o.lstm_stack_forward(m["emb_t"], m["tgt_layers"], nn_t, m_t, h0=h0, c0=c0, clip=cell[0] if cell else None)
    ck = dict(cell_clip=cell[0], err_clip=cell[1]) if cell else {}
    tgt, tmask, _ = o.vocab_softmax(tout)
    Vt, H = m["D"].shape
    dD, dbd = np.zeros((Vt, H), np.float64, order="F"), np.zeros(Vt, np.float64)
    err_top, loss = [], 0.0
    for t in range(T):
        h = np.asfortranarray(hs[L - 1, t])
        loss += o.softmax_loss(o.softmax_logprob_f64(o.softmax_logits(m["D"], m["b_d"], h)), tgt[t], tmask[t])
        e, dD, dbd = o.softmax_backward(m["D"], m["b_d"], h, tgt[t], tmask[t], dD, dbd)
        err_top.append(e)
    g_t, dW_t, eh0, ec0 = o.lstm_stack_backward(m["emb_t"], m["tgt_layers"], nn_t, m_t, err_top, h0=h0, c0=c0, **ck)
    sides = [("t", "tgt_layers", g_t, dW_t)]
    if not lm:
        zero_top = [np.zeros((H, mb), np.float32) for _ in range(S)]
        g_s, dW_s, _, _ = o.lstm_stack_backward(m["emb_s"], m["src_layers"], nn_s, m_s, zero_top, err_hT=eh0, err_cT=ec0,
                                                **ck)
        sides.append(("s", "src_layers", g_s, dW_s))
    whole = None
    if mode == "whole":  # src/model.hpp:1850-1892: every gradient of the model, scaled by 1 / minibatch
        ss = (np.asarray(dD, np.float64) ** 2).sum() + (np.asarray(dbd, np.float64) ** 2).sum()
        for _, _, grads, dW in sides:
            ss += (np.asarray(dW, np.float64) ** 2).sum()
            for gr in grads:
                ss += sum((np.asarray(gr[k][g], np.float64) ** 2).sum() for k in ("dM", "dWh", "db") for g in range(4))
        whole = np.sqrt(ss) / mb
        norms.append(whole)
    up = lambda W, g: _clip_update(W, g, mb, clip, lr, clipped, mode, whole)
    m["D"], m["b_d"] = up(m["D"], dD), up(m["b_d"], dbd)
    for s, key, grads, dW in sides:
        m["emb_" + s] = up(m["emb_" + s], dW)
        for ly, gr in zip(m[key], grads):
            for k, gk in (("M", "dM"), ("Wh", "dWh"), ("b", "db")):
                ly[k] = [up(ly[k][g], gr[gk][g]) for g in range(4)]
    return loss


def _compare(name, got, want, orig):
    d_got, d_want = np.asarray(got, np.float64) - orig, np.asarray(want, np.float64) - orig
    tol = 1e-4 * np.abs(d_want).max() + 1e-6
    err = np.abs(d_got - d_want).max()
    assert err <= tol, "%s: weight change off by %.3g (bound %.3g, largest change %.3g)" % (
        name, err, tol, np.abs(d_want).max())


def test_abandoned_forward_sweep_is_repeated_before_the_update(tmp_path):
    """The forward sweeps are made to give up their waits (one poll allowed; every workgroup still leaves the kernel
    normally): model_trainer must see it, run the forward pass again with one launch per diagonal, and end with the
    oracle's weights -- nothing of the abandoned sweep's outputs may reach them."""
    test_train_steps_match_oracle(tmp_path, True, 3, 64, 8, 2, 1.0, False, abandon=True)


@pytest.mark.parametrize("node_level", [False, True])
@pytest.mark.parametrize("lm,L,H,mb,steps,clip", [(True, 2, 32, 4, 1, 0.4), (False, 2, 48, 3, 1, 0.25),
                                                  (False, 1, 32, 5, 3, 5.0), (True, 3, 64, 8, 2, 1.0)])
def test_train_steps_match_oracle(tmp_path, lm, L, H, mb, steps, clip, node_level, abandon=False, mode="matrix",
                                  cell=None):
    """node_level: the same steps through the layer objects' back_prop_GPU / update_weights members
    (forward_model::compute_gradients) instead of model_trainer."""
    if not os.path.exists(DRIVER):
        pytest.fail("tests/host/train_step is not built: run `python __graft_entry__.py build`")
    g = synth.rng(131, L * 100 + H + mb)
    lr, longest = 0.5, 16
    src_vocab = ["<UNK>"] + mf.make_vocab(40, "s")
    tgt_vocab = ["<START>", "<EOF>", "<UNK>"] + mf.make_vocab(50, "t")
    Vs, Vt = len(src_vocab), len(tgt_vocab)
    m = {"emb_t": synth.uniform(g, (H, Vt), -0.5, 0.5),
         "tgt_layers": [synth.lstm_layer(g, H, forget_bias_one=True) for _ in range(L)],
         "D": synth.uniform(g, (Vt, H), -0.5, 0.5), "b_d": synth.uniform(g, (Vt,), -0.5, 0.5)}
    if not lm:
        m["emb_s"] = synth.uniform(g, (H, Vs), -0.5, 0.5)
        m["src_layers"] = [synth.lstm_layer(g, H, forget_bias_one=True) for _ in range(L)]
    model = tmp_path / "model.nn"
    _write_model(model, m, tgt_vocab, src_vocab, lm)
    n_head = 1 + (2 if lm else 3) + (0 if lm else Vs) + Vt
    orig = _read_model(model, n_head, L, H, Vs, Vt, lm)
    n_sent = 2 * mb
    tgt = mf.random_sentences(g, tgt_vocab, n_sent, 1, 8)
    data_path = tmp_path / "data.int"
    if lm:
        data = mf.integerize_targets(tgt, tgt_vocab, mb)
        rows = [[[], [], d[0], d[1]] for d in data]
    else:
        src = mf.random_sentences(g, src_vocab, n_sent, 2, 9)
        data = mf.integerize_pairs(src, tgt, src_vocab, tgt_vocab, mb)
        rows = data
    with open(data_path, "w") as f:
        for r in rows:
            for k in range(4):
                f.write(" ".join(str(v) for v in r[k]) + "\n")
    args = (["--sequence"] if lm else []) + (["--node-level"] if node_level else []) + \
        (["--abandon-sweeps"] if abandon else []) + (["--whole-clip"] if mode == "whole" else []) + \
        (["--ind-clip=%r" % clip] if mode == "element" else []) + \
        (["--clip-cell=%r,%r" % cell] if cell else []) + \
        [str(model), str(data_path), str(mb), str(longest), str(lr), str(clip), str(steps)]
    r = subprocess.run([DRIVER] + args, capture_output=True, text=True, timeout=300)
    assert r.returncode == 0, r.stderr[-2000:]
    got_loss = [float(ln.split()[2]) for ln in r.stdout.splitlines() if ln.startswith("loss")]
    if abandon:
        n_abandoned = [int(ln.split()[1]) for ln in r.stdout.splitlines() if ln.startswith("abandoned")]
        assert n_abandoned == [steps], "every step's forward sweep should have been abandoned and repeated"
    chunks = [data[i:i + mb] for i in range(0, len(data), mb)]
    clipped, want_loss, want_norms = [], [], []
    if cell:  # the clamps must matter: one step without them moves a recurrent matrix somewhere else
        import copy
        m_with, m_without = copy.deepcopy(m), copy.deepcopy(m)
        _oracle_step(m_with, chunks[0], mb, lm, lr, clip, [], mode, [], cell)
        _oracle_step(m_without, chunks[0], mb, lm, lr, clip, [], mode, [], None)
        moved = np.abs(np.asarray(m_with["tgt_layers"][0]["Wh"][0]) - np.asarray(m["tgt_layers"][0]["Wh"][0])).max()
        apart = np.abs(np.asarray(m_with["tgt_layers"][0]["Wh"][0]) - np.asarray(m_without["tgt_layers"][0]["Wh"][0])).max()
        assert apart > 0.02 * moved, "thresholds too high to act (%g of %g)" % (apart, moved)
    for s in range(steps):
        want_loss.append(_oracle_step(m, chunks[s % len(chunks)], mb, lm, lr, clip, clipped, mode, want_norms, cell))
    if mode == "whole":
        got_norms = [float(ln.split()[2]) for ln in r.stdout.splitlines() if ln.startswith("global_norm")]
        assert got_norms == pytest.approx(want_norms, rel=1e-4)
    assert len(got_loss) == steps
    for a, b in zip(got_loss, want_loss):
        assert a == pytest.approx(b, rel=1e-4, abs=1e-4)
    if clip < 5.0:
        assert any(clipped) and not all(clipped), "pick the threshold so that both branches of the clipping run: %s" % (
            want_norms if mode == "whole" else clipped)
    new = _read_model(str(model) + ".trained", n_head, L, H, Vs, Vt, lm)
    _compare("D", new["D"], m["D"], orig["D"])
    _compare("b_d", new["b_d"], m["b_d"], orig["b_d"])
    for s, key in (("t", "tgt_layers"),) + (() if lm else (("s", "src_layers"),)):
        _compare("embedding " + s, new["emb_" + s], m["emb_" + s], orig["emb_" + s])
        for l in range(L):
            for k in ("M", "Wh", "b"):
                for gate in range(4):
                    _compare("%s layer %d %s[%d]" % (key, l, k, gate), new[key][l][k][gate], m[key][l][k][gate],
                             orig[key][l][k][gate])


@pytest.mark.parametrize("node_level", [False, True])
@pytest.mark.parametrize("mode,lm,L,H,mb,steps,clip", [("whole", False, 2, 48, 3, 3, 3.5), ("whole", True, 2, 32, 4, 2, 1e3),
                                                       ("element", False, 2, 48, 3, 2, 0.02),
                                                       ("element", True, 1, 32, 5, 2, 0.05)])
def test_train_steps_with_whole_model_and_element_clipping(tmp_path, mode, lm, L, H, mb, steps, clip, node_level):
    """The reference's other two clipping modes (src/main.cu:495-511) through both training paths: norm_clip bounding
    the norm of ALL gradients together (the first case clips in some steps and not in others, the second never), and a
    clamp of every gradient element.  In whole-model mode the norm the driver reports is compared too."""
    test_train_steps_match_oracle(tmp_path, lm, L, H, mb, steps, clip, node_level, mode=mode)


@pytest.mark.parametrize("lm,L,H,mb,steps,cell", [(False, 2, 48, 3, 2, (0.2, 0.004)), (True, 3, 32, 4, 1, (0.15, 0.002))])
def test_train_steps_with_cell_and_error_clamps(tmp_path, lm, L, H, mb, steps, cell):
    """--clip-cell (src/main.cu:399-405): the cell clamped in the forward pass, and the errors sent to h_{t-1} and to the
    layer below clamped in the backward pass, through the node classes (model_trainer hands such models to them).  The
    thresholds are low enough to act: the same steps without them end at weights that differ by far more than the
    tolerance (checked on the oracle)."""
    test_train_steps_match_oracle(tmp_path, lm, L, H, mb, steps, 5.0, False, cell=cell)
    test_train_steps_match_oracle(tmp_path, lm, L, H, mb, steps, 5.0, True, cell=cell)


def test_repeated_steps_on_one_minibatch_raise_its_likelihood(tmp_path):
    """Property check without the oracle: gradient ASCENT on the log-likelihood, so training on the same minibatch
    again and again must raise it."""
    g = synth.rng(132, 0)
    H, L, mb = 64, 2, 6
    tgt_vocab = ["<START>", "<EOF>", "<UNK>"] + mf.make_vocab(80, "w")
    Vt = len(tgt_vocab)
    m = {"emb_t": synth.uniform(g, (H, Vt), -0.1, 0.1),
         "tgt_layers": [synth.lstm_layer(g, H, forget_bias_one=True) for _ in range(L)],
         "D": synth.uniform(g, (Vt, H), -0.1, 0.1), "b_d": synth.uniform(g, (Vt,), -0.1, 0.1)}
    model = tmp_path / "lm.nn"
    _write_model(model, m, tgt_vocab, [], True)
    data = mf.integerize_targets(mf.random_sentences(g, tgt_vocab, mb, 3, 9), tgt_vocab, mb)
    with open(tmp_path / "data.int", "w") as f:
        for d in data:
            f.write("\n\n" + " ".join(map(str, d[0])) + "\n" + " ".join(map(str, d[1])) + "\n")
    r = subprocess.run([DRIVER, "--sequence", str(model), str(tmp_path / "data.int"), str(mb), "16", "0.2", "5", "12"],
                       capture_output=True, text=True, timeout=300)
    assert r.returncode == 0, r.stderr[-2000:]
    loss = [float(ln.split()[2]) for ln in r.stdout.splitlines() if ln.startswith("loss")]
    assert len(loss) == 12 and all(b > a for a, b in zip(loss, loss[1:])), [round(v, 2) for v in loss]
    assert loss[-1] > loss[0] + 0.1 * abs(loss[0])


@pytest.mark.parametrize("lm,L", [(False, 2), (True, 1)])
def test_model_file_dumped_by_the_layer_objects_reads_back_under_the_reference_scripts_layout(tmp_path, lm, L):
    """The C++ side's writer (forward_model::dump_weights -> the layers' dump_weights members) against the second
    description of the format, the reference's own Python reader restated in model_files_util.parse_like_reference_script:
    a model is loaded and dumped again without a training step (steps = 0)."""
    if not os.path.exists(DRIVER):
        pytest.fail("tests/host/train_step is not built: run `python __graft_entry__.py build`")
    g = synth.rng(133, L)
    H, mb = 16, 2
    src_vocab = ["<UNK>"] + mf.make_vocab(12, "s")
    tgt_vocab = ["<START>", "<EOF>", "<UNK>"] + mf.make_vocab(14, "t")
    Vs, Vt = len(src_vocab), len(tgt_vocab)
    m = {"emb_t": synth.uniform(g, (H, Vt)), "tgt_layers": [synth.lstm_layer(g, H, forget_bias_one=True) for _ in range(L)],
         "D": synth.uniform(g, (Vt, H)), "b_d": synth.uniform(g, (Vt,))}
    if not lm:
        m["emb_s"] = synth.uniform(g, (H, Vs))
        m["src_layers"] = [synth.lstm_layer(g, H) for _ in range(L)]
    model = tmp_path / "model.nn"
    _write_model(model, m, tgt_vocab, src_vocab, lm)
    data = tmp_path / "data.int"
    data.write_text("")
    args = (["--sequence"] if lm else []) + [str(model), str(data), str(mb), "8", "0.5", "5", "0"]
    r = subprocess.run([DRIVER] + args, capture_output=True, text=True, timeout=120)
    assert r.returncode == 0, r.stderr[-2000:]
    head, sv, tv, sl, tl, D, b = mf.parse_like_reference_script(str(model) + ".trained")
    assert head[:4] == [L, H, Vt, 0 if lm else Vs]
    assert tv == dict(enumerate(tgt_vocab))
    if not lm:
        assert sv == dict(enumerate(src_vocab))
        mf.check_layers_against_script_reading(m["src_layers"], m["emb_s"], sl)
    mf.check_layers_against_script_reading(m["tgt_layers"], m["emb_t"], tl)
    assert np.allclose(D, m["D"], rtol=1e-6, atol=0) and np.allclose(b.reshape(-1), m["b_d"], rtol=1e-6, atol=0)
