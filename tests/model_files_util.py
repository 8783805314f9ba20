"""Shared by the model-file / force-decode tests: a Python restatement of the reference's data preparation
(independent of the C++ one in zoph_rnn_amd/host/zoph_model.h) and writers for synthetic model files.

Reference formats: model header and vocabulary blocks src/input_file_prep.h:304-357 + src/add_model_info.h:7-23;
integerization src/input_file_prep.h:403-500 (pairs) and :1590-1670 (sequence model); matrix text layout
src/Eigen_Util.h:148-163; file order src/model.hpp:2058-2070."""
import os
import subprocess

import numpy as np

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
FORCE_DECODE = os.path.join(ROOT, "zoph_rnn_amd", "host", "force_decode")
SEP = "=" * 58


def ensure_force_decode():
    if not os.path.exists(FORCE_DECODE):
        from zoph_rnn_amd import build
        build.build_force_decode()
    return FORCE_DECODE


def make_vocab(n, prefix):
    return ["%s%d" % (prefix, i) for i in range(n)]


def write_header(f, L, H, tgt_vocab, src_vocab, attention, feed_input, lm=False):
    f.write("%d %d %d %d %d %d 0 0 0\n" % (L, H, len(tgt_vocab), 0 if lm else len(src_vocab), int(attention),
                                           int(feed_input)))
    f.write(SEP + "\n")
    if not lm:
        for i, w in enumerate(src_vocab):
            f.write("%d %s\n" % (i, w))
        f.write(SEP + "\n")
    for i, w in enumerate(tgt_vocab):
        f.write("%d %s\n" % (i, w))
    f.write(SEP + "\n")


def integerize_pairs(src_sents, tgt_sents, src_vocab, tgt_vocab, minibatch):
    """Returns a list of (src, minus_two, tgt_in, tgt_out) integer lists, padded per minibatch."""
    smap = {w: i for i, w in enumerate(src_vocab)}
    tmap = {w: i for i, w in enumerate(tgt_vocab)}
    data = []
    for s, t in zip(src_sents, tgt_sents):
        si = [smap.get(w, smap["<UNK>"]) for w in s][::-1]
        ti = [tmap.get(w, tmap["<UNK>"]) for w in t]
        data.append([si, [-2] * len(si), [0] + ti, ti + [1]])
    for base in range(0, len(data), minibatch):
        chunk = data[base:base + minibatch]
        ms, mt = max(len(d[0]) for d in chunk), max(len(d[2]) for d in chunk)
        for d in chunk:
            pad = ms - len(d[0])
            d[0] = [-1] * pad + d[0]
            d[1] = [-1] * pad + d[1]
            d[2] = d[2] + [-1] * (mt - len(d[2]))
            d[3] = d[3] + [-1] * (mt - len(d[3]))
    return data


def integerize_targets(tgt_sents, tgt_vocab, minibatch):
    tmap = {w: i for i, w in enumerate(tgt_vocab)}
    data = []
    for t in tgt_sents:
        ti = [tmap.get(w, tmap["<UNK>"]) for w in t]
        data.append([[0] + ti, ti + [1]])
    for base in range(0, len(data), minibatch):
        chunk = data[base:base + minibatch]
        mt = max(len(d[0]) for d in chunk) + 1  # the reference pads `while size <= max`
        for d in chunk:
            d[0] = d[0] + [-1] * (mt - len(d[0]))
            d[1] = d[1] + [-1] * (mt - len(d[1]))
    return data


def read_int_file(path):
    lines = open(path).read().split("\n")
    if lines and lines[-1] == "":
        lines.pop()
    assert len(lines) % 4 == 0
    return [[[int(x) for x in lines[i + k].split()] for k in range(4)] for i in range(0, len(lines), 4)]


def run_force_decode(args, timeout=300):
    exe = ensure_force_decode()
    return subprocess.run([exe] + [str(a) for a in args], capture_output=True, text=True, timeout=timeout)


def run_program(name, args, timeout=300, env=None):
    """Runs zoph_rnn_amd/host/<name> (built by `python __graft_entry__.py build`); env: extra environment variables."""
    exe = os.path.join(ROOT, "zoph_rnn_amd", "host", name)
    assert os.path.exists(exe), "%s is not built: run `python __graft_entry__.py build`" % exe
    full_env = None
    if env:
        full_env = dict(os.environ)
        full_env.update({k: str(v) for k, v in env.items()})
    return subprocess.run([exe] + [str(a) for a in args], capture_output=True, text=True, timeout=timeout, env=full_env)


def random_sentences(g, vocab, n, min_len, max_len, oov_rate=0.1, oov_prefix="oov"):
    out = []
    for _ in range(n):
        k = int(g.integers(min_len, max_len + 1))
        words = []
        for _ in range(k):
            if g.random() < oov_rate:
                words.append("%s%d" % (oov_prefix, int(g.integers(0, 5))))
            else:
                words.append(vocab[int(g.integers(3, len(vocab)))])
        out.append(words)
    return out


def parse_like_reference_script(path):
    """A second, independent reading of a model file: the steps of the reference's own Python reader for models without
    attention (scripts/load_model.py:8-20 read_matrix -- `rows` lines of numbers, then one empty line; :53-67 and
    :121-135 the matrix order of the two layer kinds; :184-186 the loss layer; :264-277 a vocabulary block runs to the
    next line that starts with "==="; :289-334 header, one separator line, source vocabulary unless the model is a
    sequence model, target vocabulary, source layers, target layers, loss layer).  The script keys "sequence model" on
    a three-field header; the current header always has nine fields and a zero source vocabulary instead.
    Returns (header ints, source vocab or None, target vocab, source layers or None, target layers, D, b) with every layer
    a dict of the script's parameter names."""
    f = open(path)
    head = [int(x) for x in f.readline().split()]
    L, H, Vt, Vs = head[0], head[1], head[2], head[3]
    lm = Vs == 0
    f.readline()

    def vocab():
        out = {}
        while True:
            line = f.readline()
            assert line, "file ended inside a vocabulary block"
            if line.startswith("==="):
                return out
            idx, word = line.split()
            out[int(idx)] = word

    def matrix(rows, cols):
        m = np.zeros((rows, cols))
        for i in range(rows):
            vals = [float(x) for x in f.readline().split()]
            assert len(vals) == cols, "row of %d numbers where %d were expected" % (len(vals), cols)
            m[i] = vals
        assert f.readline().strip() == "", "a matrix must be followed by an empty line"
        return m

    def layer(V):
        names = ["w_hi", "b_i", "w_hf", "b_f", "w_hc", "b_c", "w_ho", "b_o"] + (["w"] if V else []) + \
                ["m_i", "m_f", "m_o", "m_c"]
        out = {}
        for nme in names:
            out[nme] = matrix(H, V if nme == "w" else (1 if nme.startswith("b_") else H))
        return out

    src_vocab = None if lm else vocab()
    tgt_vocab = vocab()
    src_layers = None if lm else [layer(Vs)] + [layer(0) for _ in range(L - 1)]
    tgt_layers = [layer(Vt)] + [layer(0) for _ in range(L - 1)]
    D, b = matrix(Vt, H), matrix(Vt, 1)
    assert f.read().strip() == "", "data left after the loss layer"
    return head, src_vocab, tgt_vocab, src_layers, tgt_layers, D, b


def check_layers_against_script_reading(layers_np, embed, parsed_layers):
    """layers_np: the dictionaries the writers take (gate order i, f, c, o); parsed_layers: parse_like_reference_script's."""
    gate = {"i": 0, "f": 1, "c": 2, "o": 3}
    for l, (ly, got) in enumerate(zip(layers_np, parsed_layers)):
        for g, k in gate.items():
            assert np.allclose(got["w_h" + g], ly["Wh"][k], rtol=1e-6, atol=0), (l, "w_h" + g)
            assert np.allclose(got["m_" + g], ly["M"][k], rtol=1e-6, atol=0), (l, "m_" + g)
            assert np.allclose(got["b_" + g].reshape(-1), ly["b"][k], rtol=1e-6, atol=0), (l, "b_" + g)
        if l == 0:
            assert np.allclose(got["w"], embed, rtol=1e-6, atol=0)
