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


def run_program(name, args, timeout=300):
    """Runs zoph_rnn_amd/host/<name> (built by `python __graft_entry__.py build`)."""
    exe = os.path.join(ROOT, "zoph_rnn_amd", "host", name)
    assert os.path.exists(exe), "%s is not built: run `python __graft_entry__.py build`" % exe
    return subprocess.run([exe] + [str(a) for a in args], capture_output=True, text=True, timeout=timeout)


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
