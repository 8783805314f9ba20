"""Writes the golden fixtures of this directory: small seeded inputs of every hot-path stage together with what the
CPU oracle (oracle/libzoph_oracle.so, double accumulation) makes of them.

The reference ships no expected outputs for this path (sample_data/ holds raw text only) and none of it can be
compiled or imported here, so these vectors come from the oracle and serve two purposes: they freeze the oracle (a
change to it that moves a result fails tests/test_golden_fixtures.py on the CPU), and they give the GPU tests inputs and
expected outputs that do not depend on the oracle being built on the GPU box.

Run from the repository root:  python tests/golden/make_fixtures.py
Each fixture is one .npz (numpy arrays only, loaded with allow_pickle=False).
"""
import os
import sys

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.dirname(HERE))
sys.path.insert(0, os.path.dirname(os.path.dirname(HERE)))
import oracle_lib as o  # noqa: E402
from zoph_rnn_amd import synth  # noqa: E402

U = synth.uniform


def lstm_fixture():
    """Two stacked decoder nodes with feed-input on the lower one, a masked column, cell clipping, H % 32 != 0."""
    g = synth.rng(2024, 1)
    H, mb, V = 40, 7, 23
    embed = U(g, (H, V), -1, 1)
    ids = g.integers(0, V, size=mb).astype(np.int32)
    ids[2] = ids[1]
    mask = np.ones(mb, np.int32)
    mask[3] = 0
    out = {"embed": embed, "ids": ids, "mask": mask, "clip": np.float32(0.8)}
    x = o.embed_gather(embed, ids)
    for l in range(2):
        ly = synth.lstm_layer(g, H, feed_input=(l == 0), forget_bias_one=True)
        hp, cp = U(g, (H, mb), -1, 1), U(g, (H, mb), -1, 1)
        ht = U(g, (H, mb), -1, 1) if l == 0 else None
        r = o.lstm_step(ly["M"], ly["Wh"], ly["b"], x, hp, cp, mask, Q=ly.get("Q"), htild=ht, clip=0.8)
        for k in ("M", "Wh", "Q"):
            if k in ly:
                for gi, m in enumerate(ly[k]):
                    out["l%d_%s%d" % (l, k, gi)] = m
        for gi, b in enumerate(ly["b"]):
            out["l%d_b%d" % (l, gi)] = b
        out["l%d_hprev" % l], out["l%d_cprev" % l] = hp, cp
        if ht is not None:
            out["l%d_htild" % l] = ht
        out["l%d_h" % l], out["l%d_c" % l] = r["h"], r["c"]
        x = r["h"]
    return out


def attention_fixture():
    """Local-p attention with ragged source lengths, a masked column and a window shorter than the longest source."""
    g = synth.rng(2024, 2)
    H, mb, S, D = 36, 6, 9, 2
    w = synth.attention_weights(g, H)
    for k in ("W_a", "W_p", "W_c1", "W_c2"):
        w[k] = U(g, (H, H), -0.3, 0.3)
    hs = (g.standard_normal(size=(S, H, mb)) * 0.5).astype(np.float32)
    lens = np.array([9, 4, 7, 1, 9, 6], np.int32)
    binfo = np.concatenate([lens, S - lens]).astype(np.int32)
    mask = np.array([1, 1, 0, 1, 1, 1], np.int32)
    h_t = U(g, (H, mb), -1, 1)
    r = o.attention_forward(hs_table=hs, batch_info=binfo, h_t=h_t, mask01=mask, D=D, **w)
    out = dict(w)
    out.update({"hs": hs, "batch_info": binfo, "mask": mask, "h_t": h_t, "D": np.int32(D)})
    for k in ("h_tild", "alignments", "indices", "p_t", "c_ctx"):
        out["out_" + k] = r[k]
    return out


def softmax_fixture():
    """Output layer: logits, probabilities, double log-probabilities and the masked loss; V % 32 != 0."""
    g = synth.rng(2024, 3)
    V, H, mb = 211, 24, 5
    Dm, bd, h = U(g, (V, H), -1, 1), U(g, (V,), -1, 1), U(g, (H, mb), -1, 1)
    logits = o.softmax_logits(Dm, bd, h)
    tgt = g.integers(0, V, size=mb).astype(np.int32)
    mask = np.array([1, 0, 1, 1, 1], np.int32)
    logp = o.softmax_logprob_f64(logits)
    return {"D": Dm, "b_d": bd, "h": h, "target": tgt, "mask": mask, "logits": logits, "prob": o.softmax_dist(logits),
            "logprob": logp, "loss": np.float64(o.softmax_loss(logp, tgt, mask))}


def beam_fixture():
    """Five expansion steps and the forced finish of one sentence, beam 4, with <EOF> made likely and a word penalty."""
    g = synth.rng(2024, 4)
    V, beam, steps, max_len = 37, 4, 5, 9
    dec = o.Decoder(beam, V, max_len, penalty=0.25)
    probs, words, backs, scores = [], [], [], []
    for index in range(steps + 1):
        lg = g.standard_normal(size=(V, beam)) * 2.0
        lg[1, :] += 3.0
        e = np.exp(lg - lg.max(axis=0))
        P = np.asfortranarray((e / e.sum(axis=0)).astype(np.float32))
        probs.append(P)
        if index == steps:
            dec.finish(P)
            break
        dec.expand(P, index)
        st = dec.state()
        words.append(st["current_indices"].copy())
        backs.append(st["new_indicies_changes"].copy())
        scores.append(st["scores"].copy())
    hyps = dec.hypotheses()
    width = max(len(wd) for wd, _ in hyps)
    hw = np.full((len(hyps), width), -1, np.int32)
    for i, (wd, _) in enumerate(hyps):
        hw[i, :len(wd)] = wd
    return {"prob": np.stack(probs), "words": np.stack(words), "backptr": np.stack(backs), "scores": np.stack(scores),
            "hyp_words": hw, "hyp_scores": np.array([s for _, s in hyps], np.float32), "beam": np.int32(beam),
            "max_len": np.int32(max_len), "penalty": np.float32(0.25)}


def beam_viterbi_fixture():
    """The same decode with the attention layer's Viterbi alignment of every column handed to each step (unk
    replacement): the alignments every finished hypothesis ends up with."""
    g = synth.rng(2024, 5)
    V, beam, steps, max_len = 41, 5, 6, 10
    dec = o.Decoder(beam, V, max_len, penalty=0.1)
    probs, vits = [], []
    for index in range(steps + 1):
        lg = g.standard_normal(size=(V, beam)) * 2.0
        lg[1, :] += 2.5
        e = np.exp(lg - lg.max(axis=0))
        P = np.asfortranarray((e / e.sum(axis=0)).astype(np.float32))
        vit = g.integers(0, 30, size=beam).astype(np.int32)
        probs.append(P)
        vits.append(vit)
        if index == steps:
            dec.finish(P, vit)
        else:
            dec.expand(P, index, vit)
    hyps, hv = dec.hypotheses(), dec.hypotheses_viterbi()
    width = max(len(wd) for wd, _ in hyps)
    hw = np.full((len(hyps), width), -1, np.int32)
    hvit = np.full((len(hyps), width), -1, np.int32)
    for i, ((wd, _), v) in enumerate(zip(hyps, hv)):
        hw[i, :len(wd)] = wd
        hvit[i, :len(v)] = v
    return {"prob": np.stack(probs), "viterbi": np.stack(vits), "hyp_words": hw, "hyp_viterbi": hvit,
            "hyp_len": np.array([len(wd) for wd, _ in hyps], np.int32), "beam": np.int32(beam),
            "max_len": np.int32(max_len), "penalty": np.float32(0.1)}


def backward_clamped_fixture():
    """Back-propagation through a two-layer stack with the cell clamp and the error clamps of --clip-cell acting
    (thresholds far below the values they meet): gradients of one recurrent and one input matrix, the embedding
    gradient and the errors of the initial states."""
    g = synth.rng(2024, 6)
    L, H, mb, T, V = 2, 12, 4, 5, 15
    embed = U(g, (H, V), -0.5, 0.5)
    layers = [synth.lstm_layer(g, H) for _ in range(L)]
    for ly in layers:
        ly["M"] = [U(g, (H, H), -0.6, 0.6) for _ in range(4)]
        ly["Wh"] = [U(g, (H, H), -0.6, 0.6) for _ in range(4)]
    ids = g.integers(0, V, size=(T, mb)).astype(np.int32)
    ids[0, 2] = -1
    nn, mask = o.vocab_prep(ids)
    h0 = [U(g, (H, mb), -0.5, 0.5) for _ in range(L)]
    c0 = [U(g, (H, mb), -0.9, 0.9) for _ in range(L)]
    err_top = [U(g, (H, mb), -1, 1) for _ in range(T)]
    grads, d_embed, eh0, ec0 = o.lstm_stack_backward(embed, layers, nn, mask, err_top, h0, c0, cell_clip=0.35,
                                                     err_clip=0.08)
    out = {"embed": embed, "ids": ids, "err_top": np.stack(err_top), "h0": np.stack(h0), "c0": np.stack(c0),
           "cell_clip": np.float32(0.35), "err_clip": np.float32(0.08), "d_embed": d_embed,
           "err_h0": np.stack(eh0), "err_c0": np.stack(ec0)}
    for l, ly in enumerate(layers):
        for k in ("M", "Wh", "b"):
            for q in range(4):
                out["l%d_%s%d" % (l, k, q)] = ly[k][q]
        out["l%d_dWh0" % l] = grads[l]["dWh"][0]
        out["l%d_dM2" % l] = grads[l]["dM"][2]
        out["l%d_db3" % l] = grads[l]["db"][3]
    return out


FIXTURES = {"lstm_two_layers": lstm_fixture, "attention_local_p": attention_fixture, "softmax_output_layer": softmax_fixture,
            "beam_one_sentence": beam_fixture, "beam_viterbi_one_sentence": beam_viterbi_fixture,
            "lstm_stack_backward_clamped": backward_clamped_fixture}

if __name__ == "__main__":
    for name, fn in FIXTURES.items():
        path = os.path.join(HERE, name + ".npz")
        np.savez_compressed(path, **fn())
        print(path, os.path.getsize(path), "bytes")
