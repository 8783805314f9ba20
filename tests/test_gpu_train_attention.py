"""Training steps of attention models (with feed-input, with dropout) through forward_model::compute_gradients -- the
layer objects' own back_prop members in the reference's node-by-node order, tests/host/train_step --node-level --
against the same steps composed from the oracle's node functions in numpy: forward over the (layer, time) grid,
the loss layer's error per step, attention backward, node backward with the feed-input error handed to the previous
step's attention node, the source-state errors arriving at the encoder's top layer, 1/minibatch scaling, per-matrix
norm clipping and the ascent update.  The oracle's backward functions are pinned by torch autograd in
tests/test_oracle_backward_pins.py.  Dropout masks are the library's own uniform numbers, fetched through the C-ABI
with the (seed, call) the layers use.  Tolerance: 1e-4 of the largest weight change of each matrix plus 1e-6."""
import os
import subprocess

import numpy as np
import pytest

import model_files_util as mf
import oracle_lib as o
from test_gpu_force_decode import _time_major
from test_gpu_host_layers import _write_hh, _write_ih, _write_matrix
from test_gpu_train_step import _clip_update, _compare
from zoph_rnn_amd import capi, synth

pytestmark = pytest.mark.gpu
DRIVER = os.path.join(mf.ROOT, "tests", "host", "train_step")
F64 = lambda a: np.asarray(a, np.float64)
GATES = ("i", "f", "c_tilde", "o")
# stream numbers of the dropout masks (BZ_CUDA::DROPOUT_STREAM_* in zoph_rnn_amd/host/zoph_layers.h)
SRC_IN, TGT_IN, SRC_HID, TGT_HID, ATT = 1, 2, 16, 48, 96


class Masks:
    """The uniform numbers the layers draw for node `index` of a stream in minibatch number `step`."""

    def __init__(self, ctx, seed, H, mb, rate):
        self.ctx, self.seed, self.H, self.mb, self.rate, self.step = ctx, seed, H, mb, rate, 0

    def apply(self, stream, index, x):
        if self.rate >= 1.0:
            return x
        d = self.ctx.empty((self.H, self.mb))
        self.ctx.uniform_fill(self.seed + self.step, (stream << 24) | index, d, self.H * self.mb)
        self.ctx.sync()
        return o.dropout(d.get(), self.rate, x)


def _node_forward(ly, x, hp, cp, mask, htild=None):
    r = o.lstm_step(ly["M"], ly["Wh"], ly["b"], x, hp, cp, mask, Q=ly.get("Q") if htild is not None else None,
                    htild=htild)
    return {"x": x, "hp": hp, "cp": cp, "htild": htild, "out": r}


def _node_backward(ly, nd, mask, err_h, err_c_next, g):
    """Returns (err_hprev, err_cprev, err_below, err_htild or None); accumulates the node's weight gradients into g."""
    dg, err_cp = o.lstm_step_backward({k: nd["out"][k] for k in GATES}, nd["out"]["c"], nd["cp"], mask, err_h, err_c_next)
    d = [F64(dg[k]) for k in ("i", "f", "c", "o")]
    err_hp = sum(F64(ly["Wh"][k]).T @ d[k] for k in range(4))
    err_below = sum(F64(ly["M"][k]).T @ d[k] for k in range(4))
    for k in range(4):
        g["M"][k] += d[k] @ F64(nd["x"]).T
        g["Wh"][k] += d[k] @ F64(nd["hp"]).T
        g["b"][k] += d[k].sum(axis=1)
    err_ht = None
    if nd["htild"] is not None:
        err_ht = sum(F64(ly["Q"][k]).T @ d[k] for k in range(4))
        for k in range(4):
            g["Q"][k] += d[k] @ F64(nd["htild"]).T
    return err_hp.astype(np.float32), err_cp, err_below.astype(np.float32), err_ht


def _zero_grads(ly, H):
    g = {"M": [np.zeros((H, H)) for _ in range(4)], "Wh": [np.zeros((H, H)) for _ in range(4)],
         "b": [np.zeros(H) for _ in range(4)]}
    if "Q" in ly:
        g["Q"] = [np.zeros((H, H)) for _ in range(4)]
    return g


def _oracle_step(m, chunk, mb, lr, clip, clipped, D, longest, feed, masks, mode="matrix", norms=None):
    L, H = len(m["src_layers"]), m["emb_s"].shape[0]
    src, tin, tout = (_time_major([c[k] for c in chunk], mb) for k in (0, 2, 3))
    S, T = src.shape[0], tin.shape[0]
    lens = np.array([(src[:, b] != -1).sum() if b < len(chunk) else 1 for b in range(mb)], np.int32)
    binfo = np.concatenate([lens, S - lens]).astype(np.int32)
    nn_s, m_s = o.vocab_prep(src)
    nn_t, m_t = o.vocab_prep(tin)
    tgt, tmask, _ = o.vocab_softmax(tout)
    zero = np.zeros((H, mb), np.float32, order="F")
    # ---- forward
    enc = [[None] * S for _ in range(L)]
    for t in range(S):
        x = masks.apply(SRC_IN, t, o.embed_gather(m["emb_s"], nn_s[t]))
        for l in range(L):
            if l > 0:
                x = masks.apply(SRC_HID + l - 1, t, enc[l - 1][t]["out"]["h"])
            hp = enc[l][t - 1]["out"]["h"] if t > 0 else zero
            cp = enc[l][t - 1]["out"]["c"] if t > 0 else zero
            enc[l][t] = _node_forward(m["src_layers"][l], x, hp, cp, m_s[t])
    table = np.zeros((longest, H, mb), np.float32)
    for t in range(S):
        table[t] = enc[L - 1][t]["out"]["h"]
    dec = [[None] * T for _ in range(L)]
    att = [None] * T
    loss = 0.0
    for t in range(T):
        x = masks.apply(TGT_IN, t, o.embed_gather(m["emb_t"], nn_t[t]))
        for l in range(L):
            if l > 0:
                x = masks.apply(TGT_HID + l - 1, t, dec[l - 1][t]["out"]["h"])
            hp = dec[l][t - 1]["out"]["h"] if t > 0 else enc[l][S - 1]["out"]["h"]
            cp = dec[l][t - 1]["out"]["c"] if t > 0 else enc[l][S - 1]["out"]["c"]
            ht = att[t - 1]["fwd"]["h_tild"] if (feed and l == 0 and t > 0) else None
            dec[l][t] = _node_forward(m["tgt_layers"][l], x, hp, cp, m_t[t], htild=ht)
        h_att = masks.apply(ATT, t, dec[L - 1][t]["out"]["h"])
        fwd = o.attention_forward(hs_table=table, batch_info=binfo, h_t=h_att, mask01=m_t[t], D=D, **m["attn"])
        frac = fwd["p_t"] - np.floor(fwd["p_t"])
        live = m_t[t] == 1
        assert np.all((frac[live] > 1e-4) & (frac[live] < 1 - 1e-4)), "p_t on an integer boundary; pick another seed"
        att[t] = {"h_att": h_att, "fwd": fwd}
        loss += o.softmax_loss(o.softmax_logprob_f64(o.softmax_logits(m["D"], m["b_d"], fwd["h_tild"])), tgt[t], tmask[t])
    # ---- backward, target side
    Vt = m["D"].shape[0]
    dD, dbd = np.zeros((Vt, H), np.float64, order="F"), np.zeros(Vt, np.float64)
    a = m["attn"]
    ag = {k: np.zeros((H, H), np.float32, order="F") for k in ("W_a", "W_p", "W_c1", "W_c2")}
    ag["v_p"], ag["bias"] = np.zeros(H, np.float32), np.zeros(H, np.float32)
    err_hs = np.zeros((longest, H, mb), np.float32)
    g_t = [_zero_grads(ly, H) for ly in m["tgt_layers"]]
    g_s = [_zero_grads(ly, H) for ly in m["src_layers"]]
    dW_t, dW_s = np.zeros(m["emb_t"].shape), np.zeros(m["emb_s"].shape)
    eh = [zero.copy() for _ in range(L)]
    ec = [zero.copy() for _ in range(L)]
    feed_err = None
    for t in range(T - 1, -1, -1):
        e, dD, dbd = o.softmax_backward(m["D"], m["b_d"], att[t]["fwd"]["h_tild"], tgt[t], tmask[t], dD, dbd)
        if feed_err is not None:
            e = (e + feed_err).astype(np.float32)
        err_above, err_hs, ag = o.attention_backward(a["W_a"], a["W_p"], a["v_p"], a["W_c1"], a["W_c2"], table, binfo,
                                                     att[t]["h_att"], m_t[t], att[t]["fwd"], e, D, grads=ag, err_hs=err_hs)
        err_above = masks.apply(ATT, t, err_above)
        feed_err = None
        for l in range(L - 1, -1, -1):
            err_h = (err_above + eh[l]).astype(np.float32)
            eh[l], ec[l], below, e_ht = _node_backward(m["tgt_layers"][l], dec[l][t], m_t[t], err_h, ec[l], g_t[l])
            if l > 0:
                err_above = masks.apply(TGT_HID + l - 1, t, below)
            else:
                below = masks.apply(TGT_IN, t, below)
                for b in range(mb):
                    if m_t[t][b] == 1:
                        dW_t[:, nn_t[t][b]] += below[:, b]
                if e_ht is not None:
                    feed_err = e_ht
    # ---- source side: starts from the errors the target side left at its first step; the attention layer's
    # source-state errors arrive at the top layer
    for t in range(S - 1, -1, -1):
        err_above = err_hs[t]
        for l in range(L - 1, -1, -1):
            err_h = (err_above + eh[l]).astype(np.float32)
            eh[l], ec[l], below, _ = _node_backward(m["src_layers"][l], enc[l][t], m_s[t], err_h, ec[l], g_s[l])
            if l > 0:
                err_above = masks.apply(SRC_HID + l - 1, t, below)
            else:
                below = masks.apply(SRC_IN, t, below)
                for b in range(mb):
                    if m_s[t][b] == 1:
                        dW_s[:, nn_s[t][b]] += below[:, b]
    # ---- update
    whole = None
    if mode == "whole":  # the norm of every gradient of the model together (src/model.hpp:1850-1892)
        sq = lambda x: (np.asarray(x, np.float64) ** 2).sum()
        ss = sq(dD) + sq(dbd) + sq(dW_t) + sq(dW_s) + sum(sq(ag[k]) for k in ("W_a", "W_p", "v_p", "bias", "W_c1", "W_c2"))
        for grads in (g_t, g_s):
            for gr in grads:
                ss += sum(sq(gr[k][q]) for k in gr for q in range(4))
        whole = np.sqrt(ss) / mb
        norms.append(whole)
    up = lambda W, g: _clip_update(W, g, mb, clip, lr, clipped, mode, whole)
    m["D"], m["b_d"] = up(m["D"], dD), up(m["b_d"], dbd)
    m["emb_t"], m["emb_s"] = up(m["emb_t"], dW_t), up(m["emb_s"], dW_s)
    for layers, grads in ((m["tgt_layers"], g_t), (m["src_layers"], g_s)):
        for ly, gr in zip(layers, grads):
            for k in gr:
                ly[k] = [up(ly[k][q], gr[k][q]) for q in range(4)]
    for k, gk in (("W_a", "W_a"), ("W_p", "W_p"), ("v_p", "v_p"), ("out_bias", "bias"), ("W_c1", "W_c1"), ("W_c2", "W_c2")):
        a[k] = up(a[k], ag[gk]).reshape(np.asarray(a[k]).shape)
    masks.step += 1
    return loss


def _write_model(path, m, tgt_vocab, src_vocab, feed):
    L, H = len(m["tgt_layers"]), m["emb_t"].shape[0]
    with open(path, "w") as f:
        mf.write_header(f, L, H, tgt_vocab, src_vocab, True, feed)
        _write_ih(f, m["src_layers"][0], m["emb_s"])
        for ly in m["src_layers"][1:]:
            _write_hh(f, ly)
        _write_ih(f, m["tgt_layers"][0], m["emb_t"], attn=m["attn"] if L == 1 else None)
        for i, ly in enumerate(m["tgt_layers"][1:]):
            _write_hh(f, ly, attn=m["attn"] if i == L - 2 else None)
        _write_matrix(f, m["D"])
        _write_matrix(f, m["b_d"].reshape(-1, 1))


def _read_model(path, n_head, L, H, Vs, Vt, feed):
    vals = np.array(" ".join(open(path).read().split("\n")[n_head:]).split(), dtype=np.float64)
    pos = [0]

    def take(r, c):
        x = vals[pos[0]:pos[0] + r * c].reshape(r, c)
        pos[0] += r * c
        return x

    def attn():
        a = {"W_a": take(H, H), "W_p": take(H, H), "v_p": take(H, 1).reshape(-1), "out_bias": take(H, 1).reshape(-1)}
        a["W_c1"], a["W_c2"] = take(H, H), take(H, H)
        return a

    def layer(V, q):
        ly = {"M": [None] * 4, "Wh": [None] * 4, "b": [None] * 4}
        for g in range(4):
            ly["Wh"][g] = take(H, H)
            ly["b"][g] = take(H, 1).reshape(-1)
        emb = take(H, V) if V else None
        for g in (0, 1, 3, 2):
            ly["M"][g] = take(H, H)
        if q:
            ly["Q"] = [None] * 4
            for g in (0, 1, 3, 2):
                ly["Q"][g] = take(H, H)
        return ly, emb

    m = {}
    first, m["emb_s"] = layer(Vs, False)
    m["src_layers"] = [first] + [layer(0, False)[0] for _ in range(L - 1)]
    first, m["emb_t"] = layer(Vt, feed)
    m["tgt_layers"] = [first]
    if L == 1:
        m["attn"] = attn()
    for i in range(L - 1):
        m["tgt_layers"].append(layer(0, False)[0])
        if i == L - 2:
            m["attn"] = attn()
    m["D"] = take(Vt, H)
    m["b_d"] = take(Vt, 1).reshape(-1)
    assert pos[0] == vals.size
    return m


@pytest.mark.parametrize("L,H,mb,D,feed,rate,steps,clip,trainer",
                         [(2, 32, 3, 2, True, 1.0, 1, 0.5, False), (1, 24, 4, 3, True, 1.0, 2, 5.0, False),
                          (2, 32, 3, 4, False, 1.0, 1, 5.0, False), (3, 40, 5, 2, True, 0.7, 2, 0.5, False),
                          (1, 24, 2, 2, False, 0.5, 1, 5.0, False), (2, 32, 3, 2, True, 0.8, 2, 0.5, True)])
def test_attention_model_train_steps_match_oracle(tmp_path, L, H, mb, D, feed, rate, steps, clip, trainer, mode="matrix"):
    """trainer: through model_trainer::train_minibatch, which hands attention / dropout models to the node-level path."""
    if not os.path.exists(DRIVER):
        pytest.fail("tests/host/train_step is not built: run `python __graft_entry__.py build`")
    g = synth.rng(141, L * 100 + H + mb)
    lr, longest, seed = 0.5, 16, 4242
    src_vocab = ["<UNK>"] + mf.make_vocab(40, "s")
    tgt_vocab = ["<START>", "<EOF>", "<UNK>"] + mf.make_vocab(50, "t")
    Vs, Vt = len(src_vocab), len(tgt_vocab)
    m = {"emb_s": synth.uniform(g, (H, Vs), -0.5, 0.5), "emb_t": synth.uniform(g, (H, Vt), -0.5, 0.5),
         "src_layers": [synth.lstm_layer(g, H, forget_bias_one=True) for _ in range(L)],
         "tgt_layers": [synth.lstm_layer(g, H, feed_input=(feed and l == 0), forget_bias_one=True) for l in range(L)],
         "attn": synth.attention_weights(g, H), "D": synth.uniform(g, (Vt, H), -0.5, 0.5),
         "b_d": synth.uniform(g, (Vt,), -0.5, 0.5)}
    for ly in m["src_layers"] + m["tgt_layers"]:
        for k in ("M", "Wh"):
            ly[k] = [synth.uniform(g, (H, H), -0.3, 0.3) for _ in range(4)]
    for k in ("W_a", "W_p", "W_c1", "W_c2"):
        m["attn"][k] = synth.uniform(g, (H, H), -0.3, 0.3)
    model = tmp_path / "model.nn"
    _write_model(model, m, tgt_vocab, src_vocab, feed)
    n_head = 1 + 3 + Vs + Vt
    orig = _read_model(model, n_head, L, H, Vs, Vt, feed)
    n_sent = 2 * mb
    src = mf.random_sentences(g, src_vocab, n_sent, 2, 9)
    tgt = mf.random_sentences(g, tgt_vocab, n_sent, 1, 8)
    data = mf.integerize_pairs(src, tgt, src_vocab, tgt_vocab, mb)
    data_path = tmp_path / "data.int"
    with open(data_path, "w") as f:
        for r in data:
            for k in range(4):
                f.write(" ".join(str(v) for v in r[k]) + "\n")
    args = ([] if trainer else ["--node-level"]) + (["--whole-clip"] if mode == "whole" else []) + ["--attention-D=%d" % D, "--dropout=%g" % rate, "--dropout-seed=%d" % seed, str(model),
            str(data_path), str(mb), str(longest), str(lr), str(clip), str(steps)]
    r = subprocess.run([DRIVER] + args, capture_output=True, text=True, timeout=300)
    assert r.returncode == 0, r.stderr[-2000:]
    got_loss = [float(ln.split()[2]) for ln in r.stdout.splitlines() if ln.startswith("loss")]
    ctx = capi.Context(0)
    try:
        masks = Masks(ctx, seed, H, mb, rate)
        chunks = [data[i:i + mb] for i in range(0, len(data), mb)]
        clipped, want_loss, want_norms = [], [], []
        for s in range(steps):
            want_loss.append(_oracle_step(m, chunks[s % len(chunks)], mb, lr, clip, clipped, D, longest, feed, masks, mode,
                                          want_norms))
    finally:
        ctx.close()
    if mode == "whole":
        got_norms = [float(ln.split()[2]) for ln in r.stdout.splitlines() if ln.startswith("global_norm")]
        assert got_norms == pytest.approx(want_norms, rel=1e-4)
        assert all(n > clip for n in want_norms), "the threshold should act: %s" % want_norms
    # the driver's loss line is the log-likelihood of the evaluation-mode forward pass (no dropout) before the update
    if rate >= 1.0:
        for x, y in zip(got_loss, want_loss):
            assert x == pytest.approx(y, rel=1e-4, abs=1e-4)
    if clip < 5.0 and mode == "matrix":
        assert any(clipped) and not all(clipped), "pick norm_clip so that both branches of the clipping run"
    new = _read_model(str(model) + ".trained", n_head, L, H, Vs, Vt, feed)
    _compare("D", new["D"], m["D"], orig["D"])
    _compare("b_d", new["b_d"], m["b_d"], orig["b_d"])
    for k in ("W_a", "W_p", "v_p", "out_bias", "W_c1", "W_c2"):
        _compare("attention " + k, new["attn"][k], m["attn"][k], orig["attn"][k])
    for s, key in (("t", "tgt_layers"), ("s", "src_layers")):
        _compare("embedding " + s, new["emb_" + s], m["emb_" + s], orig["emb_" + s])
        for l in range(L):
            for k in m[key][l]:
                for gate in range(4):
                    _compare("%s layer %d %s[%d]" % (key, l, k, gate), new[key][l][k][gate], m[key][l][k][gate],
                             orig[key][l][k][gate])


def test_attention_model_train_steps_with_whole_model_clipping(tmp_path):
    """--whole-clip-gradients on a feed-input attention model: the attention layer's six gradients and the Q matrices'
    take part in the model's norm (attention_layer::norm_p1 / norm_p2), which the driver reports."""
    test_attention_model_train_steps_match_oracle(tmp_path, 2, 32, 3, 2, True, 1.0, 2, 1.0, False, mode="whole")
