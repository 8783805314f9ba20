"""The C++ layer classes (zoph_rnn_amd/host/zoph_layers.h: same names and members as the reference's layer objects)
driven the way neuralMT_model::getError drives them, checked against the oracle.  Also covers the model-file text
layout (load_weights / dump_weights order and matrix format)."""
import os
import subprocess

import numpy as np
import pytest

import oracle_lib as o
from gpu_util import assert_close, round_bf16
from zoph_rnn_amd import synth

pytestmark = pytest.mark.gpu

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
DRIVER = os.path.join(ROOT, "tests", "host", "layers_forward")


def _write_matrix(f, m):
    m = np.atleast_2d(m)
    for row in m:
        f.write(" ".join("%.9g" % v for v in row) + "\n")
    f.write("\n")


def _write_ih(f, ly, embed, attn=None):
    """Input_To_Hidden_Layer::dump_weights_GPU order (reference: src/Input_To_Hidden_Layer.hpp:1050-1085)."""
    M, Wh, b = ly["M"], ly["Wh"], ly["b"]  # gate order i, f, c, o
    for g in (0, 1, 2, 3):
        _write_matrix(f, Wh[g])
        _write_matrix(f, b[g].reshape(-1, 1))
    _write_matrix(f, embed)
    for g in (0, 1, 3, 2):  # M_i, M_f, M_o, M_c
        _write_matrix(f, M[g])
    if "Q" in ly:
        for g in (0, 1, 3, 2):
            _write_matrix(f, ly["Q"][g])
    if attn is not None:
        _write_attn(f, attn)


def _write_hh(f, ly, attn=None):
    M, Wh, b = ly["M"], ly["Wh"], ly["b"]
    for g in (0, 1, 2, 3):
        _write_matrix(f, Wh[g])
        _write_matrix(f, b[g].reshape(-1, 1))
    for g in (0, 1, 3, 2):
        _write_matrix(f, M[g])
    if attn is not None:
        _write_attn(f, attn)


def _write_attn(f, a):
    """attention_layer::dump_weights order (reference: src/attention_layer.hpp:467-473)."""
    _write_matrix(f, a["W_a"])
    _write_matrix(f, a["W_p"])
    _write_matrix(f, a["v_p"].reshape(-1, 1))
    _write_matrix(f, a["out_bias"].reshape(-1, 1))
    _write_matrix(f, a["W_c1"])
    _write_matrix(f, a["W_c2"])


def _run_driver(tmp_path, weights_writer, ids_blocks, H, mb, V, L, S, T, D, bf16=False):
    if not os.path.exists(DRIVER):
        pytest.fail("tests/host/layers_forward is not built: run `python __graft_entry__.py build`")
    wpath, ipath = str(tmp_path / "model.nn"), str(tmp_path / "ids.txt")
    with open(wpath, "w") as f:
        weights_writer(f)
    with open(ipath, "w") as f:
        for blk in ids_blocks:
            f.write(" ".join(str(int(v)) for v in np.asarray(blk).reshape(-1)) + "\n")
    env = dict(os.environ, ZOPH_BF16_WEIGHTS="1" if bf16 else "0")
    out = subprocess.run([DRIVER, wpath, ipath] + [str(v) for v in (H, mb, V, L, S, T, D)], capture_output=True,
                         text=True, timeout=120, env=env)
    assert out.returncode == 0, out.stderr[-2000:]
    losses, hs = {}, {}
    for line in out.stdout.splitlines():
        p = line.split()
        if p[0] == "loss":
            losses[int(p[1])] = float(p[2])
        elif p[0] == "h":
            hs[int(p[1])] = np.array(p[2:], dtype=np.float32).reshape(H, mb, order="F")
        elif p[0] in ("dec_h", "swap_before", "swap_after"):
            hs[p[0]] = np.array(p[1:], dtype=np.float32).reshape(H, mb, order="F")
        elif p[0] == "viterbi":
            hs["viterbi"] = np.array(p[1:], dtype=np.int32)
    # dump_weights must reproduce the file it loaded (same order, same layout)
    dumped = np.array(open(wpath + ".dump").read().split(), dtype=np.float64)
    loaded = np.array(open(wpath).read().split(), dtype=np.float64)
    assert dumped.shape == loaded.shape and np.allclose(dumped, loaded, rtol=1e-6, atol=0)
    return losses, hs


def test_language_model_through_layer_classes(tmp_path):
    g = synth.rng(51, 1)
    H, mb, V, L, T = 48, 5, 120, 2, 6
    embed = synth.uniform(g, (H, V))
    layers = [synth.lstm_layer(g, H, forget_bias_one=True) for _ in range(L)]
    Dm, bd = synth.uniform(g, (V, H)), synth.uniform(g, (V,))
    tin = g.integers(0, V, size=(T, mb)).astype(np.int32)
    tout = g.integers(0, V, size=(T, mb)).astype(np.int32)
    tin[4:, 2] = -1  # target side pads at the end
    tout[4:, 2] = -1

    def writer(f):
        _write_ih(f, layers[0], embed)
        for ly in layers[1:]:
            _write_hh(f, ly)
        _write_matrix(f, Dm)
        _write_matrix(f, bd.reshape(-1, 1))

    losses, hs = _run_driver(tmp_path, writer, [[], tin, tout, np.zeros(2 * mb, np.int32)], H, mb, V, L, 0, T, 0)
    nn, m = o.vocab_prep(tin)
    want_h, _ = o.lstm_stack_forward(embed, layers, nn, m)
    tgt, tmask, _ = o.vocab_softmax(tout)
    for t in range(T):
        assert_close(hs[t], want_h[L - 1, t], what="top h step %d" % t)
        lp = o.softmax_logprob_f64(o.softmax_logits(Dm, bd, np.asfortranarray(want_h[L - 1, t])))
        assert losses[t] == pytest.approx(o.softmax_loss(lp, tgt[t], tmask[t]), rel=1e-5, abs=1e-6)


@pytest.mark.parametrize("L,bf16", [(1, False), (3, False), (2, True)])
def test_seq2seq_attention_feed_input_through_layer_classes(tmp_path, L, bf16):
    """bf16: BZ_CUDA::bf16_weights set in the driver (every streamed matrix snapshotted as bf16), weights in the file
    already bf16-representable, bf16 tolerance (1e-4 relative, floor 0.25; 1e-4 absolute behind the attention)."""
    g = synth.rng(52, L)
    H, mb, V, S, T, D = (48 if bf16 else 40), 4, 90, 7, 5, 3
    emb_s, emb_t = synth.uniform(g, (H, V)), synth.uniform(g, (H, V))
    src_layers = [synth.lstm_layer(g, H, forget_bias_one=True) for _ in range(L)]
    tgt_layers = [synth.lstm_layer(g, H, feed_input=(l == 0), forget_bias_one=True) for l in range(L)]
    attn = synth.attention_weights(g, H)
    for k in ("W_a", "W_p", "W_c1", "W_c2"):
        attn[k] = synth.uniform(g, (H, H), -0.3, 0.3)
    Dm, bd = synth.uniform(g, (V, H)), synth.uniform(g, (V,))
    if bf16:
        rb = lambda m: np.asfortranarray(round_bf16(m))
        for ly in src_layers + tgt_layers:
            for k in ("M", "Wh", "Q"):
                if k in ly:
                    ly[k] = [rb(m) for m in ly[k]]
        for k in ("W_a", "W_p", "W_c1", "W_c2"):
            attn[k] = rb(attn[k])
        Dm = rb(Dm)
    lens = np.array([7, 5, 7, 2], np.int32)
    src = g.integers(0, V, size=(S, mb)).astype(np.int32)
    for b in range(mb):
        src[:S - lens[b], b] = -1  # source is left padded
    tin = g.integers(0, V, size=(T, mb)).astype(np.int32)
    tout = g.integers(0, V, size=(T, mb)).astype(np.int32)
    tin[3:, 1] = -1
    tout[3:, 1] = -1
    binfo = np.concatenate([lens, S - lens]).astype(np.int32)

    def writer(f):
        _write_ih(f, src_layers[0], emb_s)
        for ly in src_layers[1:]:
            _write_hh(f, ly)
        _write_ih(f, tgt_layers[0], emb_t, attn if L == 1 else None)
        for i, ly in enumerate(tgt_layers[1:]):
            _write_hh(f, ly, attn if i == L - 2 else None)
        _write_matrix(f, Dm)
        _write_matrix(f, bd.reshape(-1, 1))

    losses, hs = _run_driver(tmp_path, writer, [src, tin, tout, binfo], H, mb, V, L, S, T, D, bf16=bf16)

    # oracle: source sweep, then the target sweep with attention on the top layer and feed-input into layer 0
    nn_s, m_s = o.vocab_prep(src)
    hs_src, cs_src = o.lstm_stack_forward(emb_s, src_layers, nn_s, m_s)
    longest = max(S, T)
    table = np.zeros((longest, H, mb), np.float32)
    table[:S] = hs_src[L - 1]
    nn_t, m_t = o.vocab_prep(tin)
    tgt, tmask, _ = o.vocab_softmax(tout)
    hp = [np.asfortranarray(hs_src[l, S - 1]) for l in range(L)]
    cp = [np.asfortranarray(cs_src[l, S - 1]) for l in range(L)]
    h_tild_prev = None
    for t in range(T):
        below = o.embed_gather(emb_t, nn_t[t])
        for l in range(L):
            ly = tgt_layers[l]
            feed = (l == 0 and t > 0)
            r = o.lstm_step(ly["M"], ly["Wh"], ly["b"], below, hp[l], cp[l], m_t[t], Q=ly["Q"] if feed else None,
                            htild=h_tild_prev if feed else None)
            hp[l], cp[l], below = r["h"], r["c"], r["h"]
        att = o.attention_forward(hs_table=table, batch_info=binfo, h_t=below, mask01=m_t[t], D=D, **attn)
        frac = att["p_t"] - np.floor(att["p_t"])
        assert np.all((frac > 1e-4) & (frac < 1 - 1e-4)), "p_t on an integer boundary; pick another seed"
        h_tild_prev = att["h_tild"]
        assert_close(hs[t], att["h_tild"], floor=1.0 if bf16 else 5e-2, what="h_tild step %d" % t)
        lp = o.softmax_logprob_f64(o.softmax_logits(Dm, bd, att["h_tild"]))
        assert losses[t] == pytest.approx(o.softmax_loss(lp, tgt[t], tmask[t]), rel=1e-4 if bf16 else 1e-5, abs=1e-6)
    if not bf16:
        # the decode-time attention layer (init_att_decoder, one node, all columns unmasked) on the last step's top h
        ones = np.ones(mb, np.int32)
        dec = o.attention_forward(hs_table=table, batch_info=binfo, h_t=below, mask01=ones, D=D, **attn)
        assert_close(hs["dec_h"], dec["h_tild"], what="decode-time attention layer h_tild")
        assert hs["viterbi"].tolist() == o.attention_viterbi(dec["alignments"], dec["indices"]).tolist()
        # swap_states_decoding with a host index vector: column i <- column (3 i + 1) mod mb
        order = [(b * 3 + 1) % mb for b in range(mb)]
        assert np.array_equal(hs["swap_after"], hs["swap_before"][:, order])
