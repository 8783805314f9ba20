"""Pins for the CPU oracle: every oracle function is checked against something that is not the oracle's own
formula retyped -- brute force on tiny inputs, closed forms, invariants, or a library routine
(numpy float64 matmul, scipy logsumexp, torch.nn.LSTMCell).  The reference holds no golden vectors for this
path (it has no tests directory), so these are what keeps the restatement honest."""
import numpy as np
import pytest
from scipy.special import logsumexp

import oracle_lib as o

RNG = np.random.default_rng(20240607)


def U(shape, lo=-0.08, hi=0.08, rng=RNG):
    return np.asfortranarray(rng.uniform(lo, hi, size=shape).astype(np.float32))


# ----------------------------------------------------------------------------- A1
def test_vocab_prep_bruteforce():
    ids = np.array([5, -1, 0, 7, -1, -1, 3], dtype=np.int32)
    nn, m = o.vocab_prep(ids)
    assert nn.tolist() == [5, 0, 0, 7, 0, 0, 3]
    assert m.tolist() == [1, 0, 1, 1, 0, 0, 1]
    ids2, m2, mf2 = o.vocab_softmax(ids)
    assert ids2.tolist() == nn.tolist() and m2.tolist() == m.tolist()
    assert mf2.dtype == np.float32 and mf2.tolist() == [1, 0, 1, 1, 0, 0, 1]


# ----------------------------------------------------------------------------- A2
def test_embed_gather_bit_exact():
    W = U((13, 29))
    ids = np.array([0, 28, 5, 5, 0, 17], dtype=np.int32)  # duplicates, first and last column
    x = o.embed_gather(W, ids)
    assert x.tobytes() == np.asfortranarray(W[:, ids]).tobytes()


# ----------------------------------------------------------------------------- A3
@pytest.mark.parametrize("M,N,K", [(8, 3, 8), (32, 5, 32), (100, 8, 100), (257, 9, 61)])
def test_gemm_against_numpy_f64(M, N, K):
    A, B = U((M, K), -1, 1), U((K, N), -1, 1)
    want = A.astype(np.float64) @ B.astype(np.float64)
    assert np.allclose(o.gemm_nn(A, B, acc64=True), want, rtol=0, atol=1e-6)
    assert np.allclose(o.gemm_nn(A, B, acc64=False), want, rtol=0, atol=1e-4)
    # transposed first operand: a swapped/transposed operand would fail on the non-square shapes
    At = np.asfortranarray(A.T)
    assert np.allclose(o.gemm_tn(At, B, acc64=True), want, rtol=0, atol=1e-6)


def test_gemm_special_cases():
    B = U((16, 4), -1, 1)
    assert np.array_equal(o.gemm_nn(np.eye(16, dtype=np.float32), B), B)
    assert np.array_equal(o.gemm_nn(np.zeros((7, 16), np.float32), B), np.zeros((7, 4), np.float32))
    onehot = np.zeros((3, 16), np.float32)
    onehot[0, 5] = onehot[1, 0] = onehot[2, 15] = 1
    assert np.array_equal(o.gemm_nn(onehot, B), B[[5, 0, 15], :])
    A = U((9, 16), -1, 1)
    # column independence: permuting batch columns permutes outputs
    perm = [2, 0, 3, 1]
    assert np.array_equal(o.gemm_nn(A, B[:, perm]), o.gemm_nn(A, B)[:, perm])
    # linearity in the second operand (exact for a power-of-two scale)
    assert np.array_equal(o.gemm_nn(A, 4 * B), 4 * o.gemm_nn(A, B))


# ----------------------------------------------------------------------------- A4/A5
def _rand_layer(H, feed=False):
    ly = {"M": [U((H, H)) for _ in range(4)], "Wh": [U((H, H)) for _ in range(4)], "b": [U(H) for _ in range(4)]}
    if feed:
        ly["Q"] = [U((H, H)) for _ in range(4)]
    return ly


def test_lstm_step_zero_weights_closed_form():
    H, mb = 6, 3
    Z = [np.zeros((H, H), np.float32)] * 4
    b0 = [np.zeros(H, np.float32)] * 4
    x, hp = U((H, mb), -1, 1), U((H, mb), -1, 1)
    cp = U((H, mb), -2, 2)
    r = o.lstm_step(Z, Z, b0, x, hp, cp, np.ones(mb, np.int32))
    assert np.array_equal(r["i"], np.full((H, mb), 0.5, np.float32))
    assert np.array_equal(r["f"], r["i"]) and np.array_equal(r["o"], r["i"])
    assert np.array_equal(r["c_tilde"], np.zeros((H, mb), np.float32))
    assert np.array_equal(r["c"], 0.5 * cp)
    assert np.allclose(r["h"], 0.5 * np.tanh(0.5 * cp.astype(np.float64)), atol=1e-7)
    # b_f = 1 (the reference's forget-bias init): f = sigmoid(1)
    b1 = [np.zeros(H, np.float32), np.ones(H, np.float32), np.zeros(H, np.float32), np.zeros(H, np.float32)]
    r = o.lstm_step(Z, Z, b1, x, hp, cp, np.ones(mb, np.int32))
    assert np.allclose(r["f"], 1 / (1 + np.exp(-1.0)), atol=1e-7)
    assert np.allclose(r["c"], cp / (1 + np.exp(-1.0)), atol=1e-6)


def test_lstm_step_gate_routing_one_hot():
    """Each gate must read its own matrices and bias: give every gate a distinct constant pre-activation through
    a one-hot M (from x) and one-hot Wh (from h_prev) and check all six outputs against scalars."""
    H, mb = 4, 2
    x = np.zeros((H, mb), np.float32)
    x[0, :] = 1.0
    hp = np.zeros((H, mb), np.float32)
    hp[1, :] = 1.0
    cp = np.full((H, mb), 0.25, np.float32)
    vals_x = [0.3, -0.7, 1.1, 2.0]   # coefficient picked up from x[0]
    vals_h = [0.05, 0.2, -0.4, -1.0]  # coefficient picked up from h_prev[1]
    bias = [0.01, 0.02, 0.03, 0.04]
    M, Wh, b = [], [], []
    for g in range(4):
        m = np.zeros((H, H), np.float32)
        m[:, 0] = vals_x[g]
        w = np.zeros((H, H), np.float32)
        w[:, 1] = vals_h[g]
        M.append(m)
        Wh.append(w)
        b.append(np.full(H, bias[g], np.float32))
    r = o.lstm_step(M, Wh, b, x, hp, cp, np.ones(mb, np.int32))
    pre = [vals_x[g] + vals_h[g] + bias[g] for g in range(4)]
    sig = lambda v: 1 / (1 + np.exp(-v))
    i, f, ct, og = sig(pre[0]), sig(pre[1]), np.tanh(pre[2]), sig(pre[3])
    c = f * 0.25 + i * ct
    assert np.allclose(r["i"], i, atol=1e-6) and np.allclose(r["f"], f, atol=1e-6)
    assert np.allclose(r["c_tilde"], ct, atol=1e-6) and np.allclose(r["o"], og, atol=1e-6)
    assert np.allclose(r["c"], c, atol=1e-6) and np.allclose(r["h"], og * np.tanh(c), atol=1e-6)


def test_lstm_step_against_torch_lstmcell():
    """Library pin: torch.nn.LSTMCell uses the same equations with gate order (i, f, g, o)."""
    torch = pytest.importorskip("torch")
    H, mb = 24, 5
    ly = _rand_layer(H)
    x, hp, cp = U((H, mb), -1, 1), U((H, mb), -1, 1), U((H, mb), -1, 1)
    cell = torch.nn.LSTMCell(H, H).double()
    with torch.no_grad():
        cell.weight_ih.copy_(torch.tensor(np.concatenate(ly["M"], axis=0), dtype=torch.float64))
        cell.weight_hh.copy_(torch.tensor(np.concatenate(ly["Wh"], axis=0), dtype=torch.float64))
        cell.bias_ih.copy_(torch.tensor(np.concatenate(ly["b"]), dtype=torch.float64))
        cell.bias_hh.zero_()
        h1, c1 = cell(torch.tensor(x.T.copy(), dtype=torch.float64),
                      (torch.tensor(hp.T.copy(), dtype=torch.float64), torch.tensor(cp.T.copy(), dtype=torch.float64)))
    r = o.lstm_step(ly["M"], ly["Wh"], ly["b"], x, hp, cp, np.ones(mb, np.int32))
    assert np.allclose(r["h"], h1.numpy().T, atol=2e-6)
    assert np.allclose(r["c"], c1.numpy().T, atol=2e-6)


def test_lstm_step_saturation_mask_clip_and_bounds():
    H, mb = 5, 4
    ly = _rand_layer(H)
    x, hp = U((H, mb), -1, 1), U((H, mb), -1, 1)
    cp = U((H, mb), -3, 3)
    big = [np.full(H, 40.0, np.float32), np.full(H, -40.0, np.float32), np.full(H, 40.0, np.float32),
           np.full(H, -40.0, np.float32)]
    r = o.lstm_step(ly["M"], ly["Wh"], big, x, hp, cp, np.ones(mb, np.int32))
    assert np.all(r["i"] == 1.0) and np.all(r["c_tilde"] == 1.0)
    assert np.all(np.abs(r["f"]) < 1e-15) and np.all(np.abs(r["o"]) < 1e-15) and np.all(np.isfinite(r["h"]))
    # masked column -> h = c = 0 exactly; others untouched
    mask = np.array([1, 0, 1, 0], np.int32)
    r1 = o.lstm_step(ly["M"], ly["Wh"], ly["b"], x, hp, cp, np.ones(mb, np.int32))
    r2 = o.lstm_step(ly["M"], ly["Wh"], ly["b"], x, hp, cp, mask)
    assert np.all(r2["h"][:, [1, 3]] == 0) and np.all(r2["c"][:, [1, 3]] == 0)
    assert np.array_equal(r2["h"][:, [0, 2]], r1["h"][:, [0, 2]])
    # |h| < 1 and |c_t| <= |c_{t-1}| + 1
    assert np.all(np.abs(r1["h"]) < 1) and np.all(np.abs(r1["c"]) <= np.abs(cp) + 1)
    # clip: result equals clamp of the unclipped cell, and h follows the clipped cell
    r3 = o.lstm_step(ly["M"], ly["Wh"], ly["b"], x, hp, cp, np.ones(mb, np.int32), clip=0.75)
    assert np.array_equal(r3["c"], np.clip(r1["c"], -0.75, 0.75))
    assert np.allclose(r3["h"], r1["o"] * np.tanh(r3["c"].astype(np.float64)), atol=1e-7)


def test_lstm_step_feed_input_reduces_and_adds():
    H, mb = 12, 3
    ly = _rand_layer(H, feed=True)
    x, hp, cp, ht = U((H, mb), -1, 1), U((H, mb), -1, 1), U((H, mb), -1, 1), U((H, mb), -1, 1)
    ones = np.ones(mb, np.int32)
    base = o.lstm_step(ly["M"], ly["Wh"], ly["b"], x, hp, cp, ones)
    zq = [np.zeros((H, H), np.float32)] * 4
    feed0 = o.lstm_step(ly["M"], ly["Wh"], ly["b"], x, hp, cp, ones, Q=zq, htild=ht)
    # Q = 0: same pre-activations; the feed kernels evaluate the sigmoid in double, so allow 1 ulp
    for k in ("i", "f", "o", "c_tilde", "c", "h"):
        assert np.allclose(feed0[k], base[k], rtol=0, atol=2e-7), k
    # Q term really is Q @ htild added to the pre-activation: fold it into the bias column by column
    feed = o.lstm_step(ly["M"], ly["Wh"], ly["b"], x, hp, cp, ones, Q=ly["Q"], htild=ht)
    for col in range(mb):
        b_eff = [ly["b"][g] + (ly["Q"][g].astype(np.float64) @ ht[:, col].astype(np.float64)).astype(np.float32)
                 for g in range(4)]
        r = o.lstm_step(ly["M"], ly["Wh"], b_eff, x[:, [col]], hp[:, [col]], cp[:, [col]], ones[:1])
        assert np.allclose(feed["h"][:, [col]], r["h"], atol=1e-6)
        assert np.allclose(feed["c"][:, [col]], r["c"], atol=1e-6)


# ----------------------------------------------------------------------------- A8/A9
def test_softmax_properties():
    V, H, mb = 211, 16, 6
    D, bd, h = U((V, H), -1, 1), U(V, -1, 1), U((H, mb), -1, 1)
    logits = o.softmax_logits(D, bd, h)
    assert np.allclose(logits, D.astype(np.float64) @ h.astype(np.float64) + bd[:, None], atol=1e-6)
    for tree in (False, True):
        P = o.softmax_dist(logits, emulate_tree=tree)
        assert np.allclose(P.sum(axis=0, dtype=np.float64), 1.0, atol=1e-5)
        assert np.array_equal(P.argmax(axis=0), logits.argmax(axis=0))
        want = np.exp(logits.astype(np.float64) - logsumexp(logits.astype(np.float64), axis=0))
        assert np.allclose(P, want, rtol=1e-5, atol=1e-9)
    LP = o.softmax_logprob_f64(logits)
    assert LP.dtype == np.float64
    assert np.allclose(LP, logits.astype(np.float64) - logsumexp(logits.astype(np.float64), axis=0), atol=1e-12)
    # shift invariance: adding a constant to every bias leaves the distribution unchanged
    P2 = o.softmax_dist(o.softmax_logits(D, bd + np.float32(0.5), h))
    assert np.allclose(P2, o.softmax_dist(logits), rtol=2e-5, atol=1e-9)
    # D = 0, b = 0 -> uniform
    LP0 = o.softmax_logprob_f64(o.softmax_logits(np.zeros((V, H), np.float32), np.zeros(V, np.float32), h))
    assert np.allclose(LP0, np.log(1.0 / V), atol=1e-12)
    # extreme logits: no overflow, still normalised
    ext = np.asfortranarray(RNG.choice(np.array([-80.0, 0.0, 80.0], np.float32), size=(V, mb)))
    ext[0, :] = 80.0
    Pe = o.softmax_dist(ext)
    assert np.all(np.isfinite(Pe)) and np.allclose(Pe.sum(axis=0, dtype=np.float64), 1.0, atol=1e-5)
    # loss = sum over unmasked columns of logp[target]
    tgt = np.array([3, 0, 210, 7, 7, 100], np.int32)
    mask = np.array([1, 1, 0, 1, 0, 1], np.int32)
    want = sum(LP[tgt[b], b] for b in range(mb) if mask[b])
    assert o.softmax_loss(LP, tgt, mask) == pytest.approx(want, abs=1e-12)


# ----------------------------------------------------------------------------- A10
def _attn_weights(H):
    return dict(W_a=U((H, H), -0.3, 0.3), W_p=U((H, H), -0.3, 0.3), v_p=U(H, -0.5, 0.5), out_bias=U(H),
                W_c1=U((H, H), -0.3, 0.3), W_c2=U((H, H), -0.3, 0.3))


def test_attention_window_and_invariants():
    H, mb, S, D = 10, 6, 9, 2
    w = _attn_weights(H)
    hs = RNG.normal(0, 0.5, size=(S, H, mb)).astype(np.float32)
    lens = np.array([9, 7, 9, 3, 5, 1], np.int32)
    batch_info = np.concatenate([lens, S - lens]).astype(np.int32)
    mask = np.array([1, 1, 1, 1, 0, 1], np.int32)
    h_t = U((H, mb), -1, 1)
    r = o.attention_forward(hs_table=hs, batch_info=batch_info, h_t=h_t, mask01=mask, D=D, **w)
    Wn = 2 * D + 1
    idx, a, p = r["indices"], r["alignments"], r["p_t"]
    sigma_sq = D * D / 4.0
    for b in range(mb):
        if mask[b] == 0:
            assert np.all(idx[b] == -1) and np.all(a[b] == 0) and np.all(r["h_tild"][:, b] == 0)
            continue
        assert 0 < p[b] < lens[b]
        lo, hi = max(0, int(p[b]) - D), min(lens[b] - 1, int(p[b]) + D)
        want_idx = [lo + j if lo + j <= hi else -1 for j in range(Wn)]
        assert idx[b].tolist() == want_idx
        valid = idx[b] != -1
        gauss = np.exp(-(p[b] - idx[b][valid].astype(np.float64)) ** 2 / (2 * sigma_sq))
        # the pre-Gaussian softmax is normalised over the valid slots
        assert np.sum(a[b][valid] / gauss) == pytest.approx(1.0, abs=1e-5)
        assert np.all(a[b][~valid] == 0)
        # context = sum_j a_j * hs[source position], source stored reversed and left padded
        ctx = np.zeros(H)
        for j in np.nonzero(valid)[0]:
            t = lens[b] - 1 - idx[b, j] + (S - lens[b])
            ctx += a[b, j] * hs[t, :, b].astype(np.float64)
        assert np.allclose(r["c_ctx"][:, b], ctx, atol=1e-6)
        ht = np.tanh(w["W_c1"].astype(np.float64) @ ctx + w["W_c2"].astype(np.float64) @ h_t[:, b] + w["out_bias"])
        assert np.allclose(r["h_tild"][:, b], ht, atol=1e-5)


def test_attention_reversed_padded_indexing_one_hot():
    """hs table t holds e_t (scaled) in every column, so the context reveals which table each slot read."""
    H, mb, S, D = 12, 3, 8, 8  # D >= S: every source position has a slot
    w = _attn_weights(H)
    w["W_a"] = np.zeros((H, H), np.float32)  # uniform pre-Gaussian weights
    hs = np.zeros((S, H, mb), np.float32)
    for t in range(S):
        hs[t, t, :] = 1.0
    lens = np.array([8, 5, 2], np.int32)
    batch_info = np.concatenate([lens, S - lens]).astype(np.int32)
    r = o.attention_forward(hs_table=hs, batch_info=batch_info, h_t=U((H, mb), -1, 1), mask01=np.ones(mb, np.int32),
                            D=D, **w)
    sigma_sq = D * D / 4.0
    for b in range(mb):
        idx = r["indices"][b]
        assert idx[:lens[b]].tolist() == list(range(lens[b])) and np.all(idx[lens[b]:] == -1)
        for s in range(lens[b]):
            t = lens[b] - 1 - s + (S - lens[b])
            want = (1.0 / lens[b]) * np.exp(-(r["p_t"][b] - s) ** 2 / (2 * sigma_sq))
            assert r["c_ctx"][t, b] == pytest.approx(want, rel=1e-5)
        pad_rows = [t for t in range(H) if t < S - lens[b] or t >= S]
        assert np.all(r["c_ctx"][pad_rows, b] == 0)


def test_attention_max_zero_quirk_and_equal_hs():
    """All scores negative: the reference's max starts at 0, so weights are exp(score)/sum exp(score) computed
    without a shift; this is mathematically the same softmax but it must not be a -inf initialised max when
    scores are very negative (exp underflow -> sum == 0 -> alignments stay un-normalised exp values * gauss)."""
    H, mb, S, D = 4, 2, 5, 5
    w = _attn_weights(H)
    w["W_a"] = np.asfortranarray(-200.0 * np.eye(H, dtype=np.float32))  # q = -200 h ; score = -200 |h|^2-ish
    h_t = np.ones((H, mb), np.float32)
    hs = np.ones((S, H, mb), np.float32)  # score = -800 for every slot: expf(-800) == 0 -> sum == 0
    lens = np.array([5, 5], np.int32)
    r = o.attention_forward(hs_table=hs, batch_info=np.concatenate([lens, S - lens]).astype(np.int32), h_t=h_t,
                            mask01=np.ones(mb, np.int32), D=D, **w)
    assert np.all(r["alignments"] == 0) and np.all(np.isfinite(r["h_tild"]))
    # mild negative scores: equal hs -> context = (sum a) * hs column
    w["W_a"] = np.asfortranarray(-0.1 * np.eye(H, dtype=np.float32))
    r = o.attention_forward(hs_table=hs, batch_info=np.concatenate([lens, S - lens]).astype(np.int32), h_t=h_t,
                            mask01=np.ones(mb, np.int32), D=D, **w)
    for b in range(mb):
        assert np.allclose(r["c_ctx"][:, b], r["alignments"][b].sum() * 1.0, rtol=1e-6)


# ----------------------------------------------------------------------------- A12
def test_gather_columns():
    src = U((7, 5))
    assert np.array_equal(o.gather_columns(src, np.arange(5)), src)
    perm = np.array([4, 4, 0, 2, 2, 1], np.int32)
    assert o.gather_columns(src, perm).tobytes() == np.asfortranarray(src[:, perm]).tobytes()


# ----------------------------------------------------------------------------- A13
def _bruteforce_expand(P, scores, beam, index, live):
    """Independent statement of the selection rule for tie-free inputs: candidates are the beam+1 most probable
    words of every live column, ranked by log p + column score; <START>=0 skipped, <EOF>=1 finishes."""
    V = P.shape[0]
    cols = 1 if index == 0 else beam
    cands = []
    for i in range(cols):
        if not live[i]:
            break
        order = np.argsort(-P[:, i], kind="stable")[:beam + 1]
        for v in order:
            cands.append((np.float32(np.log(P[v, i])) + np.float32(scores[i]), i, int(v)))
    cands.sort(key=lambda t: -t[0])
    words, back, sc, finished = [], [], [], []
    for val, i, v in cands:
        if len(words) == beam:
            break
        if v == 0:
            continue
        if v == 1:
            finished.append((i, val))
            continue
        words.append(v)
        back.append(i)
        sc.append(val)
    return words, back, sc, finished


@pytest.mark.parametrize("V,beam", [(50, 4), (23, 3), (40, 1)])
def test_beam_expand_against_bruteforce(V, beam):
    rng = np.random.default_rng(V * 31 + beam)
    dec = o.Decoder(beam, V, max_len=12)
    scores = np.zeros(beam, np.float32)
    live = [True] * beam
    for index in range(5):
        logits = rng.normal(0, 2.0, size=(V, beam))
        P = np.asfortranarray((np.exp(logits) / np.exp(logits).sum(axis=0)).astype(np.float32))
        words, back, sc, fin = _bruteforce_expand(P, scores, beam, index, live)
        n_before = len(dec.hypotheses())
        dec.expand(P, index)
        st = dec.state()
        assert st["current_indices"].tolist() == words
        assert st["new_indicies_changes"].tolist() == back
        assert np.allclose(st["scores"], sc, rtol=1e-6)
        assert 0 not in st["current_indices"].tolist()
        hyps = dec.hypotheses()[n_before:]
        assert len(hyps) == len(fin)
        for (hw, hs), (bi, val) in zip(hyps, fin):
            assert hw[-1] == 1 and len(hw) == index + 2 and hs == pytest.approx(val, rel=1e-6)
        # scores never increase along a hypothesis when penalty = 0
        assert np.all(st["scores"] <= scores[st["new_indicies_changes"]] + 1e-6)
        scores = st["scores"].copy()


def test_beam_step0_uses_first_column_only_and_ties():
    V, beam = 12, 3
    dec = o.Decoder(beam, V, max_len=6)
    P = np.zeros((V, beam), np.float32, order="F")
    P[:, 0] = np.array([0.3, 0.05, 0.2, 0.1, 0.1, 0.05, 0.05, 0.05, 0.025, 0.025, 0.025, 0.025], np.float32)
    P[:, 1] = 1.0 / V
    P[5, 1] = 0.9  # would win if column 1 were looked at
    P[:, 2] = 1.0 / V
    dec.expand(P, 0)
    st = dec.state()
    # <START>=0 skipped although most probable; ties 0.1/0.1: both selected, higher p first
    assert st["current_indices"][0] == 2 and set(st["current_indices"][1:].tolist()) == {3, 4}
    assert st["new_indicies_changes"].tolist() == [0, 0, 0]
    # integer-valued tie case: all equal probabilities -> the first beam+1 words stay in the heap
    dec2 = o.Decoder(beam, V, max_len=6)
    dec2.expand(np.full((V, beam), 0.125, np.float32, order="F"), 0)
    got = dec2.state()["current_indices"].tolist()
    # heap = words {0,1,2,3}: <START> skipped, <EOF> finishes a hypothesis, 2 and 3 survive, and the third
    # beam slot falls into the empty-heap branch (invalid symbol -1, back-pointer 0, score 0)
    assert sorted(got[:2]) == [2, 3] and got[2] == -1
    assert len(dec2.hypotheses()) == 1 and dec2.hypotheses()[0][0].tolist() == [0, 1]
    assert dec2.state()["scores"][2] == 0 and dec2.state()["new_indicies_changes"][2] == 0


def test_beam_finish_and_k_best():
    V, beam = 20, 2
    rng = np.random.default_rng(5)
    dec = o.Decoder(beam, V, max_len=8, penalty=0.5, min_ratio=0.0)
    for index in range(3):
        logits = rng.normal(0, 1.5, size=(V, beam))
        P = (np.exp(logits) / np.exp(logits).sum(axis=0)).astype(np.float32)
        dec.expand(P, index)
    before = dec.state()
    n0 = len(dec.hypotheses())
    dec.finish(P)
    hyps = dec.hypotheses()
    assert len(hyps) == n0 + beam
    for i in range(beam):
        w, s = hyps[n0 + i]
        assert w[-1] == 1 and len(w) == 5
        assert s == pytest.approx(before["scores"][i] + np.log(P[1, i]) + 0.5, rel=1e-6)
    order = dec.k_best(source_length=3, num_hypotheses=2)
    all_scores = [s for _, s in hyps]
    assert [all_scores[i] for i in order] == sorted(all_scores, reverse=True)[:2]


@pytest.mark.parametrize("V,beam,steps,seed", [(30, 3, 6, 1), (60, 5, 9, 2), (12, 2, 5, 3)])
def test_beam_viterbi_histories_follow_the_back_pointers(V, beam, steps, seed):
    """The alignments a hypothesis carries (src/decoder.h:1266-1282, 683-684), restated without row copies: the word at
    position j of a hypothesis was chosen at expand step j-1 from some beam column; chase the back pointers
    (new_indicies_changes) from the hypothesis's last column to find that column at every step, and the alignment at
    position j must be the one the attention layer reported for THAT column at THAT step.  A history indexed by the new
    slot instead of the parent column, or shifted by one position, fails.  Position 0 keeps the initial -20."""
    rng = np.random.default_rng(seed)
    dec = o.Decoder(beam, V, max_len=steps + 4, penalty=0.0)
    vit_at, parent_at, words_at, n_hyp = [], [], [], [0]
    for index in range(steps):
        logits = rng.normal(0, 2.0, size=(V, beam))
        logits[1] += 1.0  # <EOF> often near the top, so hypotheses finish at every length
        P = (np.exp(logits) / np.exp(logits).sum(axis=0)).astype(np.float32)
        vit = rng.integers(0, 50, size=beam).astype(np.int32)
        dec.expand(P, index, vit)
        st = dec.state()
        vit_at.append(vit)
        parent_at.append(st["new_indicies_changes"].copy())
        words_at.append(st["current_indices"].copy())
        n_hyp.append(len(dec.hypotheses()))
        # live beam rows: chase from slot i at this step back to step 0
        tv = dec.top_viterbi()
        for i in range(beam):
            if st["current_indices"][i] == -1:
                continue
            col = i
            for j in range(index, -1, -1):
                col_parent = parent_at[j][col]
                assert tv[i, j + 1] == vit_at[j][col_parent], (index, i, j)
                col = col_parent
            assert tv[i, 0] == -20
    fin_vit = rng.integers(0, 50, size=beam).astype(np.int32)
    live = dec.state()["current_indices"].copy()
    tv_before = dec.top_viterbi()
    dec.finish(P, fin_vit)
    hyps, hv = dec.hypotheses(), dec.hypotheses_viterbi()
    assert len(hyps) == len(hv) > n_hyp[-1] - 1
    # hypotheses finished by the forced <EOF>: the row of their slot, then the alignment of the last step
    forced = [i for i in range(beam) if live[i] != -1]
    for k, i in enumerate(forced):
        v = hv[n_hyp[-1] + k]
        assert len(v) == steps + 2 and v[-1] == fin_vit[i] and np.array_equal(v[:-1], tv_before[i, :steps + 1])
    # hypotheses finished by an <EOF> candidate at step `index`: words identify the parent row unambiguously here only
    # through the history, so check the invariants that do not need it: length, -20 at 0, every entry one of the
    # alignments reported at its step
    for (w, _), v in zip(hyps, hv):
        assert len(v) == len(w) and v[0] == -20
        for j in range(1, len(v) - (1 if len(v) == steps + 2 else 0)):
            assert v[j] in set(vit_at[j - 1].tolist())
    # no alignments given: the reference fills in -1
    dec2 = o.Decoder(beam, V, max_len=8)
    dec2.expand(P, 0)
    assert set(dec2.top_viterbi()[:, 1].tolist()) <= {-1, -20} and (dec2.top_viterbi()[:, 1] == -1).any()


# ----------------------------------------------------------------------------- A6/A7/A11 composition
def test_stack_forward_is_composition_of_steps():
    H, mb, T, V, L = 8, 3, 4, 17, 2
    embed = U((H, V))
    layers = [_rand_layer(H) for _ in range(L)]
    ids = RNG.integers(0, V, size=(T, mb)).astype(np.int32)
    ids[0, 1] = -1  # a padded position (source side pads on the left)
    nn, m = o.vocab_prep(ids)
    h_all, c_all = o.lstm_stack_forward(embed, layers, nn, m)
    hp = [np.zeros((H, mb), np.float32) for _ in range(L)]
    cp = [np.zeros((H, mb), np.float32) for _ in range(L)]
    for t in range(T):
        below = o.embed_gather(embed, nn[t])
        for l in range(L):
            r = o.lstm_step(layers[l]["M"], layers[l]["Wh"], layers[l]["b"], below, hp[l], cp[l], m[t])
            assert np.array_equal(h_all[l, t], r["h"]) and np.array_equal(c_all[l, t], r["c"])
            hp[l], cp[l], below = r["h"], r["c"], r["h"]
    assert np.all(h_all[:, 0, :, 1] == 0)


# ----------------------------------------------------------------------------- by-value brute-force pins
def _attention_numpy_f64(w, hs, lens, offs, h_t, mask, D):
    """Luong local-p attention written from the paper's formulas in float64, column by column, with plain numpy
    products: p_t = S sigmoid(v_p . tanh(W_p h)); score_s = h_s . (W_a^T h) = h^T W_a h_s over the window
    [max(0, floor(p_t) - D), min(S - 1, floor(p_t) + D)]; softmax over the window times exp(-(p_t - s)^2 / (2 (D/2)^2));
    context = sum a_s h_s; h~ = tanh(W_c1 c + W_c2 h + b).  Source position s of column b is table
    S_b - 1 - s + offset_b (the source is stored reversed and left padded)."""
    H, mb = h_t.shape
    Wa, Wp, Wc1, Wc2 = (w[k].astype(np.float64) for k in ("W_a", "W_p", "W_c1", "W_c2"))
    vp, bias = w["v_p"].astype(np.float64).reshape(-1), w["out_bias"].astype(np.float64)
    out = {"p_t": np.zeros(mb), "scores": {}, "align": {}, "c": np.zeros((H, mb)), "h_tild": np.zeros((H, mb))}
    for b in range(mb):
        h = h_t[:, b].astype(np.float64)
        p = lens[b] / (1.0 + np.exp(-(vp @ np.tanh(Wp @ h))))
        out["p_t"][b] = p
        if not mask[b]:
            continue
        lo, hi = max(0, int(p) - D), min(int(lens[b]) - 1, int(p) + D)
        pos = list(range(lo, hi + 1))
        src = [hs[lens[b] - 1 - s + offs[b], :, b].astype(np.float64) for s in pos]
        sc = np.array([h @ Wa @ hv for hv in src])
        e = np.exp(sc - sc.max())
        a = e / e.sum() * np.exp(-(p - np.array(pos)) ** 2 / (2 * (D / 2.0) ** 2))
        c = sum(ai * hv for ai, hv in zip(a, src))
        out["scores"][b], out["align"][b] = dict(zip(pos, sc)), dict(zip(pos, a))
        out["c"][:, b] = c
        out["h_tild"][:, b] = np.tanh(Wc1 @ c + Wc2 @ h + bias)
    return out


@pytest.mark.parametrize("H,mb,S,D,seed", [(10, 6, 9, 2, 1), (16, 5, 12, 12, 2), (7, 4, 30, 3, 3)])
def test_attention_by_value_against_numpy_f64(H, mb, S, D, seed):
    """Every output by value: fails for W_a in place of W_a^T (W_a is not symmetric), for a missing tanh or sigmoid
    in p_t, for a wrong Gaussian width and for a wrong source-table index."""
    rng = np.random.default_rng(seed)
    w = dict(W_a=U((H, H), -0.6, 0.6, rng), W_p=U((H, H), -0.9, 0.9, rng), v_p=U(H, -1.5, 1.5, rng),
             out_bias=U(H, -0.3, 0.3, rng), W_c1=U((H, H), -0.4, 0.4, rng), W_c2=U((H, H), -0.4, 0.4, rng))
    assert np.abs(w["W_a"] - w["W_a"].T).max() > 0.1
    hs = rng.normal(0, 0.7, size=(S, H, mb)).astype(np.float32)
    lens = rng.integers(1, S + 1, size=mb).astype(np.int32)
    lens[0] = S
    offs = (S - lens).astype(np.int32)
    mask = np.ones(mb, np.int32)
    mask[mb - 2] = 0
    h_t = U((H, mb), -1, 1, rng)
    r = o.attention_forward(hs_table=hs, batch_info=np.concatenate([lens, offs]), h_t=h_t, mask01=mask, D=D, **w)
    want = _attention_numpy_f64(w, hs, lens, offs, h_t, mask, D)
    assert np.allclose(r["p_t"], want["p_t"], rtol=2e-6)
    # p_t must actually depend on the tanh: the pre-activations are large enough that dropping it moves p_t
    lin = lens / (1.0 + np.exp(-(w["v_p"].astype(np.float64) @ (w["W_p"].astype(np.float64) @ h_t))))
    assert np.abs(lin - want["p_t"]).max() > 1e-2
    Wn = 2 * D + 1
    for b in range(mb):
        if not mask[b]:
            assert np.all(r["alignments"][b] == 0) and np.all(r["h_tild"][:, b] == 0)
            continue
        got = {int(s): r["alignments"][b, j] for j, s in enumerate(r["indices"][b]) if s != -1}
        assert sorted(got) == sorted(want["align"][b])
        for s, a in want["align"][b].items():
            assert got[s] == pytest.approx(a, rel=2e-5, abs=1e-9)
        # the alignments differ from those of the transposed score matrix by far more than the tolerance
        assert len(got) <= Wn
    assert np.allclose(r["c_ctx"], want["c"], atol=2e-6)
    assert np.allclose(r["h_tild"], want["h_tild"], atol=2e-6)
    wT = dict(w, W_a=np.asfortranarray(w["W_a"].T))
    wrong = _attention_numpy_f64(wT, hs, lens, offs, h_t, mask, D)
    assert np.abs(wrong["h_tild"] - want["h_tild"]).max() > 1e-3


def _bruteforce_decode_step(P, prev_scores, prev_sent, live, beam, index, penalty):
    """One beam step from the rules alone (tie-free inputs): candidates are the beam+1 most probable words of each
    live column scored log p + column score; best first: <START> is dropped, <EOF> closes a hypothesis with
    candidate score + penalty, anything else survives with candidate score + penalty until beam survivors exist."""
    cols = 1 if index == 0 else beam
    cands = []
    for i in range(cols):
        if not live[i]:
            break
        for v in np.argsort(-P[:, i], kind="stable")[:beam + 1]:
            cands.append((np.float32(np.float32(np.log(P[v, i])) + np.float32(prev_scores[i])), i, int(v)))
    cands.sort(key=lambda t: -t[0])
    surv, fin = [], []
    for val, i, v in cands:
        if len(surv) == beam:
            break
        if v == 0:
            continue
        if v == 1:
            fin.append((prev_sent[i] + [1], np.float32(val + np.float32(penalty))))
        else:
            surv.append((prev_sent[i] + [v], np.float32(val + np.float32(penalty)), i))
    return surv, fin


@pytest.mark.parametrize("penalty", [0.75, -0.4])
def test_beam_penalty_in_expand_and_finish_against_bruteforce(penalty):
    """Length penalty != 0: survivors and <EOF> hypotheses each gain exactly one penalty per word, and because the
    penalty enters the scores that rank the next step, dropping it anywhere changes the later selections."""
    V, beam, steps = 30, 3, 6
    rng = np.random.default_rng(77)
    dec = o.Decoder(beam, V, max_len=steps + 3, penalty=penalty)
    scores, sent, live = np.zeros(beam, np.float32), [[0] for _ in range(beam)], [True] * beam
    all_fin = []
    for index in range(steps):
        logits = rng.normal(0, 2.0, size=(V, beam))
        logits[1] += 3.0  # make <EOF> a frequent candidate
        P = np.asfortranarray((np.exp(logits) / np.exp(logits).sum(axis=0)).astype(np.float32))
        surv, fin = _bruteforce_decode_step(P, scores, sent, live, beam, index, penalty)
        assert len(surv) == beam
        dec.expand(P, index)
        st = dec.state()
        assert st["current_indices"].tolist() == [s[0][-1] for s in surv]
        assert st["new_indicies_changes"].tolist() == [s[2] for s in surv]
        assert np.allclose(st["scores"], [s[1] for s in surv], rtol=2e-6, atol=1e-6)
        for i in range(beam):
            assert st["top_sentences"][i, :index + 2].tolist() == surv[i][0]
        all_fin += fin
        scores, sent = np.array([s[1] for s in surv], np.float32), [s[0] for s in surv]
    assert len(all_fin) >= 3  # the <EOF> branch was exercised
    # forced finish: every live beam ends with <EOF>, score + log P(<EOF>) + penalty
    for i in range(beam):
        all_fin.append((sent[i] + [1], np.float32(scores[i] + np.float32(np.log(P[1, i])) + np.float32(penalty))))
    dec.finish(P)
    hyps = dec.hypotheses()
    assert len(hyps) == len(all_fin)
    for (hw, hsc), (bw, bsc) in zip(hyps, all_fin):
        assert hw.tolist() == bw and hsc == pytest.approx(bsc, rel=2e-6, abs=1e-6)


def test_k_best_ratio_filter_is_strict():
    """Hypotheses whose length / source length equals min_decoding_ratio exactly are dropped (strictly greater
    passes), src/decoder.h:1394.  Lengths count <START> and <EOF>."""
    V, beam = 8, 2

    def dist():
        # <EOF> (word 1) is the second most probable word of column 0, so every step pops: best survivor, <EOF> of
        # the best column (a finished hypothesis), second survivor.  The two columns differ, so nothing ties.
        P = np.full((V, beam), 1e-4, np.float32, order="F")
        P[1, :] = 0.3
        P[2, 0], P[3, 0] = 0.42, 0.21
        P[2, 1], P[3, 1] = 0.40, 0.22
        return P

    dec = o.Decoder(beam, V, max_len=10, penalty=0.0, min_ratio=0.5)
    for index in range(4):  # <EOF> is among the top beam+1 of every column: hypotheses of 2, 3, 4, 5 words
        dec.expand(dist(), index)
    hyps = dec.hypotheses()
    lengths = [len(w) for w, _ in hyps]
    assert {2, 3, 4, 5} <= set(lengths)
    S = 8  # ratio 0.5 <=> length 4: lengths 2, 3 and exactly 4 are out, 5 is in
    order = dec.k_best(source_length=S, num_hypotheses=len(hyps))
    assert len(order) > 0 and all(lengths[i] > 4 for i in order)
    assert sorted(order.tolist()) == [i for i, n in enumerate(lengths) if n > 4]
    scores = [hyps[i][1] for i in order]
    assert scores == sorted(scores, reverse=True)
    S = 10  # ratio 0.5 <=> length 5, the longest there is: nothing passes
    assert dec.k_best(source_length=S, num_hypotheses=len(hyps)).size == 0
    S = 9   # 4/9 < 0.5 < 5/9
    assert sorted(dec.k_best(source_length=S, num_hypotheses=len(hyps)).tolist()) == \
        [i for i, n in enumerate(lengths) if n >= 5]


def _lstm_stack_numpy_f64(embed, layers, ids, h0, c0, clip):
    """Stacked LSTM in float64 from the textbook equations (gate order i, f, c~, o); ids -1 = padded position:
    embedding column 0 is read and h, c of that column are zeroed; the cell is clamped to +-clip before h."""
    T, mb = ids.shape
    L, H = len(layers), embed.shape[0]
    sig = lambda v: 1.0 / (1.0 + np.exp(-v))
    h = [np.array(a, np.float64) for a in h0]
    c = [np.array(a, np.float64) for a in c0]
    h_all, c_all = np.zeros((L, T, H, mb)), np.zeros((L, T, H, mb))
    for t in range(T):
        below = embed[:, np.maximum(ids[t], 0)].astype(np.float64)
        m = (ids[t] >= 0).astype(np.float64)
        for l, ly in enumerate(layers):
            pre = [ly["M"][g].astype(np.float64) @ below + ly["Wh"][g].astype(np.float64) @ h[l] +
                   ly["b"][g].astype(np.float64)[:, None] for g in range(4)]
            cn = sig(pre[1]) * c[l] + sig(pre[0]) * np.tanh(pre[2])
            if clip is not None:
                cn = np.clip(cn, -clip, clip)
            hn = sig(pre[3]) * np.tanh(cn)
            h[l], c[l] = hn * m, cn * m
            h_all[l, t], c_all[l, t] = h[l], c[l]
            below = h[l]
    return h_all, c_all


@pytest.mark.parametrize("clip", [None, 0.3])
def test_stack_forward_nonzero_initial_state_and_clip_against_numpy_f64(clip):
    H, mb, T, V, L = 9, 4, 5, 23, 3
    rng = np.random.default_rng(11)
    embed = U((H, V), -1, 1, rng)
    layers = [{"M": [U((H, H), -0.8, 0.8, rng) for _ in range(4)], "Wh": [U((H, H), -0.8, 0.8, rng) for _ in range(4)],
               "b": [U(H, -0.5, 0.5, rng) for _ in range(4)]} for _ in range(L)]
    ids = rng.integers(0, V, size=(T, mb)).astype(np.int32)
    ids[:2, 2] = -1
    h0 = [U((H, mb), -0.9, 0.9, rng) for _ in range(L)]
    c0 = [U((H, mb), -1.5, 1.5, rng) for _ in range(L)]
    nn, m = o.vocab_prep(ids)
    h_all, c_all = o.lstm_stack_forward(embed, layers, nn, m, h0=h0, c0=c0, clip=clip)
    want_h, want_c = _lstm_stack_numpy_f64(embed, layers, ids, h0, c0, clip)
    assert np.allclose(h_all, want_h, atol=2e-6) and np.allclose(c_all, want_c, atol=2e-6)
    # the cases must exercise what they claim to: the initial state matters, and the clip binds somewhere
    z = [np.zeros((H, mb), np.float32)] * L
    hz, _ = _lstm_stack_numpy_f64(embed, layers, ids, z, z, clip)
    assert np.abs(hz[:, 0] - want_h[:, 0]).max() > 1e-2
    if clip is not None:
        unclipped, cu = _lstm_stack_numpy_f64(embed, layers, ids, h0, c0, None)
        assert np.abs(cu).max() > clip + 0.1 and np.abs(want_c).max() <= clip + 1e-12
        assert np.abs(unclipped - want_h).max() > 1e-3
        # each layer has its own initial state: swapping two layers' states changes the result
    h_sw, _ = o.lstm_stack_forward(embed, layers, nn, m, h0=h0[::-1], c0=c0[::-1], clip=clip)
    assert np.abs(h_sw - want_h).max() > 1e-2


def test_attention_viterbi_first_maximum_wins():
    """Independent statement: numpy argmax returns the first maximum, the rule of a scan that only replaces on a
    strictly larger weight; a masked column (all weights 0, all indices -1) reports -1."""
    rng = np.random.default_rng(9)
    mb, D = 7, 4
    Wn = 2 * D + 1
    al = np.asfortranarray(rng.random((mb, Wn)).astype(np.float32))
    ix = np.asfortranarray(rng.integers(0, 40, size=(mb, Wn)).astype(np.int32))
    al[1, 2] = al[1, 6] = 2.0           # tie: slot 2 wins
    al[3, :] = 0.0                      # all zero, live column: first slot's index
    al[4, :], ix[4, :] = 0.0, -1        # masked column
    al[5, 5:], ix[5, 5:] = 0.0, -1      # short window: tail slots empty
    want = [int(ix[b, int(np.argmax(al[b]))]) for b in range(mb)]
    assert want[1] == ix[1, 2] and want[3] == ix[3, 0] and want[4] == -1
    assert o.attention_viterbi(al, ix).tolist() == want
