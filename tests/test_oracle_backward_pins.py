"""Pins of the oracle's backward restatement (CPU only).  The reference holds no gradient fixtures, so every function
is pinned by what the mathematics fixes: torch autograd (float64) on a network written from the forward equations,
central finite differences of the oracle's own forward pass, and closed forms."""
import numpy as np
import pytest
import torch

import oracle_lib as o
from zoph_rnn_amd import synth

U = synth.uniform


class _ClampGradient(torch.autograd.Function):
    """Identity whose backward clamps the gradient passing through it to +-limit."""
    @staticmethod
    def forward(ctx, x, limit):
        ctx.limit = limit
        return x.view_as(x)

    @staticmethod
    def backward(ctx, grad):
        return grad.clamp(-ctx.limit, ctx.limit), None


def _torch_stack(embed, layers, ids, mask, h0, c0, err_top, err_hT=None, err_cT=None, cell_clip=0.0, err_clip=0.0):
    """The forward equations in torch float64; the scalar whose gradient is wanted is sum_t <err_top[t], h_top[t]>
    (+ <err_hT, h_T> + <err_cT, c_T>).  cell_clip > 0 (the reference's --clip-cell): the cell is clamped in the forward
    pass and the gradient passes the clamp unchanged; what flows back into h_{t-1} through the recurrent products, and
    what flows into the layer below through the input products of a layer above the first, is clamped to +-err_clip."""
    td = lambda a: torch.tensor(np.asarray(a, dtype=np.float64), requires_grad=True)
    E = td(embed)
    W = [{"M": [td(m) for m in ly["M"]], "Wh": [td(m) for m in ly["Wh"]], "b": [td(b) for b in ly["b"]]} for ly in layers]
    H0, C0 = [td(a) for a in h0], [td(a) for a in c0]
    T, mb = ids.shape
    L = len(layers)
    h, c = list(H0), list(C0)
    loss = torch.zeros((), dtype=torch.float64)
    for t in range(T):
        m = torch.tensor(mask[t].astype(np.float64))
        x = E[:, torch.tensor(np.maximum(ids[t], 0).astype(np.int64))]
        for l in range(L):
            w = W[l]
            hr = h[l]
            if cell_clip > 0:
                hr = _ClampGradient.apply(hr, err_clip)
                if l > 0:
                    x = _ClampGradient.apply(x, err_clip)
            pre = [w["M"][g] @ x + w["Wh"][g] @ hr + w["b"][g][:, None] for g in range(4)]
            i, f, ct, og = torch.sigmoid(pre[0]), torch.sigmoid(pre[1]), torch.tanh(pre[2]), torch.sigmoid(pre[3])
            cell = f * c[l] + i * ct
            if cell_clip > 0:
                cell = cell + (cell.clamp(-cell_clip, cell_clip) - cell).detach()
            cn = cell * m
            hn = og * torch.tanh(cell) * m
            h[l], c[l] = hn, cn
            x = hn
        loss = loss + (torch.tensor(np.asarray(err_top[t], np.float64)) * h[L - 1]).sum()
    if err_hT is not None:
        for l in range(L):
            loss = loss + (torch.tensor(np.asarray(err_hT[l], np.float64)) * h[l]).sum()
            loss = loss + (torch.tensor(np.asarray(err_cT[l], np.float64)) * c[l]).sum()
    loss.backward()
    return E, W, H0, C0


@pytest.mark.parametrize("L,H,mb,T,V,pad", [(1, 6, 3, 4, 9, False), (3, 10, 5, 6, 20, True), (2, 7, 4, 5, 11, True)])
def test_stack_backward_matches_torch_autograd(L, H, mb, T, V, pad):
    g = synth.rng(101, L * 100 + H)
    embed = U(g, (H, V), -0.5, 0.5)
    layers = [synth.lstm_layer(g, H) for _ in range(L)]
    for ly in layers:
        ly["M"] = [U(g, (H, H), -0.4, 0.4) for _ in range(4)]
        ly["Wh"] = [U(g, (H, H), -0.4, 0.4) for _ in range(4)]
        ly["b"] = [U(g, (H,), -0.3, 0.3) for _ in range(4)]
    ids = g.integers(0, V, size=(T, mb)).astype(np.int32)
    if pad:
        ids[:2, 1] = -1   # left padding (source side)
        ids[T - 1:, 2] = -1  # right padding (target side)
    nn, mask = o.vocab_prep(ids)
    h0 = [U(g, (H, mb), -0.5, 0.5) for _ in range(L)]
    c0 = [U(g, (H, mb), -0.5, 0.5) for _ in range(L)]
    err_top = [U(g, (H, mb), -1, 1) for _ in range(T)]
    err_hT = [U(g, (H, mb), -1, 1) for _ in range(L)]
    err_cT = [U(g, (H, mb), -1, 1) for _ in range(L)]
    grads, d_embed, eh0, ec0 = o.lstm_stack_backward(embed, layers, nn, mask, err_top, h0, c0, err_hT, err_cT)
    E, W, H0, C0 = _torch_stack(embed, layers, ids, mask, h0, c0, err_top, err_hT, err_cT)
    tol = dict(rtol=2e-4, atol=2e-5)  # the oracle stores float32 intermediates
    for l in range(L):
        for q in range(4):
            assert np.allclose(grads[l]["dM"][q], W[l]["M"][q].grad.numpy(), **tol), (l, q, "dM")
            assert np.allclose(grads[l]["dWh"][q], W[l]["Wh"][q].grad.numpy(), **tol), (l, q, "dWh")
            assert np.allclose(grads[l]["db"][q], W[l]["b"][q].grad.numpy(), **tol), (l, q, "db")
        assert np.allclose(eh0[l], H0[l].grad.numpy(), **tol)
        assert np.allclose(ec0[l], C0[l].grad.numpy(), **tol)
    assert np.allclose(d_embed, E.grad.numpy(), **tol)
    # columns of the embedding that no unmasked token selected receive nothing
    used = set(int(v) for v in ids[ids >= 0])
    for v in range(V):
        if v not in used:
            assert np.all(d_embed[:, v] == 0)


@pytest.mark.parametrize("L,H,mb,T,V", [(1, 6, 3, 4, 9), (3, 10, 5, 6, 20)])
def test_stack_backward_with_cell_and_error_clamps_matches_torch_autograd(L, H, mb, T, V):
    """--clip-cell: thresholds small enough that the cell clamp and both error clamps act on a good share of the
    elements (checked), so that a clamp applied at another place -- to the summed error of h_t, to the cell error, to the
    embedding's error -- or left out changes the gradients."""
    g = synth.rng(102, L * 100 + H)
    embed = U(g, (H, V), -0.5, 0.5)
    layers = [synth.lstm_layer(g, H) for _ in range(L)]
    for ly in layers:
        ly["M"] = [U(g, (H, H), -0.6, 0.6) for _ in range(4)]
        ly["Wh"] = [U(g, (H, H), -0.6, 0.6) for _ in range(4)]
        ly["b"] = [U(g, (H,), -0.3, 0.3) for _ in range(4)]
    ids = g.integers(0, V, size=(T, mb)).astype(np.int32)
    ids[:1, 1] = -1
    nn, mask = o.vocab_prep(ids)
    h0 = [U(g, (H, mb), -0.5, 0.5) for _ in range(L)]
    c0 = [U(g, (H, mb), -0.9, 0.9) for _ in range(L)]
    err_top = [U(g, (H, mb), -1, 1) for _ in range(T)]
    cell_clip, err_clip = 0.35, 0.08
    args = (embed, layers, nn, mask, err_top, h0, c0)
    grads, d_embed, eh0, ec0 = o.lstm_stack_backward(*args, cell_clip=cell_clip, err_clip=err_clip)
    plain = o.lstm_stack_backward(*args)
    assert not np.allclose(plain[0][0]["dWh"][0], grads[0]["dWh"][0], rtol=1e-2, atol=1e-3), "the clamps never acted"
    E, W, H0, C0 = _torch_stack(embed, layers, ids, mask, h0, c0, err_top, cell_clip=cell_clip, err_clip=err_clip)
    tol = dict(rtol=2e-4, atol=2e-5)
    for l in range(L):
        for q in range(4):
            assert np.allclose(grads[l]["dM"][q], W[l]["M"][q].grad.numpy(), **tol), (l, q, "dM")
            assert np.allclose(grads[l]["dWh"][q], W[l]["Wh"][q].grad.numpy(), **tol), (l, q, "dWh")
            assert np.allclose(grads[l]["db"][q], W[l]["b"][q].grad.numpy(), **tol), (l, q, "db")
        assert np.allclose(eh0[l], H0[l].grad.numpy(), **tol)
        assert np.allclose(ec0[l], C0[l].grad.numpy(), **tol)
        assert np.abs(eh0[l]).max() <= err_clip + 1e-7
    assert max((np.abs(e) >= err_clip - 1e-7).mean() for e in eh0) > 0.05, "no error of an initial state was clamped"
    assert np.allclose(d_embed, E.grad.numpy(), **tol)
    if L == 1:  # the error reaching the embedding is NOT clamped: some of it exceeds the bound
        assert np.abs(d_embed).max() > err_clip
    # a huge error bound and no cell clamp in reach: the plain gradients
    same = o.lstm_stack_backward(*args, cell_clip=1e6, err_clip=1e6)
    assert np.array_equal(same[1], plain[1]) and all(np.array_equal(a, b) for a, b in zip(same[2], plain[2]))


def test_step_backward_closed_forms():
    g = synth.rng(102, 1)
    H, mb = 5, 4
    gates = {k: U(g, (H, mb), 0.1, 0.9) for k in ("i", "f", "o")}
    gates["c_tilde"] = U(g, (H, mb), -0.9, 0.9)
    cprev = U(g, (H, mb), -1, 1)
    c = np.asfortranarray(gates["f"] * cprev + gates["i"] * gates["c_tilde"])
    err_h, err_c = U(g, (H, mb), -1, 1), U(g, (H, mb), -1, 1)
    mask = np.array([1, 0, 1, 1], np.int32)
    dg, ecp = o.lstm_step_backward(gates, c, cprev, mask, err_h, err_c)
    # masked column: nothing flows
    for k in dg:
        assert np.all(dg[k][:, 1] == 0)
    assert np.all(ecp[:, 1] == 0)
    # hand-written derivative (float64)
    th = np.tanh(c.astype(np.float64))
    ec = err_c + err_h * gates["o"] * (1 - th * th)
    live = [0, 2, 3]
    assert np.allclose(dg["o"][:, live], (err_h * th * gates["o"] * (1 - gates["o"]))[:, live], rtol=1e-5, atol=1e-7)
    assert np.allclose(dg["i"][:, live], (ec * gates["c_tilde"] * gates["i"] * (1 - gates["i"]))[:, live], rtol=1e-5, atol=1e-7)
    assert np.allclose(dg["f"][:, live], (ec * cprev * gates["f"] * (1 - gates["f"]))[:, live], rtol=1e-5, atol=1e-7)
    assert np.allclose(dg["c"][:, live], (ec * gates["i"] * (1 - gates["c_tilde"] ** 2))[:, live], rtol=1e-5, atol=1e-7)
    assert np.allclose(ecp[:, live], (ec * gates["f"])[:, live], rtol=1e-5, atol=1e-7)
    # no error from the cell path and a saturated output gate (o = 1): d o-gate error vanishes
    gates["o"][:] = 1.0
    dg2, _ = o.lstm_step_backward(gates, c, cprev, np.ones(mb, np.int32), err_h, None)
    assert np.all(dg2["o"] == 0)


@pytest.mark.parametrize("V,H,mb", [(13, 5, 4), (40, 8, 6)])
def test_softmax_backward_matches_torch_and_finite_differences(V, H, mb):
    g = synth.rng(103, V)
    D, b, h = U(g, (V, H), -1, 1), U(g, (V,), -1, 1), U(g, (H, mb), -1, 1)
    target = g.integers(0, V, size=mb).astype(np.int32)
    mask = np.ones(mb, np.int32)
    mask[1] = 0
    err_h, dD, db = o.softmax_backward(D, b, h, target, mask)
    Dt, bt, ht = (torch.tensor(a.astype(np.float64), requires_grad=True) for a in (D, b, h))
    logp = torch.log_softmax(Dt @ ht + bt[:, None], dim=0)
    ll = sum(logp[int(target[j]), j] for j in range(mb) if mask[j] == 1)
    ll.backward()
    assert np.allclose(err_h, ht.grad.numpy(), rtol=1e-4, atol=1e-6)
    assert np.allclose(dD, Dt.grad.numpy(), rtol=1e-4, atol=1e-6)
    assert np.allclose(db, bt.grad.numpy(), rtol=1e-4, atol=1e-6)
    assert np.all(err_h[:, 1] == 0)
    # each unmasked column's bias gradient sums to zero (onehot - p), so the whole vector does
    assert abs(db.sum()) < 1e-5
    # central finite difference of the oracle's own loss in one direction of D
    R = U(g, (V, H), -1, 1).astype(np.float64)
    eps = 1e-3
    def loss(Dm):
        lp = o.softmax_logprob_f64(o.softmax_logits(np.asfortranarray(Dm.astype(np.float32)), b, h))
        return o.softmax_loss(lp, target, mask)
    fd = (loss(D + eps * R) - loss(D - eps * R)) / (2 * eps)
    assert fd == pytest.approx(float((dD * R).sum()), rel=2e-3, abs=1e-4)
    # accumulation across calls
    _, dD2, db2 = o.softmax_backward(D, b, h, target, mask, dD.copy(order="F"), db.copy())
    assert np.allclose(dD2, 2 * dD) and np.allclose(db2, 2 * db)


def _torch_attention(w, hs, lens, offs, h_t, mask, D, err_htild):
    """Luong local-p attention from the paper's formulas in torch float64, column by column (window positions are
    integers and carry no gradient); the scalar is <err_htild, h~>.  Returns the leaf tensors with their gradients."""
    td = lambda a: torch.tensor(np.asarray(a, dtype=np.float64), requires_grad=True)
    W = {k: td(w[k]) for k in ("W_a", "W_p", "W_c1", "W_c2")}
    W["v_p"], W["out_bias"] = td(np.asarray(w["v_p"]).reshape(-1)), td(w["out_bias"])
    HS, Ht = td(hs), td(h_t)
    H, mb = h_t.shape
    loss = torch.zeros((), dtype=torch.float64)
    for b in range(mb):
        if not mask[b]:
            continue
        h = Ht[:, b]
        p = float(lens[b]) * torch.sigmoid(W["v_p"] @ torch.tanh(W["W_p"] @ h))
        ip = int(p.item())
        pos = list(range(max(0, ip - D), min(int(lens[b]) - 1, ip + D) + 1))
        src = torch.stack([HS[int(lens[b]) - 1 - s + int(offs[b]), :, b] for s in pos])  # window x H
        sc = src @ (W["W_a"].T @ h)
        a = torch.softmax(sc, 0) * torch.exp(-(p - torch.tensor(pos, dtype=torch.float64)) ** 2 / (2 * (D / 2.0) ** 2))
        c = a @ src
        ht = torch.tanh(W["W_c1"] @ c + W["W_c2"] @ h + W["out_bias"])
        loss = loss + (torch.tensor(np.asarray(err_htild[:, b], np.float64)) * ht).sum()
    loss.backward()
    return W, HS, Ht


@pytest.mark.parametrize("H,mb,S,D,seed", [(10, 6, 9, 2, 1), (16, 5, 12, 12, 2), (7, 4, 30, 3, 3), (12, 3, 5, 1, 4)])
def test_attention_backward_matches_torch_autograd(H, mb, S, D, seed):
    """Every output of the attention backward by value against autograd: the error of h_t, of every source state, and
    the six weight gradients; short sources, a window cut at both ends, a masked column.  A dropped term (the Gaussian's
    derivative through p_t, the soft-max Jacobian's off-diagonal part, the W_p path into h_t) moves the result by far
    more than the tolerance."""
    rng = np.random.default_rng(seed)
    w = dict(W_a=U(rng, (H, H), -0.6, 0.6), W_p=U(rng, (H, H), -0.9, 0.9), v_p=U(rng, (H,), -1.5, 1.5),
             out_bias=U(rng, (H,), -0.3, 0.3), W_c1=U(rng, (H, H), -0.4, 0.4), W_c2=U(rng, (H, H), -0.4, 0.4))
    hs = rng.normal(0, 0.7, size=(S, H, mb)).astype(np.float32)
    lens = rng.integers(1, S + 1, size=mb).astype(np.int32)
    lens[0] = S
    offs = (S - lens).astype(np.int32)
    mask = np.ones(mb, np.int32)
    mask[mb - 2] = 0
    h_t = U(rng, (H, mb), -1, 1)
    err = U(rng, (H, mb), -1, 1)
    binfo = np.concatenate([lens, offs])
    fwd = o.attention_forward(hs_table=hs, batch_info=binfo, h_t=h_t, mask01=mask, D=D, **w)
    # gradients accumulate: start them from a non-zero value and check the increment
    g0 = {k: np.asfortranarray(U(rng, (H, H), -1, 1)) for k in ("W_a", "W_p", "W_c1", "W_c2")}
    g0["v_p"], g0["bias"] = U(rng, (H,), -1, 1), U(rng, (H,), -1, 1)
    ehs0 = rng.normal(0, 1, size=(S, H, mb)).astype(np.float32)
    grads = {k: v.copy(order="F") for k, v in g0.items()}
    err_h, err_hs, grads = o.attention_backward(w["W_a"], w["W_p"], w["v_p"], w["W_c1"], w["W_c2"], hs, binfo, h_t, mask,
                                                fwd, err, D, grads=grads, err_hs=ehs0)
    W, HS, Ht = _torch_attention(w, hs, lens, offs, h_t, mask, D, err)

    def close(got, want, what):
        want = np.asarray(want, np.float64)
        tol = 2e-5 * max(1.0, np.abs(want).max())
        assert np.abs(np.asarray(got, np.float64) - want).max() <= tol, what

    close(err_h, Ht.grad.numpy(), "error of h_t")
    close(err_hs - ehs0, HS.grad.numpy(), "error of the source states")
    for k, t in (("W_a", "W_a"), ("W_p", "W_p"), ("W_c1", "W_c1"), ("W_c2", "W_c2"), ("v_p", "v_p"), ("bias", "out_bias")):
        close(grads[k] - g0[k], W[t].grad.numpy(), "gradient of " + k)
    # the terms a plausible mistake drops are large here
    assert np.abs(W["W_p"].grad.numpy()).max() > 1e-3 and np.abs(W["W_a"].grad.numpy()).max() > 1e-3
    assert np.all(err_h[:, mb - 2] == 0)


def test_dropout_keeps_with_probability_rate_and_rescales():
    """dropout_kernel: `rate` is the KEEP probability; kept values are divided by it, the others become 0."""
    rng = np.random.default_rng(5)
    x = U(rng, (7, 5), -2, 2)
    u = rng.random((7, 5)).astype(np.float32)
    u[0, 0], u[1, 0] = 0.3, np.float32(0.29999998)
    got = o.dropout(u, 0.3, x)
    want = np.where(u < np.float32(0.3), x * (np.float32(1) / np.float32(0.3)), 0).astype(np.float32)
    assert np.array_equal(got, want)  # (a dropped negative value is -0, which equals 0)
    assert got[0, 0] == 0 and got[1, 0] != 0  # strict comparison


def test_lstm_feed_backward_matches_torch_autograd():
    """z_g = Q_g h~ enters gate g's pre-activation: with d_g the pre-activation errors, the error of h~ is
    sum_g Q_g^T d_g and Q_g's gradient d_g h~^T."""
    rng = np.random.default_rng(6)
    H, mb = 9, 4
    Q = [U(rng, (H, H), -1, 1) for _ in range(4)]
    ht = U(rng, (H, mb), -1, 1)
    dg = U(rng, (4 * H, mb), -1, 1)
    dQ0 = [np.asfortranarray(U(rng, (H, H), -1, 1)) for _ in range(4)]
    err, dQ = o.lstm_feed_backward(Q, dg, ht, dQ=[q.copy(order="F") for q in dQ0])
    tQ = [torch.tensor(q.astype(np.float64), requires_grad=True) for q in Q]
    th = torch.tensor(ht.astype(np.float64), requires_grad=True)
    loss = sum((torch.tensor(dg[g * H:(g + 1) * H].astype(np.float64)) * (tQ[g] @ th)).sum() for g in range(4))
    loss.backward()
    assert np.abs(err - th.grad.numpy()).max() < 1e-5
    for g in range(4):
        assert np.abs(dQ[g] - dQ0[g] - tQ[g].grad.numpy()).max() < 1e-5
