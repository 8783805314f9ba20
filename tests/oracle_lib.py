"""ctypes binding of the CPU oracle (oracle/libzoph_oracle.so).

Test infrastructure only: imported by tests/, by the smoke check and by the bench's cpu_baseline leg.
Matrices are numpy float32 arrays in Fortran (column-major) order, as in the reference (IDX2C).
"""
import ctypes as C
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
ORACLE_DIR = os.path.join(os.path.dirname(_HERE), "oracle")
ORACLE_SO = os.path.join(ORACLE_DIR, "libzoph_oracle.so")

_lib = None

f32p = C.POINTER(C.c_float)
f64p = C.POINTER(C.c_double)
i32p = C.POINTER(C.c_int)
f32pp = C.POINTER(f32p)


def build_oracle(force=False):
    if force or not os.path.exists(ORACLE_SO):
        subprocess.check_call(["make", "-C", ORACLE_DIR, "-B" if force else "-s"])
    return ORACLE_SO


def lib():
    global _lib
    if _lib is None:
        build_oracle()
        _lib = C.CDLL(ORACLE_SO)
        _lib.orc_softmax_loss.restype = C.c_double
        _lib.orc_decoder_create.restype = C.c_void_p
        _lib.orc_decoder_create.argtypes = [C.c_int, C.c_int, C.c_int, C.c_int, C.c_int, C.c_float, C.c_float]
        for name in ("orc_decoder_destroy", "orc_decoder_init"):
            getattr(_lib, name).argtypes = [C.c_void_p]
        _lib.orc_decoder_expand.argtypes = [C.c_void_p, f32p, C.c_int]
        _lib.orc_decoder_finish.argtypes = [C.c_void_p, f32p]
        _lib.orc_decoder_state.argtypes = [C.c_void_p, i32p, i32p, f32p, i32p]
        _lib.orc_decoder_expand_viterbi.argtypes = [C.c_void_p, f32p, C.c_int, i32p]
        _lib.orc_decoder_finish_viterbi.argtypes = [C.c_void_p, f32p, i32p]
        _lib.orc_decoder_hypothesis_viterbi.argtypes = [C.c_void_p, C.c_int, i32p, C.c_int]
        _lib.orc_decoder_top_viterbi.argtypes = [C.c_void_p, i32p]
        _lib.orc_decoder_current_index.argtypes = [C.c_void_p]
        _lib.orc_decoder_num_hypotheses.argtypes = [C.c_void_p]
        _lib.orc_decoder_hypothesis.argtypes = [C.c_void_p, C.c_int, i32p, C.c_int, f32p]
        _lib.orc_decoder_k_best.argtypes = [C.c_void_p, C.c_int, C.c_int, i32p]
    return _lib


def F(a, dtype=np.float32):
    """Column-major contiguous array of the given dtype."""
    return np.asfortranarray(np.asarray(a, dtype=dtype))


def _p(a, ct=f32p):
    return a.ctypes.data_as(ct)


def _pp(arrs):
    """float** from a list of float32 arrays (keeps nothing alive: callers hold the arrays)."""
    arr = (f32p * len(arrs))()
    for i, a in enumerate(arrs):
        arr[i] = _p(a) if a is not None else f32p()
    return arr


def num_threads():
    return lib().orc_num_threads()


def vocab_prep(ids):
    ids = np.ascontiguousarray(ids, dtype=np.int32)
    nn = np.empty_like(ids)
    m = np.empty_like(ids)
    lib().orc_vocab_prep(_p(ids, i32p), C.c_int(ids.size), _p(nn, i32p), _p(m, i32p))
    return nn, m


def vocab_softmax(ids):
    ids = np.array(ids, dtype=np.int32, copy=True)
    m = np.empty_like(ids)
    mf = np.empty(ids.shape, dtype=np.float32)
    lib().orc_vocab_softmax(_p(ids, i32p), C.c_int(ids.size), _p(m, i32p), _p(mf))
    return ids, m, mf


def embed_gather(W, ids):
    W = F(W)
    H, V = W.shape
    ids = np.ascontiguousarray(ids, dtype=np.int32)
    x = np.empty((H, ids.size), dtype=np.float32, order="F")
    lib().orc_embed_gather(_p(W), C.c_int(H), C.c_int(V), _p(ids, i32p), C.c_int(ids.size), _p(x))
    return x


def gemm_nn(A, B, acc64=True):
    A, B = F(A), F(B)
    M, K = A.shape
    K2, N = B.shape
    assert K == K2
    Cm = np.empty((M, N), dtype=np.float32, order="F")
    lib().orc_gemm_nn(C.c_int(int(acc64)), C.c_int(M), C.c_int(N), C.c_int(K), _p(A), C.c_int(M), _p(B),
                      C.c_int(K), _p(Cm), C.c_int(M))
    return Cm


def gemm_tn(A, B, acc64=True):
    """A^T @ B with A stored K x M."""
    A, B = F(A), F(B)
    K, M = A.shape
    K2, N = B.shape
    assert K == K2
    Cm = np.empty((M, N), dtype=np.float32, order="F")
    lib().orc_gemm_tn(C.c_int(int(acc64)), C.c_int(M), C.c_int(N), C.c_int(K), _p(A), C.c_int(K), _p(B),
                      C.c_int(K), _p(Cm), C.c_int(M))
    return Cm


def lstm_step(M, Wh, b, x, hprev, cprev, mask01, Q=None, htild=None, clip=None, acc64=True):
    """M, Wh, Q: lists of 4 HxH; b: list of 4 H-vectors (gate order i,f,c,o).  Returns dict of outputs."""
    M = [F(m) for m in M]
    Wh = [F(m) for m in Wh]
    b = [np.ascontiguousarray(v, dtype=np.float32) for v in b]
    x, hprev, cprev = F(x), F(hprev), F(cprev)
    H, mb = x.shape
    mask01 = np.ascontiguousarray(mask01, dtype=np.int32)
    feed = Q is not None and htild is not None
    if feed:
        Q = [F(m) for m in Q]
        htild = F(htild)
    outs = {k: np.empty((H, mb), dtype=np.float32, order="F") for k in ("i", "f", "c_tilde", "o", "c", "h")}
    Mp, Whp, bp = _pp(M), _pp(Wh), _pp(b)
    Qp = _pp(Q) if feed else f32pp()
    lib().orc_lstm_step(C.c_int(int(acc64)), C.c_int(H), C.c_int(mb), Mp, Whp, Qp, bp, _p(x), _p(hprev),
                        _p(cprev), _p(htild) if feed else f32p(), _p(mask01, i32p),
                        C.c_int(0 if clip is None else 1), C.c_float(0.0 if clip is None else clip),
                        _p(outs["i"]), _p(outs["f"]), _p(outs["c_tilde"]), _p(outs["o"]), _p(outs["c"]),
                        _p(outs["h"]))
    return outs


def softmax_logits(D, b_d, h, acc64=True):
    D, h = F(D), F(h)
    V, H = D.shape
    mb = h.shape[1]
    b_d = np.ascontiguousarray(b_d, dtype=np.float32)
    out = np.empty((V, mb), dtype=np.float32, order="F")
    lib().orc_softmax_logits(C.c_int(int(acc64)), _p(D), _p(b_d), C.c_int(V), C.c_int(H), _p(h), C.c_int(mb),
                             _p(out))
    return out


def softmax_dist(logits, emulate_tree=False):
    logits = F(logits)
    V, mb = logits.shape
    out = np.empty((V, mb), dtype=np.float32, order="F")
    lib().orc_softmax_dist(_p(logits), C.c_int(V), C.c_int(mb), C.c_int(int(emulate_tree)), _p(out))
    return out


def softmax_logprob_f64(logits):
    logits = F(logits)
    V, mb = logits.shape
    out = np.empty((V, mb), dtype=np.float64, order="F")
    lib().orc_softmax_logprob_f64(_p(logits), C.c_int(V), C.c_int(mb), _p(out, f64p))
    return out


def softmax_loss(logp, target, mask01):
    logp = F(logp, np.float64)
    V, mb = logp.shape
    target = np.ascontiguousarray(target, dtype=np.int32)
    mask01 = np.ascontiguousarray(mask01, dtype=np.int32)
    return lib().orc_softmax_loss(_p(logp, f64p), C.c_int(V), C.c_int(mb), _p(target, i32p), _p(mask01, i32p))


def attention_forward(W_a, W_p, v_p, out_bias, W_c1, W_c2, hs_table, batch_info, h_t, mask01, D, acc64=True):
    """hs_table: array (S_max, H, mb) of column-major H x mb tables (C-order over the first axis)."""
    W_a, W_p, W_c1, W_c2, h_t = F(W_a), F(W_p), F(W_c1), F(W_c2), F(h_t)
    H, mb = h_t.shape
    v_p = np.ascontiguousarray(v_p, dtype=np.float32).reshape(-1)
    out_bias = np.ascontiguousarray(out_bias, dtype=np.float32)
    hs = pack_hs_table(hs_table)
    batch_info = np.ascontiguousarray(batch_info, dtype=np.int32)
    mask01 = np.ascontiguousarray(mask01, dtype=np.int32)
    Wn = 2 * D + 1
    out = {
        "h_tild": np.empty((H, mb), dtype=np.float32, order="F"),
        "alignments": np.empty((mb, Wn), dtype=np.float32, order="F"),
        "indices": np.empty((mb, Wn), dtype=np.int32, order="F"),
        "p_t": np.empty(mb, dtype=np.float32),
        "c_ctx": np.empty((H, mb), dtype=np.float32, order="F"),
    }
    lib().orc_attention_forward(C.c_int(int(acc64)), C.c_int(H), C.c_int(mb), C.c_int(D), _p(W_a), _p(W_p), _p(v_p),
                                _p(out_bias), _p(W_c1), _p(W_c2), _p(hs), _p(batch_info, i32p), _p(h_t),
                                _p(mask01, i32p), _p(out["h_tild"]), _p(out["alignments"]),
                                _p(out["indices"], i32p), _p(out["p_t"]), _p(out["c_ctx"]))
    return out


def attention_backward(W_a, W_p, v_p, W_c1, W_c2, hs_table, batch_info, h_t, mask01, fwd, err_htild, D, grads=None,
                       err_hs=None):
    """fwd: the dictionary attention_forward returned for the same inputs.  Returns (err_h_t, err_hs, grads); err_hs
    (S, H, mb) and grads {"W_a", "W_p", "v_p", "bias", "W_c1", "W_c2"} are accumulated into when given."""
    W_a, W_p, W_c1, W_c2, h_t, err_htild = F(W_a), F(W_p), F(W_c1), F(W_c2), F(h_t), F(err_htild)
    H, mb = h_t.shape
    v_p = np.ascontiguousarray(v_p, dtype=np.float32).reshape(-1)
    hs = pack_hs_table(hs_table)
    S = np.asarray(hs_table).shape[0]
    batch_info = np.ascontiguousarray(batch_info, dtype=np.int32)
    mask01 = np.ascontiguousarray(mask01, dtype=np.int32)
    if grads is None:
        grads = {k: np.zeros((H, H), np.float32, order="F") for k in ("W_a", "W_p", "W_c1", "W_c2")}
        grads["v_p"] = np.zeros(H, np.float32)
        grads["bias"] = np.zeros(H, np.float32)
    ehs = np.zeros(S * H * mb, np.float32) if err_hs is None else pack_hs_table(err_hs)
    err_h_t = np.empty((H, mb), dtype=np.float32, order="F")
    lib().orc_attention_backward(C.c_int(H), C.c_int(mb), C.c_int(D), _p(W_a), _p(W_p), _p(v_p), _p(W_c1), _p(W_c2),
                                 _p(hs), _p(batch_info, i32p), _p(h_t), _p(mask01, i32p), _p(F(fwd["h_tild"])),
                                 _p(F(fwd["alignments"])), _p(F(fwd["indices"], np.int32), i32p), _p(F(fwd["p_t"])),
                                 _p(F(fwd["c_ctx"])), _p(err_htild), _p(err_h_t), _p(ehs), _p(grads["W_a"]),
                                 _p(grads["W_p"]), _p(grads["v_p"]), _p(grads["bias"]), _p(grads["W_c1"]),
                                 _p(grads["W_c2"]))
    err_hs_out = np.stack([ehs[t * H * mb:(t + 1) * H * mb].reshape(H, mb, order="F") for t in range(S)])
    return err_h_t, err_hs_out, grads


def dropout(uniform, rate, x):
    """dropout_kernel: x * (uniform < rate) / rate; returns a new array."""
    x = F(x).copy(order="F")
    u = F(uniform)
    assert u.shape == x.shape
    lib().orc_dropout(_p(u), C.c_float(rate), _p(x), C.c_size_t(x.size))
    return x


def lstm_feed_backward(Q, dgates, htild, dQ=None):
    """dgates: (4H, mb) stacked pre-activation errors.  Returns (err_htild, dQ list of four H x H)."""
    dgates, htild = F(dgates), F(htild)
    H, mb = htild.shape
    Qs = [F(q) for q in Q]
    dQ = [np.zeros((H, H), np.float32, order="F") for _ in range(4)] if dQ is None else [F(q) for q in dQ]
    err = np.empty((H, mb), dtype=np.float32, order="F")
    lib().orc_lstm_feed_backward(C.c_int(H), C.c_int(mb), _pp(Qs), _p(dgates), _p(htild), _p(err), _pp(dQ))
    return err, dQ


def attention_viterbi(alignments, indices):
    """alignments, indices: (mb, 2D+1) arrays laid out [b + mb*j] (column-major)."""
    al, ix = F(alignments), F(indices, np.int32)
    mb, Wn = al.shape
    out = np.empty(mb, dtype=np.int32)
    lib().orc_attention_viterbi(_p(al), _p(ix, i32p), C.c_int((Wn - 1) // 2), C.c_int(mb), _p(out, i32p))
    return out


def pack_hs_table(hs_table):
    """(S, H, mb) logical array -> flat float32 buffer of S column-major H x mb tables."""
    hs_table = np.asarray(hs_table, dtype=np.float32)
    S, H, mb = hs_table.shape
    flat = np.empty(S * H * mb, dtype=np.float32)
    for t in range(S):
        flat[t * H * mb:(t + 1) * H * mb] = hs_table[t].reshape(-1, order="F")
    return flat


def gather_columns(src, perm):
    src = F(src)
    H = src.shape[0]
    perm = np.ascontiguousarray(perm, dtype=np.int32)
    dst = np.empty((H, perm.size), dtype=np.float32, order="F")
    lib().orc_gather_columns(_p(src), C.c_int(H), _p(perm, i32p), C.c_int(perm.size), _p(dst))
    return dst


def lstm_stack_forward(embed, layers, ids_nonneg, mask01, h0=None, c0=None, clip=None, acc64=True):
    """layers: list of dicts with keys M, Wh, b (lists of 4).  ids_nonneg/mask01: (T, mb) arrays (time-major).
    Returns h_all, c_all with shape (L, T, H, mb) (each [l,t] viewed column-major H x mb)."""
    embed = F(embed)
    H, V = embed.shape
    ids_nonneg = np.ascontiguousarray(ids_nonneg, dtype=np.int32)
    mask01 = np.ascontiguousarray(mask01, dtype=np.int32)
    T, mb = ids_nonneg.shape
    L = len(layers)
    keep = []
    wptrs = (f32p * (12 * L))()
    for l, ly in enumerate(layers):
        mats = [F(m) for m in ly["M"]] + [F(m) for m in ly["Wh"]] + \
               [np.ascontiguousarray(v, dtype=np.float32) for v in ly["b"]]
        keep.append(mats)
        for j, m in enumerate(mats):
            wptrs[12 * l + j] = _p(m)
    n = H * mb
    h0f = np.zeros(L * n, dtype=np.float32) if h0 is None else np.concatenate(
        [F(a).reshape(-1, order="F") for a in h0])
    c0f = np.zeros(L * n, dtype=np.float32) if c0 is None else np.concatenate(
        [F(a).reshape(-1, order="F") for a in c0])
    h_all = np.empty(L * T * n, dtype=np.float32)
    c_all = np.empty(L * T * n, dtype=np.float32)
    lib().orc_lstm_stack_forward(C.c_int(int(acc64)), C.c_int(L), C.c_int(H), C.c_int(mb), C.c_int(T), C.c_int(V),
                                 _p(embed), wptrs, _p(ids_nonneg, i32p), _p(mask01, i32p), _p(h0f), _p(c0f),
                                 C.c_int(0 if clip is None else 1), C.c_float(0.0 if clip is None else clip),
                                 _p(h_all), _p(c_all))

    def view(flat):
        return flat.reshape(L, T, mb, H).transpose(0, 1, 3, 2)  # [l,t] -> (H, mb) with column-major memory

    return view(h_all), view(c_all)


class Decoder:
    """Reference beam search rules (decoder<dType>, non-FSA path)."""

    def __init__(self, beam, vocab, max_len, penalty=0.0, min_ratio=0.0, start_symbol=0, end_symbol=1):
        self.beam, self.vocab, self.max_len = beam, vocab, max_len
        self.h = lib().orc_decoder_create(beam, vocab, start_symbol, end_symbol, max_len, min_ratio, penalty)
        lib().orc_decoder_init(self.h)

    def __del__(self):
        if getattr(self, "h", None):
            lib().orc_decoder_destroy(self.h)
            self.h = None

    def init(self):
        lib().orc_decoder_init(self.h)

    def expand(self, outputdist, index, viterbi=None):
        """viterbi: the attention layer's Viterbi alignment of every beam column (None: the reference's -1)."""
        od = F(outputdist)
        assert od.shape == (self.vocab, self.beam)
        if viterbi is None:
            lib().orc_decoder_expand(self.h, _p(od), index)
        else:
            v = np.ascontiguousarray(viterbi, dtype=np.int32)
            assert v.shape == (self.beam,)
            lib().orc_decoder_expand_viterbi(self.h, _p(od), index, _p(v, i32p))

    def finish(self, outputdist, viterbi=None):
        od = F(outputdist)
        if viterbi is None:
            lib().orc_decoder_finish(self.h, _p(od))
        else:
            v = np.ascontiguousarray(viterbi, dtype=np.int32)
            lib().orc_decoder_finish_viterbi(self.h, _p(od), _p(v, i32p))

    def hypotheses_viterbi(self):
        """Per finished hypothesis: one alignment per word (entry 0 is the initial -20)."""
        out = []
        for i in range(lib().orc_decoder_num_hypotheses(self.h)):
            v = np.empty(self.max_len + 2, dtype=np.int32)
            n = lib().orc_decoder_hypothesis_viterbi(self.h, i, _p(v, i32p), v.size)
            out.append(v[:n].copy())
        return out

    def top_viterbi(self):
        v = np.empty((self.beam, self.max_len), dtype=np.int32)
        lib().orc_decoder_top_viterbi(self.h, _p(v, i32p))
        return v

    def state(self):
        ci = np.empty(self.beam, dtype=np.int32)
        nc = np.empty(self.beam, dtype=np.int32)
        sc = np.empty(self.beam, dtype=np.float32)
        ts = np.empty((self.beam, self.max_len), dtype=np.int32)
        lib().orc_decoder_state(self.h, _p(ci, i32p), _p(nc, i32p), _p(sc), _p(ts, i32p))
        return {"current_indices": ci, "new_indicies_changes": nc, "scores": sc, "top_sentences": ts,
                "current_index": lib().orc_decoder_current_index(self.h)}

    def hypotheses(self):
        out = []
        for i in range(lib().orc_decoder_num_hypotheses(self.h)):
            w = np.empty(self.max_len + 2, dtype=np.int32)
            s = C.c_float()
            n = lib().orc_decoder_hypothesis(self.h, i, _p(w, i32p), w.size, C.byref(s))
            out.append((w[:n].copy(), s.value))
        return out

    def k_best(self, source_length, num_hypotheses):
        idx = np.empty(max(num_hypotheses, 1), dtype=np.int32)
        n = lib().orc_decoder_k_best(self.h, source_length, num_hypotheses, _p(idx, i32p))
        return idx[:n].copy()


def lstm_step_backward(gates, c, cprev, mask01, err_h, err_c_next=None):
    """gates: dict with i, f, c_tilde, o (H x mb).  Returns dgate dict (i, f, c, o pre-activation errors) and
    err_cprev."""
    gi, gf, gc, go = (F(gates[k]) for k in ("i", "f", "c_tilde", "o"))
    c, cprev, err_h = F(c), F(cprev), F(err_h)
    H, mb = c.shape
    mask01 = np.ascontiguousarray(mask01, dtype=np.int32)
    ecn = F(err_c_next) if err_c_next is not None else None
    outs = [np.empty((H, mb), dtype=np.float32, order="F") for _ in range(5)]
    lib().orc_lstm_step_backward(C.c_int(H), C.c_int(mb), _p(gi), _p(gf), _p(gc), _p(go), _p(c), _p(cprev),
                                 _p(mask01, i32p), _p(err_h), _p(ecn) if ecn is not None else None,
                                 *[_p(a) for a in outs])
    return {"i": outs[0], "f": outs[1], "c": outs[2], "o": outs[3]}, outs[4]


def lstm_stack_backward(embed, layers, ids_nonneg, mask01, err_top, h0=None, c0=None, err_hT=None, err_cT=None,
                        cell_clip=0.0, err_clip=0.0):
    """Back-propagation through time of the stacked LSTM (gradients of a loss whose derivative with respect to the top
    layer's h_t is err_top[t], H x mb each).  Returns (grads, d_embed, err_h0, err_c0): grads[l] = dict with dM, dWh
    (lists of 4 H x H) and db (list of 4 H); d_embed H x V; err_h0 / err_c0 lists of L (H x mb).
    cell_clip > 0: the reference's --clip-cell mode (cell clamp in the forward sweep, errors to h_{t-1} and to the layer
    below clamped to +-err_clip)."""
    embed = F(embed)
    H, V = embed.shape
    ids_nonneg = np.ascontiguousarray(ids_nonneg, dtype=np.int32)
    mask01 = np.ascontiguousarray(mask01, dtype=np.int32)
    T, mb = ids_nonneg.shape
    L = len(layers)
    n = H * mb
    keep = []
    wptrs = (f32p * (12 * L))()
    gptrs = (f32p * (12 * L))()
    gmats = []
    for l, ly in enumerate(layers):
        mats = [F(m) for m in ly["M"]] + [F(m) for m in ly["Wh"]] + \
               [np.ascontiguousarray(v, dtype=np.float32) for v in ly["b"]]
        keep.append(mats)
        gl = [np.zeros((H, H), dtype=np.float32, order="F") for _ in range(8)] + \
             [np.zeros(H, dtype=np.float32) for _ in range(4)]
        gmats.append(gl)
        for j in range(12):
            wptrs[12 * l + j] = _p(mats[j])
            gptrs[12 * l + j] = _p(gl[j])

    def flat(arrs):
        if arrs is None:
            return np.zeros(L * n, dtype=np.float32)
        return np.concatenate([F(a).reshape(-1, order="F") for a in arrs])

    h0f, c0f = flat(h0), flat(c0)
    ehT = flat(err_hT) if err_hT is not None else None
    ecT = flat(err_cT) if err_cT is not None else None
    et = np.concatenate([F(err_top[t]).reshape(-1, order="F") for t in range(T)])
    d_embed = np.zeros((H, V), dtype=np.float32, order="F")
    eh0, ec0 = np.empty(L * n, dtype=np.float32), np.empty(L * n, dtype=np.float32)
    lib().orc_lstm_stack_backward_clip(C.c_int(L), C.c_int(H), C.c_int(mb), C.c_int(T), C.c_int(V), _p(embed), wptrs,
                                       _p(ids_nonneg, i32p), _p(mask01, i32p), _p(h0f), _p(c0f), _p(et),
                                       _p(ehT) if ehT is not None else None, _p(ecT) if ecT is not None else None,
                                       C.c_float(cell_clip), C.c_float(err_clip), gptrs, _p(d_embed), _p(eh0), _p(ec0))
    grads = [{"dM": gl[0:4], "dWh": gl[4:8], "db": gl[8:12]} for gl in gmats]
    unflat = lambda f: [f[l * n:(l + 1) * n].reshape(H, mb, order="F") for l in range(L)]
    return grads, d_embed, unflat(eh0), unflat(ec0)


def softmax_backward(D, b_d, h, target, mask01, dD=None, db=None):
    """Returns err_h (H x mb), dD (V x H, float64), db (V, float64); dD / db given: accumulated into."""
    D, h = F(D), F(h)
    V, H = D.shape
    mb = h.shape[1]
    b_d = np.ascontiguousarray(b_d, dtype=np.float32)
    target = np.ascontiguousarray(target, dtype=np.int32)
    mask01 = np.ascontiguousarray(mask01, dtype=np.int32)
    add = dD is not None
    if add:
        assert dD.flags.f_contiguous and dD.dtype == np.float64 and db.dtype == np.float64, "dD must be column-major f64"
    if not add:
        dD = np.zeros((V, H), dtype=np.float64, order="F")
        db = np.zeros(V, dtype=np.float64)
    err_h = np.empty((H, mb), dtype=np.float32, order="F")
    lib().orc_softmax_backward(_p(D), _p(b_d), C.c_int(V), C.c_int(H), _p(h), C.c_int(mb), _p(target, i32p),
                               _p(mask01, i32p), C.c_int(int(add)), _p(err_h), _p(dD, f64p), _p(db, f64p))
    return err_h, dD, db
