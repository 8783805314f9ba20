"""ctypes binding of the C-ABI in include/zoph_rnn.h (libzoph_rnn_hip.so).

This is plumbing for tests and the benchmark: device buffers, numpy <-> device copies and one thin Python
function per entry point.  There is no CPU fallback: importing works without a GPU (so the symbol table can be
checked), but every compute call needs the built library and a device, and raises otherwise.
"""
import ctypes as C
import os

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "libzoph_rnn_hip.so")

ZR_OPT_LSTM_FUSED_EPILOGUE = 1
ZR_OPT_LSTM_TN = 2
ZR_OPT_GEMM_CFG = 3
ZR_OPT_LSTM_KSPLIT = 4
ZR_OPT_LSTM_KERNEL = 5
ZR_OPT_LSTM_KPARTS = 6
ZR_OPT_LSTM_SWEEP = 7
ZR_OPT_LSTM_SWEEP_SPIN = 8
ZR_OPT_BF16_ACTIVATION_TERMS = 9
ZR_OPT_LSTM_STEP_WAIT_EXTRA = 10
ZR_OPT_ATTN_SINGLE_LAUNCH = 11
ZR_QUERY_LSTM_STACK_PATH = 1
ZR_QUERY_LSTM_SWEEP_ABANDONED = 2
ZR_QUERY_ATTN_PATH = 3
ZR_QUERY_SCRATCH_KIB = 4
ZR_ATTN_PATH_SINGLE_LAUNCH = 1
ZR_ATTN_PATH_THREE_LAUNCHES = 2
ZR_ATTN_PATH_SEPARATE = 3
ZR_LSTM_STACK_PATH_SWEEP = 1
ZR_LSTM_STACK_PATH_DIAGONALS = 2
ZR_LSTM_STACK_PATH_STEP_SINGLE_LAUNCH = 3
ZR_LSTM_STACK_PATH_STEP_PER_LAYER = 4
ZR_SOFTMAX_PROB = 0
ZR_SOFTMAX_LOGPROB = 1
ZR_CLIP_NONE, ZR_CLIP_MATRIX_NORM, ZR_CLIP_WHOLE_NORM, ZR_CLIP_ELEMENT = 0, 1, 2, 3
ZR_SOFTMAX_LOGITS = 2  # d_out: V*mb logits followed by 2*mb column statistics (max, sum of exp(x - max))
ZR_SOFTMAX_LOGITS_BLOCKS = 3  # d_out: the logits, then (max, sum exp) per 32-row block and column at softmax_blocks_offset

# every symbol include/zoph_rnn.h declares
SYMBOLS = [
    "zr_ctx_create", "zr_ctx_destroy", "zr_ctx_sync", "zr_ctx_set_stream", "zr_ctx_set_option", "zr_last_error",
    "zr_version", "zr_timer_start", "zr_timer_stop", "zr_malloc", "zr_free", "zr_h2d", "zr_d2h", "zr_d2d", "zr_memset_zero", "zr_vocab_prep",
    "zr_vocab_prep_softmax", "zr_embed_gather", "zr_lstm_pack_weights", "zr_lstm_pack_weights_bf16", "zr_lstm_weights_destroy", "zr_lstm_step",
    "zr_lstm_gates", "zr_lstm_stack_forward", "zr_gemm", "zr_softmax_prepare", "zr_softmax_prepare_bf16", "zr_softmax_release", "zr_softmax_forward", "zr_softmax_logprob_f64",
    "zr_softmax_loss", "zr_attn_create", "zr_attn_use_bf16_weights", "zr_attn_destroy", "zr_attn_step", "zr_gather_columns",
    "zr_broadcast_column", "zr_beam_create", "zr_beam_destroy", "zr_beam_init", "zr_beam_expand", "zr_beam_finish", "zr_beam_expand_logits", "zr_beam_finish_logits",
    "zr_beam_expand_blocks", "zr_beam_finish_blocks", "zr_softmax_block_count", "zr_softmax_blocks_offset",
    "zr_beam_hypotheses", "zr_beam_state", "zr_beam_set_viterbi", "zr_beam_set_input_ids", "zr_beam_hypotheses_viterbi", "zr_ensemble_average",
    "zr_attn_viterbi_ensemble",
    "zr_lstm_stack_forward_train", "zr_lstm_train_create", "zr_lstm_train_refresh", "zr_lstm_train_destroy",
    "zr_unstack_gates", "zr_lstm_stack_backward", "zr_lstm_weight_gradients", "zr_embed_gradient",
    "zr_softmax_backward", "zr_sgd_update", "zr_grad_sumsq_accumulate", "zr_sgd_update_clipped", "zr_clip_inplace", "zr_lstm_stack_backward_clamped", "zr_lstm_node_backward", "zr_lstm_node_gradients",
    "zr_softmax_backward_accumulate", "zr_gather_columns_multi", "zr_softmax_backward_loss",
    "zr_softmax_forward_static", "zr_ctx_query", "zr_attn_prepare", "zr_lstm_step_embed", "zr_attn_viterbi", "zr_lstm_decoder_step", "zr_decoder_step", "zr_lstm_feed_backward", "zr_attn_set_error_tables",
    "zr_attn_backward", "zr_dropout_apply", "zr_uniform_fill", "zr_add_inplace",
]

_lib = None


class ZrError(RuntimeError):
    def __init__(self, code, msg):
        super().__init__("zoph_rnn error %d: %s" % (code, msg))
        self.code = code


def load():
    """Loads the HIP library; raises if it has not been built (no fallback path exists)."""
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            raise RuntimeError("%s is missing: run `python __graft_entry__.py build` (or zoph_rnn_amd/build.py) first; "
                               "there is no CPU fallback for the HIP path" % LIB_PATH)
        _lib = C.CDLL(LIB_PATH)
        _lib.zr_last_error.restype = C.c_char_p
        _lib.zr_version.restype = C.c_char_p
        _lib.zr_softmax_blocks_offset.restype = C.c_longlong
    return _lib


def softmax_block_count(V):
    return int(load().zr_softmax_block_count(C.c_int(V)))


def softmax_blocks_offset(V, cols):
    """ZR_SOFTMAX_LOGITS_BLOCKS: where the per-block pairs start in d_out, in floats."""
    return int(load().zr_softmax_blocks_offset(C.c_int(V), C.c_int(cols)))


def _chk(rc):
    if rc != 0:
        raise ZrError(rc, load().zr_last_error().decode())


def _vp(x):
    """void* for a DeviceArray, raw int address, or None."""
    if x is None:
        return C.c_void_p(None)
    if isinstance(x, DeviceArray):
        return C.c_void_p(x.ptr)
    return C.c_void_p(int(x))


class DeviceArray:
    """A device allocation with a numpy-like shape/dtype.  2-D arrays are column-major (Fortran order)."""

    def __init__(self, ctx, shape, dtype=np.float32, zero=False):
        self.ctx = ctx
        self.shape = tuple(int(s) for s in (shape if isinstance(shape, (tuple, list)) else (shape,)))
        self.dtype = np.dtype(dtype)
        self.nbytes = int(np.prod(self.shape, dtype=np.int64)) * self.dtype.itemsize
        p = C.c_void_p()
        _chk(load().zr_malloc(ctx.h, C.c_size_t(max(self.nbytes, 4)), C.byref(p)))
        self.ptr = p.value
        self._owned = True
        if zero and self.nbytes:
            _chk(load().zr_memset_zero(ctx.h, C.c_void_p(self.ptr), C.c_size_t((self.nbytes + 3) // 4 * 4)))

    @classmethod
    def from_numpy(cls, ctx, a, dtype=None):
        a = np.asarray(a, dtype=dtype if dtype is not None else a.dtype)
        d = cls(ctx, a.shape, a.dtype)
        d.set(a)
        return d

    def set(self, a):
        a = np.asfortranarray(np.asarray(a, dtype=self.dtype))
        assert a.shape == self.shape, (a.shape, self.shape)
        flat = a.reshape(-1, order="F")
        _chk(load().zr_h2d(self.ctx.h, C.c_void_p(self.ptr), flat.ctypes.data_as(C.c_void_p), C.c_size_t(self.nbytes)))

    def get(self):
        flat = np.empty(int(np.prod(self.shape, dtype=np.int64)), dtype=self.dtype)
        _chk(load().zr_d2h(self.ctx.h, flat.ctypes.data_as(C.c_void_p), C.c_void_p(self.ptr), C.c_size_t(self.nbytes)))
        return flat.reshape(self.shape, order="F")

    def at(self, elem_offset):
        """Raw device address elem_offset elements into the buffer."""
        return self.ptr + int(elem_offset) * self.dtype.itemsize

    def free(self):
        if self._owned and self.ptr:
            load().zr_free(self.ctx.h, C.c_void_p(self.ptr))
            self.ptr = 0

    def __del__(self):
        try:
            if self.ctx.h:
                self.free()
        except Exception:
            pass


def _ptr_array(items):
    arr = (C.c_void_p * len(items))()
    for i, it in enumerate(items):
        arr[i] = it.ptr if isinstance(it, DeviceArray) else (None if it is None else int(it))
    return arr


class Context:
    def __init__(self, device=0):
        self.h = C.c_void_p()
        _chk(load().zr_ctx_create(C.c_int(device), C.byref(self.h)))

    def close(self):
        if self.h:
            load().zr_ctx_destroy(self.h)
            self.h = C.c_void_p()

    def sync(self):
        _chk(load().zr_ctx_sync(self.h))

    def timer_start(self):
        _chk(load().zr_timer_start(self.h))

    def timer_stop(self):
        ms = C.c_float()
        _chk(load().zr_timer_stop(self.h, C.byref(ms)))
        return ms.value

    def query(self, what):
        v = C.c_int(0)
        _chk(load().zr_ctx_query(self.h, C.c_int(what), C.byref(v)))
        return v.value

    def set_option(self, opt, value):
        _chk(load().zr_ctx_set_option(self.h, C.c_int(opt), C.c_int(value)))

    def array(self, a, dtype=None):
        return DeviceArray.from_numpy(self, a, dtype)

    def empty(self, shape, dtype=np.float32):
        return DeviceArray(self, shape, dtype)

    def zeros(self, shape, dtype=np.float32):
        return DeviceArray(self, shape, dtype, zero=True)

    def memset_zero(self, d_arr):
        _chk(load().zr_memset_zero(self.h, C.c_void_p(d_arr.ptr), C.c_size_t((d_arr.nbytes + 3) // 4 * 4)))

    # ---- A1
    def vocab_prep(self, d_ids, n, vocab, d_nonneg, d_mask):
        _chk(load().zr_vocab_prep(self.h, _vp(d_ids), C.c_int(n), C.c_int(vocab), _vp(d_nonneg), _vp(d_mask)))

    def vocab_prep_softmax(self, d_ids, n, vocab, d_mask, d_maskf):
        _chk(load().zr_vocab_prep_softmax(self.h, _vp(d_ids), C.c_int(n), C.c_int(vocab), _vp(d_mask), _vp(d_maskf)))

    # ---- A2
    def embed_gather(self, d_W, H, V, d_ids, mb, d_x):
        _chk(load().zr_embed_gather(self.h, _vp(d_W), C.c_int(H), C.c_int(V), _vp(d_ids), C.c_int(mb), _vp(d_x)))

    # ---- A3-A5
    def lstm_pack(self, M, Wh, b, H, Q=None, bf16=False):
        w = C.c_void_p()
        fn = load().zr_lstm_pack_weights_bf16 if bf16 else load().zr_lstm_pack_weights
        _chk(fn(self.h, _ptr_array(M), _ptr_array(Wh), _ptr_array(Q) if Q else None, _ptr_array(b), C.c_int(H),
                C.byref(w)))
        return w

    def lstm_weights_destroy(self, w):
        _chk(load().zr_lstm_weights_destroy(self.h, w))

    def lstm_step(self, w, d_in, d_hprev, d_cprev, d_mask, mb, d_h, d_c, d_htild=None, clip=0.0, gates=None):
        _chk(load().zr_lstm_step(self.h, w, _vp(d_in), _vp(d_hprev), _vp(d_cprev), _vp(d_htild), _vp(d_mask),
                                 C.c_float(clip), C.c_int(mb), _vp(d_h), _vp(d_c),
                                 _ptr_array(gates) if gates else None))

    def lstm_step_embed(self, w, d_embed, V, d_ids, d_hprev, d_cprev, d_mask, mb, d_h, d_c, d_htild=None, clip=0.0,
                        gates=None):
        _chk(load().zr_lstm_step_embed(self.h, w, _vp(d_embed), C.c_int(V), _vp(d_ids), _vp(d_hprev), _vp(d_cprev),
                                       _vp(d_htild), _vp(d_mask), C.c_float(clip), C.c_int(mb), _vp(d_h), _vp(d_c),
                                       _ptr_array(gates) if gates else None))

    def lstm_decoder_step(self, layers, d_embed, V, d_ids, hprev, cprev, d_mask, mb, h, c, d_htild=None, clip=0.0):
        L = len(layers)
        larr = (C.c_void_p * L)(*[w.value for w in layers])
        _chk(load().zr_lstm_decoder_step(self.h, C.c_int(L), larr, _vp(d_embed), C.c_int(V), _vp(d_ids),
                                         _ptr_array(hprev), _ptr_array(cprev), _vp(d_htild), _vp(d_mask),
                                         C.c_float(clip), C.c_int(mb), _ptr_array(h), _ptr_array(c)))

    def decoder_step(self, layers, d_embed, V_in, d_ids, hprev, cprev, d_mask, mb, h, c, attn, d_batch_info, d_htild, d_D,
                     d_b_d, V_out, mode, d_out, d_htild_prev=None, clip=0.0, d_align=None, d_idx=None, d_pt=None,
                     d_ctx=None):
        L = len(layers)
        larr = (C.c_void_p * L)(*[w.value for w in layers])
        _chk(load().zr_decoder_step(self.h, C.c_int(L), larr, _vp(d_embed), C.c_int(V_in), _vp(d_ids), _ptr_array(hprev),
                                    _ptr_array(cprev), _vp(d_htild_prev), _vp(d_mask), C.c_float(clip), C.c_int(mb),
                                    _ptr_array(h), _ptr_array(c), attn, _vp(d_batch_info), _vp(d_htild), _vp(d_align),
                                    _vp(d_idx), _vp(d_pt), _vp(d_ctx), _vp(d_D), _vp(d_b_d), C.c_int(V_out), C.c_int(mode),
                                    _vp(d_out)))

    def lstm_gates(self, d_preact, b, d_cprev, d_mask, H, mb, d_h, d_c, clip=0.0, gates=None):
        _chk(load().zr_lstm_gates(self.h, _vp(d_preact), _ptr_array(b), _vp(d_cprev), _vp(d_mask), C.c_float(clip),
                                  C.c_int(H), C.c_int(mb), _vp(d_h), _vp(d_c), _ptr_array(gates) if gates else None))

    def lstm_stack_forward(self, layers, d_embed, V, d_ids, d_mask, T, mb, h0, c0, h_all, c_all, clip=0.0):
        L = len(layers)
        larr = (C.c_void_p * L)(*[w.value for w in layers])
        _chk(load().zr_lstm_stack_forward(self.h, C.c_int(L), larr, _vp(d_embed), C.c_int(V), _vp(d_ids), _vp(d_mask),
                                          C.c_int(T), C.c_int(mb), _ptr_array(h0), _ptr_array(c0), C.c_float(clip),
                                          _ptr_array(h_all), _ptr_array(c_all)))

    def gemm(self, trans_a, M, N, K, d_A, lda, d_B, ldb, d_C, ldc):
        _chk(load().zr_gemm(self.h, C.c_int(trans_a), C.c_int(M), C.c_int(N), C.c_int(K), _vp(d_A), C.c_int(lda),
                            _vp(d_B), C.c_int(ldb), _vp(d_C), C.c_int(ldc)))

    # ---- F4: training backward
    def lstm_stack_forward_train(self, layers, d_embed, V, d_ids, d_mask, T, mb, h0, c0, h_all, c_all, gates_all,
                                 clip=0.0):
        L = len(layers)
        larr = (C.c_void_p * L)(*[w.value for w in layers])
        _chk(load().zr_lstm_stack_forward_train(self.h, C.c_int(L), larr, _vp(d_embed), C.c_int(V), _vp(d_ids),
                                                _vp(d_mask), C.c_int(T), C.c_int(mb), _ptr_array(h0), _ptr_array(c0),
                                                C.c_float(clip), _ptr_array(h_all), _ptr_array(c_all),
                                                _ptr_array(gates_all)))

    def lstm_train_create(self, M, Wh, H):
        w = C.c_void_p()
        _chk(load().zr_lstm_train_create(self.h, _ptr_array(M), _ptr_array(Wh), C.c_int(H), C.byref(w)))
        return w

    def lstm_train_refresh(self, w, M, Wh):
        _chk(load().zr_lstm_train_refresh(self.h, w, _ptr_array(M), _ptr_array(Wh)))

    def lstm_train_destroy(self, w):
        _chk(load().zr_lstm_train_destroy(self.h, w))

    def unstack_gates(self, d_stack, H, outs):
        _chk(load().zr_unstack_gates(self.h, _vp(d_stack), C.c_int(H), _ptr_array(outs)))

    def lstm_stack_backward(self, layers, T, mb, d_mask, c0, c_all, gates_all, d_err_top, dgates_all, err_h0, err_c0,
                            err_hT=None, err_cT=None, d_err_below0=None, err_clip=0.0):
        """err_clip > 0: the error clamps of the reference's --clip-cell mode (zr_lstm_stack_backward_clamped)."""
        L = len(layers)
        larr = (C.c_void_p * L)(*[w.value for w in layers])
        _chk(load().zr_lstm_stack_backward_clamped(self.h, C.c_int(L), larr, C.c_int(T), C.c_int(mb), _vp(d_mask),
                                                   _ptr_array(c0), _ptr_array(c_all), _ptr_array(gates_all),
                                                   _vp(d_err_top), _ptr_array(err_hT) if err_hT else None,
                                                   _ptr_array(err_cT) if err_cT else None, _ptr_array(dgates_all),
                                                   _vp(d_err_below0), _ptr_array(err_h0), _ptr_array(err_c0),
                                                   C.c_float(err_clip)))

    def lstm_weight_gradients(self, H, T, mb, d_dgates, d_in_all, d_h0, d_h_all, d_dM, d_dWh, d_db):
        _chk(load().zr_lstm_weight_gradients(self.h, C.c_int(H), C.c_int(T), C.c_int(mb), _vp(d_dgates), _vp(d_in_all),
                                             _vp(d_h0), _vp(d_h_all), _vp(d_dM), _vp(d_dWh), _vp(d_db)))

    def lstm_feed_backward(self, Q, H, mb, d_dgates, d_htild, d_err_htild, d_dQ_stack):
        _chk(load().zr_lstm_feed_backward(self.h, _ptr_array(Q), C.c_int(H), C.c_int(mb), _vp(d_dgates), _vp(d_htild),
                                          _vp(d_err_htild), _vp(d_dQ_stack)))

    def attn_set_error_tables(self, attn, tables):
        _chk(load().zr_attn_set_error_tables(self.h, attn, _ptr_array(tables), C.c_int(len(tables))))

    def attn_backward(self, attn, d_batch_info, d_h_t, d_mask, d_h_tild, d_align, d_idx, d_p_t, d_c_t, d_err_htild,
                      d_err_h_t, grads):
        """grads: six device arrays in the order W_a, W_p, v_p, out_bias, W_c1, W_c2 (accumulated into)."""
        g = _ptr_array(grads)  # zr_attn_grads: six pointers
        _chk(load().zr_attn_backward(self.h, attn, _vp(d_batch_info), _vp(d_h_t), _vp(d_mask), _vp(d_h_tild), _vp(d_align),
                                     _vp(d_idx), _vp(d_p_t), _vp(d_c_t), _vp(d_err_htild), _vp(d_err_h_t), g))

    def add_inplace(self, d_dst, d_src, n):
        _chk(load().zr_add_inplace(self.h, _vp(d_dst), _vp(d_src), C.c_longlong(n)))

    def dropout_apply(self, d_uniform, keep_rate, d_x, n):
        _chk(load().zr_dropout_apply(self.h, _vp(d_uniform), C.c_float(keep_rate), _vp(d_x), C.c_longlong(n)))

    def uniform_fill(self, seed, call, d_out, n):
        _chk(load().zr_uniform_fill(self.h, C.c_ulonglong(seed), C.c_ulonglong(call), _vp(d_out), C.c_longlong(n)))

    def lstm_node_backward(self, layer, mb, gates, d_c, d_c_prev, d_mask, d_err_above, d_err_h_next, d_err_c_next,
                           d_dgates, d_err_h_prev, d_err_c_prev, d_err_below=None):
        _chk(load().zr_lstm_node_backward(self.h, layer, C.c_int(mb), _ptr_array(gates), _vp(d_c), _vp(d_c_prev),
                                          _vp(d_mask), _vp(d_err_above), _vp(d_err_h_next), _vp(d_err_c_next),
                                          _vp(d_dgates), _vp(d_err_h_prev), _vp(d_err_c_prev), _vp(d_err_below)))

    def lstm_node_gradients(self, H, mb, d_dgates, d_in, d_h_prev, d_dM, d_dWh, d_db):
        _chk(load().zr_lstm_node_gradients(self.h, C.c_int(H), C.c_int(mb), _vp(d_dgates), _vp(d_in), _vp(d_h_prev),
                                           _vp(d_dM), _vp(d_dWh), _vp(d_db)))

    def embed_gradient(self, H, V, d_err, d_ids, d_mask, n, d_dW):
        _chk(load().zr_embed_gradient(self.h, C.c_int(H), C.c_int(V), _vp(d_err), _vp(d_ids), _vp(d_mask), C.c_int(n),
                                      _vp(d_dW)))

    def softmax_backward(self, d_D, d_b, V, H, d_h, n, d_target, d_mask, d_scratch, d_err_h, d_dD, d_db,
                         accumulate=False):
        fn = load().zr_softmax_backward_accumulate if accumulate else load().zr_softmax_backward
        _chk(fn(self.h, _vp(d_D), _vp(d_b), C.c_int(V), C.c_int(H), _vp(d_h), C.c_int(n),
                                        _vp(d_target), _vp(d_mask), _vp(d_scratch), _vp(d_err_h), _vp(d_dD), _vp(d_db)))

    def softmax_backward_loss(self, d_D, d_b, V, H, d_h, n, d_target, d_mask, d_scratch, d_err_h, d_dD, d_db):
        """softmax_backward plus the log-likelihood of the n columns (returned)."""
        loss = C.c_double(0.0)
        _chk(load().zr_softmax_backward_loss(self.h, _vp(d_D), _vp(d_b), C.c_int(V), C.c_int(H), _vp(d_h), C.c_int(n),
                                             _vp(d_target), _vp(d_mask), _vp(d_scratch), _vp(d_err_h), _vp(d_dD),
                                             _vp(d_db), C.byref(loss)))
        return loss.value

    def sgd_update(self, d_W, d_grad, n, scale, norm_clip, lr):
        _chk(load().zr_sgd_update(self.h, _vp(d_W), _vp(d_grad), C.c_longlong(n), C.c_float(scale), C.c_float(norm_clip),
                                  C.c_float(lr)))

    def clip_inplace(self, d_x, n, threshold):
        _chk(load().zr_clip_inplace(self.h, _vp(d_x), C.c_longlong(n), C.c_float(threshold)))

    def grad_sumsq_accumulate(self, d_grad, n, scale, d_sumsq, reset=False):
        """d_sumsq: device array of one float64"""
        _chk(load().zr_grad_sumsq_accumulate(self.h, _vp(d_grad), C.c_longlong(n), C.c_float(scale), _vp(d_sumsq),
                                             C.c_int(1 if reset else 0)))

    def sgd_update_clipped(self, d_W, d_grad, n, scale, clip_mode, threshold, d_sumsq, lr):
        _chk(load().zr_sgd_update_clipped(self.h, _vp(d_W), _vp(d_grad), C.c_longlong(n), C.c_float(scale),
                                          C.c_int(clip_mode), C.c_float(threshold), _vp(d_sumsq), C.c_float(lr)))

    # ---- A8/A9
    def softmax_prepare(self, d_D, V, H, bf16=False):
        fn = load().zr_softmax_prepare_bf16 if bf16 else load().zr_softmax_prepare
        _chk(fn(self.h, _vp(d_D), C.c_int(V), C.c_int(H)))

    def softmax_release(self, d_D):
        _chk(load().zr_softmax_release(self.h, _vp(d_D)))

    def softmax_forward(self, d_D, d_b, V, H, d_h, mb, mode, d_out, d_scratch=None, static=False):
        """static=True: the allocation-free entry point (scratch in the library's static device array)."""
        fn = load().zr_softmax_forward_static if static else load().zr_softmax_forward
        _chk(fn(self.h, _vp(d_D), _vp(d_b), C.c_int(V), C.c_int(H), _vp(d_h), C.c_int(mb),
                C.c_int(mode), _vp(d_out), _vp(d_scratch)))

    def softmax_logprob_f64(self, d_D, d_b, V, H, d_h, mb, d_logp, d_scratch):
        _chk(load().zr_softmax_logprob_f64(self.h, _vp(d_D), _vp(d_b), C.c_int(V), C.c_int(H), _vp(d_h), C.c_int(mb),
                                           _vp(d_logp), _vp(d_scratch)))

    def softmax_loss(self, d_D, d_b, V, H, d_h, mb, d_target, d_mask, d_scratch):
        loss = C.c_double()
        _chk(load().zr_softmax_loss(self.h, _vp(d_D), _vp(d_b), C.c_int(V), C.c_int(H), _vp(d_h), C.c_int(mb),
                                    _vp(d_target), _vp(d_mask), _vp(d_scratch), C.byref(loss)))
        return loss.value

    # ---- A10
    def attn_create(self, H, mb, D, W_a, W_p, v_p, out_bias, W_c1, W_c2, hs_tables):
        a = C.c_void_p()
        tab = _ptr_array(hs_tables)
        _chk(load().zr_attn_create(self.h, C.c_int(H), C.c_int(mb), C.c_int(D), _vp(W_a), _vp(W_p), _vp(v_p),
                                   _vp(out_bias), _vp(W_c1), _vp(W_c2), tab, C.c_int(len(hs_tables)), C.byref(a)))
        return a

    def attn_use_bf16_weights(self, a):
        _chk(load().zr_attn_use_bf16_weights(self.h, a))

    def attn_viterbi(self, a, d_align, d_idx, d_out):
        _chk(load().zr_attn_viterbi(self.h, a, _vp(d_align), _vp(d_idx), _vp(d_out)))

    def attn_prepare(self, a):
        _chk(load().zr_attn_prepare(self.h, a))

    def attn_destroy(self, a):
        _chk(load().zr_attn_destroy(self.h, a))

    def attn_step(self, a, d_batch_info, d_h_t, d_mask, d_htild, d_align=None, d_idx=None, d_pt=None, d_ctx=None):
        _chk(load().zr_attn_step(self.h, a, _vp(d_batch_info), _vp(d_h_t), _vp(d_mask), _vp(d_htild), _vp(d_align),
                                 _vp(d_idx), _vp(d_pt), _vp(d_ctx)))

    # ---- A12
    def gather_columns(self, d_src, H, d_perm, n, d_dst):
        _chk(load().zr_gather_columns(self.h, _vp(d_src), C.c_int(H), _vp(d_perm), C.c_int(n), _vp(d_dst)))

    def gather_columns_multi(self, srcs, H, d_perm, n_src_cols, n, dsts):
        _chk(load().zr_gather_columns_multi(self.h, C.c_int(len(srcs)), _ptr_array(srcs), C.c_int(H), _vp(d_perm),
                                            C.c_int(n_src_cols), C.c_int(n), _ptr_array(dsts)))

    def broadcast_column(self, d_src_col, H, n, d_dst):
        _chk(load().zr_broadcast_column(self.h, _vp(d_src_col), C.c_int(H), C.c_int(n), _vp(d_dst)))

    # ---- A13
    def beam_create(self, beam, vocab, n_sent, max_len, penalty=0.0):
        b = C.c_void_p()
        _chk(load().zr_beam_create(self.h, C.c_int(beam), C.c_int(vocab), C.c_int(n_sent), C.c_int(max_len),
                                   C.c_float(penalty), C.byref(b)))
        return b

    def beam_destroy(self, b):
        _chk(load().zr_beam_destroy(self.h, b))

    def beam_init(self, b):
        _chk(load().zr_beam_init(self.h, b))

    def beam_expand(self, b, d_prob, index, d_words, d_backptr):
        _chk(load().zr_beam_expand(self.h, b, _vp(d_prob), C.c_int(index), _vp(d_words), _vp(d_backptr)))

    def beam_finish(self, b, d_prob):
        _chk(load().zr_beam_finish(self.h, b, _vp(d_prob)))

    def beam_expand_logits(self, b, d_logits, d_colstats, index, d_words, d_backptr):
        _chk(load().zr_beam_expand_logits(self.h, b, _vp(d_logits), _vp(d_colstats), C.c_int(index), _vp(d_words),
                                          _vp(d_backptr)))

    def beam_finish_logits(self, b, d_logits, d_colstats):
        _chk(load().zr_beam_finish_logits(self.h, b, _vp(d_logits), _vp(d_colstats)))

    def beam_expand_blocks(self, b, d_logits, d_blocks, index, d_words, d_backptr):
        _chk(load().zr_beam_expand_blocks(self.h, b, _vp(d_logits), _vp(d_blocks), C.c_int(index), _vp(d_words),
                                          _vp(d_backptr)))

    def beam_finish_blocks(self, b, d_logits, d_blocks):
        _chk(load().zr_beam_finish_blocks(self.h, b, _vp(d_logits), _vp(d_blocks)))

    def beam_hypotheses(self, b, sentence, cap, max_len):
        words = np.full((cap, max_len), -1, dtype=np.int32)
        lens = np.zeros(cap, dtype=np.int32)
        scores = np.zeros(cap, dtype=np.float32)
        n = load().zr_beam_hypotheses(self.h, b, C.c_int(sentence), C.c_int(cap), words.ctypes.data_as(C.c_void_p),
                                      lens.ctypes.data_as(C.c_void_p), scores.ctypes.data_as(C.c_void_p))
        if n < 0:
            _chk(n)
        k = min(n, cap)
        return [(words[i, :lens[i]].copy(), float(scores[i])) for i in range(k)], n

    def ensemble_average(self, d_probs, V, cols, d_out):
        _chk(load().zr_ensemble_average(self.h, C.c_int(len(d_probs)), _ptr_array(d_probs), C.c_int(V), C.c_int(cols),
                                        _vp(d_out)))

    def attn_viterbi_ensemble(self, d_alignments, d_indices, slots, cols, longest_sent, d_viterbi):
        _chk(load().zr_attn_viterbi_ensemble(self.h, C.c_int(len(d_alignments)), _ptr_array(d_alignments),
                                             _ptr_array(d_indices), C.c_int(slots), C.c_int(cols),
                                             C.c_int(longest_sent), _vp(d_viterbi)))

    def beam_set_input_ids(self, b, d_words_nonneg):
        _chk(load().zr_beam_set_input_ids(self.h, b, _vp(d_words_nonneg)))

    def beam_set_viterbi(self, b, enable, d_viterbi=None):
        _chk(load().zr_beam_set_viterbi(self.h, b, C.c_int(1 if enable else 0), _vp(d_viterbi)))

    def beam_hypotheses_viterbi(self, b, sentence, cap, max_len):
        """Rows of max_len alignments, one row per finished hypothesis in beam_hypotheses' order; and their number."""
        vit = np.full((cap, max_len), -1, dtype=np.int32)
        n = load().zr_beam_hypotheses_viterbi(self.h, b, C.c_int(sentence), C.c_int(cap), vit.ctypes.data_as(C.c_void_p))
        if n < 0:
            _chk(n)
        return vit[:min(n, cap)], n

    def beam_state(self, b, sentence, beam):
        scores = np.zeros(beam, dtype=np.float32)
        words = np.zeros(beam, dtype=np.int32)
        _chk(load().zr_beam_state(self.h, b, C.c_int(sentence), scores.ctypes.data_as(C.c_void_p),
                                  words.ctypes.data_as(C.c_void_p)))
        return scores, words
