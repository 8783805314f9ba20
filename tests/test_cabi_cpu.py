"""CPU-side checks of the C-ABI library: it loads without a GPU, exports every symbol include/zoph_rnn.h
declares, and host-side argument validation returns error codes instead of crashing.  No compute runs here."""
import ctypes as C
import os
import re

import pytest

from zoph_rnn_amd import capi

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
HEADER = os.path.join(ROOT, "include", "zoph_rnn.h")


def _declared_functions():
    text = open(HEADER).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(zr_[a-z0-9_]+)\s*\(", text)))


def test_header_symbols_are_exported_and_bound():
    lib = capi.load()
    declared = _declared_functions()
    assert len(declared) >= 30
    missing = [s for s in declared if not hasattr(lib, s)]
    assert not missing, "declared in zoph_rnn.h but not exported: %s" % missing
    assert sorted(capi.SYMBOLS) == declared, (set(declared) ^ set(capi.SYMBOLS))


def test_version_string_names_the_target():
    assert b"gfx950" in capi.load().zr_version()


def test_library_embeds_gfx950_code_object():
    data = open(capi.LIB_PATH, "rb").read()
    assert b"gfx950" in data and b"lstm_fused_kernel" in data


def test_null_context_and_bad_arguments_return_errors():
    lib = capi.load()
    assert lib.zr_ctx_sync(None) == -1
    assert b"null context" in lib.zr_last_error()
    assert lib.zr_ctx_create(0, None) == -1
    assert lib.zr_embed_gather(None, None, 8, 8, None, 1, None) == -1  # V checked before the context is touched
    assert lib.zr_gemm(None, 0, 4, 4, 4, None, 4, None, 4, None, 4) == -1
    # entry points added later follow the same convention: a null context is an argument error, never a crash
    assert lib.zr_softmax_prepare(None, None, 10, 8) == -1
    assert lib.zr_softmax_prepare_bf16(None, None, 10, 8) == -1
    assert lib.zr_softmax_release(None, None) == -1
    assert lib.zr_attn_use_bf16_weights(None, None) == -1
    assert lib.zr_lstm_pack_weights_bf16(None, None, None, None, None, 16, None) == -1
    assert lib.zr_lstm_train_create(None, None, None, 8, None) == -1
    assert lib.zr_unstack_gates(None, None, 8, None) == -1
    assert lib.zr_lstm_stack_backward(None, 1, None, 1, 1, None, None, None, None, None, None, None, None, None, None,
                                      None) == -1
    assert lib.zr_lstm_stack_backward_clamped(None, 1, None, 1, 1, None, None, None, None, None, None, None, None, None,
                                              None, None, C.c_float(1)) == -1
    assert lib.zr_lstm_weight_gradients(None, 8, 1, 1, None, None, None, None, None, None, None) == -1
    assert lib.zr_embed_gradient(None, 8, 8, None, None, None, 1, None) == -1
    assert lib.zr_softmax_backward(None, None, None, 8, 8, None, 1, None, None, None, None, None, None) == -1
    assert lib.zr_sgd_update(None, None, None, C.c_longlong(4), C.c_float(1), C.c_float(0), C.c_float(0.1)) == -1
    assert lib.zr_beam_set_viterbi(None, None, 1, None) == -1
    assert lib.zr_ensemble_average(None, 2, None, 8, 8, None) == -1
    assert lib.zr_attn_viterbi_ensemble(None, 2, None, None, 7, 8, 20, None) == -1
    assert lib.zr_beam_hypotheses_viterbi(None, None, 0, 0, None) == -1
    assert lib.zr_clip_inplace(None, None, C.c_longlong(4), C.c_float(1)) == -1
    assert lib.zr_grad_sumsq_accumulate(None, None, C.c_longlong(4), C.c_float(1), None, 1) == -1
    assert lib.zr_sgd_update_clipped(None, None, None, C.c_longlong(4), C.c_float(1), 2, C.c_float(5), None,
                                     C.c_float(0.1)) == -1
    assert lib.zr_lstm_node_backward(None, None, 1, None, None, None, None, None, None, None, None, None, None,
                                     None) == -1
    assert lib.zr_lstm_node_gradients(None, 8, 1, None, None, None, None, None, None) == -1
    assert lib.zr_gather_columns_multi(None, 1, None, 8, None, 4, 4, None) == -1
    assert lib.zr_softmax_backward_loss(None, None, None, 8, 8, None, 1, None, None, None, None, None, None,
                                        None) == -1
    assert lib.zr_softmax_backward_accumulate(None, None, None, 8, 8, None, 1, None, None, None, None, None,
                                              None) == -1


def test_context_creation_without_gpu_fails_cleanly():
    """On a machine without a GPU the library must report an error; with a GPU it must succeed."""
    lib = capi.load()
    h = C.c_void_p()
    rc = lib.zr_ctx_create(0, C.byref(h))
    if rc == 0:
        assert lib.zr_ctx_destroy(h) == 0
    else:
        assert rc in (-1, -2) and not h.value
        assert len(lib.zr_last_error()) > 0
        with pytest.raises(capi.ZrError):
            capi.Context(0)


def test_missing_library_is_a_hard_error(monkeypatch, tmp_path):
    monkeypatch.setattr(capi, "_lib", None)
    monkeypatch.setattr(capi, "LIB_PATH", str(tmp_path / "libzoph_rnn_hip.so"))
    with pytest.raises(RuntimeError, match="no CPU fallback"):
        capi.load()
