"""The allocation-free output-layer entry point (zr_softmax_forward_static) against zr_softmax_forward, through the
C-ABI: same kernels on the library's static device scratch array instead of context scratch, so the results must be
bit-identical.  Two calls in a row, the second with a smaller input (the array keeps the first call's contents),
plus the size limit's error path."""
import numpy as np
import pytest

from zoph_rnn_amd import capi, synth

pytestmark = pytest.mark.gpu


def _run(ctx, V, H, mb, mode, prepared, seed, static):
    g = synth.rng(seed, 7)
    D, bd, h = synth.uniform(g, (V, H)), synth.uniform(g, (V,)), synth.uniform(g, (H, mb), -1, 1)
    dD, db, dh = ctx.array(D), ctx.array(bd), ctx.array(h)
    if prepared:
        ctx.softmax_prepare(dD, V, H)
    out = ctx.empty((V, mb))
    ctx.softmax_forward(dD, db, V, H, dh, mb, mode, out, static=static)
    ctx.sync()
    r = out.get()
    if prepared:
        ctx.softmax_release(dD)
    return r, (D, bd, h)


@pytest.mark.parametrize("prepared", [True, False])
def test_static_scratch_entry_point_matches_allocating_one_twice_in_a_row(prepared, oracle):
    ctx = capi.Context(0)
    try:
        # first call: a large product (the prepared path re-lays-out the activations: both scratch slots in use);
        # second call: a smaller one on the same array, whose stale contents must not leak into the result
        for (V, H, mb, mode, seed) in [(20000, 256, 96, capi.ZR_SOFTMAX_PROB, 1), (4100, 64, 24, capi.ZR_SOFTMAX_LOGPROB, 2)]:
            before = ctx.query(capi.ZR_QUERY_SCRATCH_KIB)
            got, (D, bd, h) = _run(ctx, V, H, mb, mode, prepared, seed, static=True)
            # the static call allocates nothing: the context's own scratch is what it was (nothing at all the first time)
            assert ctx.query(capi.ZR_QUERY_SCRATCH_KIB) == before
            assert before > 0 or seed != 1 or ctx.query(capi.ZR_QUERY_SCRATCH_KIB) == 0
            want, _ = _run(ctx, V, H, mb, mode, prepared, seed, static=False)
            assert ctx.query(capi.ZR_QUERY_SCRATCH_KIB) > 0  # (the allocating entry point did grow it)
            assert got.tobytes() == want.tobytes(), "static-scratch result differs from the allocating entry point"
            # and both are the oracle's soft-max
            logits = oracle.softmax_logits(D, bd, h)
            ref = oracle.softmax_dist(logits) if mode == capi.ZR_SOFTMAX_PROB else oracle.softmax_logprob_f64(logits)
            from gpu_util import assert_close
            if mode == capi.ZR_SOFTMAX_PROB:
                assert np.allclose(got.sum(axis=0, dtype=np.float64), 1.0, atol=1e-5)
                assert_close(got, ref, floor=1e-7, what="static softmax probabilities")
            else:
                assert_close(got, ref, what="static softmax log-probs")
    finally:
        ctx.close()


def test_static_scratch_entry_point_rejects_what_does_not_fit():
    ctx = capi.Context(0)
    try:
        V, H, mb = 50000, 16, 6400  # ceil(V/32) * mb * 8 bytes = 80 MB of partial statistics > 24 MiB
        g = synth.rng(3, 7)
        dD, db = ctx.array(synth.uniform(g, (V, H))), ctx.array(synth.uniform(g, (V,)))
        dh = ctx.array(synth.uniform(g, (H, mb)))
        out = ctx.empty((V, 8))  # never written: the call must fail before any launch
        with pytest.raises(capi.ZrError) as e:
            ctx.softmax_forward(dD, db, V, H, dh, mb, capi.ZR_SOFTMAX_PROB, out, static=True)
        assert e.value.code == -1 and "allocation-free" in str(e.value)
        ctx.sync()
        # the other buffer's limit: 2304 x 1000 re-laid-out activations are 9.2 MB > 8 MiB (prepared matrix)
        V, H, mb = 2048, 2304, 1000  # (the re-lay-out is taken from 2048 rows on)
        dD, db = ctx.array(synth.uniform(g, (V, H))), ctx.array(synth.uniform(g, (V,)))
        dh = ctx.array(synth.uniform(g, (H, mb)))
        ctx.softmax_prepare(dD, V, H)
        out = ctx.empty((V, mb))
        with pytest.raises(capi.ZrError) as e:
            ctx.softmax_forward(dD, db, V, H, dh, mb, capi.ZR_SOFTMAX_PROB, out, static=True)
        assert e.value.code == -1 and "allocation-free" in str(e.value) and "re-laid-out" in str(e.value)
        assert ctx.query(capi.ZR_QUERY_SCRATCH_KIB) == 0
        ctx.softmax_release(dD)
        ctx.sync()
    finally:
        ctx.close()
