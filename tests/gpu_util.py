"""Helpers shared by the GPU parity tests: tolerance, uploads, and running the HIP path on numpy inputs."""
import numpy as np

from zoph_rnn_amd import capi

# The contract for fp32 results: within 1e-4 relative of the oracle.  Pre-activations and small activations sit
# near zero, where a pure relative bound is meaningless (an fp32 dot product of K=2000 terms of size 0.02 carries
# about 1e-6 of rounding noise whatever its sum is), so the bound is |got - want| <= REL * max(|want|, FLOOR):
# 1e-4 relative above 0.05 and 5e-6 absolute below it.  The reference author's own (now commented out) check
# of these intermediates against Eigen used 1e-4 absolute (src/LSTM.hpp:129).
REL = 1e-4
FLOOR = 5e-2


def assert_close(got, want, rel=REL, floor=FLOOR, what=""):
    got = np.asarray(got, dtype=np.float64)
    want = np.asarray(want, dtype=np.float64)
    assert got.shape == want.shape, (what, got.shape, want.shape)
    assert np.all(np.isfinite(got)), what + ": non-finite values"
    bound = rel * np.maximum(np.abs(want), floor)
    err = np.abs(got - want)
    bad = err > bound
    if np.any(bad):
        i = np.unravel_index(np.argmax(err / bound), err.shape)
        raise AssertionError("%s: %d of %d elements outside tolerance; worst at %s: got %r want %r (err %.3e, bound %.3e)"
                             % (what, int(bad.sum()), bad.size, i, got[i], want[i], err[i], bound[i]))


def magnitude_floor(want):
    """Floor for assert_close on products of operands much larger than the model's own (tests that draw U(-0.5, 0.5)
    matrices against U(-1, 1) activations reach logits of +-28 at H = 1000): fp32 accumulation noise is about
    eps * sqrt(K) times the size of the PARTIAL sums, which follow the largest entries of the result, not the entry
    being compared, so the near-zero floor scales with the largest magnitude: 0.05 * max(1, max |want|).  With
    max |want| <= 1 this is the ordinary floor."""
    return FLOOR * max(1.0, float(np.max(np.abs(want))))


def round_bf16(a):
    """fp32 array rounded to the nearest bf16-representable value (ties to even), returned as fp32, same layout."""
    a = np.asarray(a, dtype=np.float32)
    if not (a.flags.c_contiguous or a.flags.f_contiguous):
        a = np.ascontiguousarray(a)
    u = a.view(np.uint32).astype(np.uint64)
    u = (u + 0x7FFF + ((u >> 16) & 1)) & 0xFFFF0000
    return u.astype(np.uint32).view(np.float32)


class Layer:
    """One LSTM layer's parameters on the device, packed for zr_lstm_step."""

    def __init__(self, ctx, ly, bf16=False):
        self.ctx = ctx
        self.H = ly["M"][0].shape[0]
        self.M = [ctx.array(m, np.float32) for m in ly["M"]]
        self.Wh = [ctx.array(m, np.float32) for m in ly["Wh"]]
        self.b = [ctx.array(v, np.float32) for v in ly["b"]]
        self.Q = [ctx.array(m, np.float32) for m in ly["Q"]] if "Q" in ly else None
        self.w = ctx.lstm_pack(self.M, self.Wh, self.b, self.H, self.Q, bf16=bf16)

    def close(self):
        self.ctx.lstm_weights_destroy(self.w)


def run_lstm_step(ctx, layer, x, hprev, cprev, mask, htild=None, clip=0.0, want_gates=False):
    H, mb = x.shape
    dx, dh, dc = ctx.array(x, np.float32), ctx.array(hprev, np.float32), ctx.array(cprev, np.float32)
    dm = ctx.array(np.asarray(mask, np.int32))
    dt = ctx.array(htild, np.float32) if htild is not None else None
    oh, oc = ctx.empty((H, mb)), ctx.empty((H, mb))
    gates = [ctx.empty((H, mb)) for _ in range(4)] if want_gates else None
    ctx.lstm_step(layer.w, dx, dh, dc, dm, mb, oh, oc, d_htild=dt, clip=clip, gates=gates)
    ctx.sync()
    out = {"h": oh.get(), "c": oc.get()}
    if want_gates:
        for k, g in zip(("i", "f", "c_tilde", "o"), gates):
            out[k] = g.get()
    return out
