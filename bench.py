#!/usr/bin/env python3
"""Benchmark of the stacked-LSTM forward path on one MI355X.

A step is one pass of the hot path over one batch of synthetic input.  The headline workload (config 2 of the
baseline) is the 4-layer H=1000 encoder forward over a 128 x 50 minibatch with a 50 000-word vocabulary:
embedding gather + four-gate contraction + fused cell for 200 layer-steps = 6400 tokens per step.  Inputs
are resident in HBM before the timed region.  The config-3 decoder step (LSTM stack with feed-input,
attention, full softmax) and the stand-alone HBM-bound kernels are measured in the same run and reported
under "extra".

Prints ONE JSON line on stdout.
"""
import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
for p in (ROOT, os.path.join(ROOT, "tests")):
    if p not in sys.path:
        sys.path.insert(0, p)

import numpy as np  # noqa: E402

PEAK_FP32_MFMA_TFLOPS = 157.3  # MI355X dense fp32 matrix peak
PEAK_HBM_GBS = 8000.0          # MI355X HBM3E peak

# HBM bytes per launch of lstm_sweep_kernel on the headline workload, from two rocprofv3 --pmc runs (FETCH_SIZE, then
# WRITE_SIZE, KiB per dispatch), each scaled by what the same counter reads for a plain copy of known size
# (bench.py --calibrate-copy): FETCH_SIZE 3394177.9 KiB x 1.9854 + WRITE_SIZE 400563.6 KiB x 1.0000.
# The summary of those runs is profiles/lstm_sweep_kernel_config2_hbm_traffic.txt.
LSTM_SWEEP_TRAFFIC_BYTES = int((3393158.5 * 1.98548 + 401142.5 * 1.0) * 1024)


def log(*a):
    print(*a, file=sys.stderr, flush=True)


class Uploaded:
    """Keeps device arrays of one LSTM layer alive next to its packed weights."""

    def __init__(self, ctx, ly, bf16=False):
        self.H = ly["M"][0].shape[0]
        self.M = [ctx.array(m) for m in ly["M"]]
        self.Wh = [ctx.array(m) for m in ly["Wh"]]
        self.b = [ctx.array(v) for v in ly["b"]]
        self.Q = [ctx.array(m) for m in ly["Q"]] if "Q" in ly else None
        self.w = ctx.lstm_pack(self.M, self.Wh, self.b, self.H, self.Q, bf16=bf16)


def time_region(ctx, fn, steps, warmup):
    for _ in range(warmup):
        fn()
    ctx.sync()
    t0 = time.perf_counter()
    ctx.timer_start()
    for _ in range(steps):
        fn()
    ev_ms = ctx.timer_stop()
    ctx.sync()
    wall_ms = (time.perf_counter() - t0) * 1e3
    return wall_ms, ev_ms


def bench_encoder(ctx, steps, warmup, H=1000, mb=128, T=50, V=50000, L=4):
    from zoph_rnn_amd import synth
    cfg = synth.encoder_config(H=H, mb=mb, T=T, V=V, L=L)
    layers = [Uploaded(ctx, ly) for ly in cfg["layers"]]
    d_embed = ctx.array(cfg["embed"])
    ids = cfg["ids"]
    d_nn, d_m = ctx.empty(ids.size, np.int32), ctx.empty(ids.size, np.int32)
    ctx.vocab_prep(ctx.array(ids.reshape(-1)), ids.size, V, d_nn, d_m)
    z = ctx.zeros((H, mb))
    h_all = [ctx.empty((H * mb * T,)) for _ in range(L)]
    c_all = [ctx.empty((H * mb * T,)) for _ in range(L)]
    ws = [ly.w for ly in layers]

    def step():
        ctx.lstm_stack_forward(ws, d_embed, V, d_nn, d_m, T, mb, [z] * L, [z] * L, h_all, c_all)

    wall_ms, ev_ms = time_region(ctx, step, steps, warmup)
    # one lstm_sweep_kernel launch per step, between a counter-clearing fill in front of it and the check behind it that
    # overwrites the outputs of a sweep that gave up a wait (4-5 us each, inside the timed region)
    flops_per_step = 2.0 * 4 * H * mb * (2 * H) * L * T
    res = {"wall_ms": wall_ms, "event_ms": ev_ms, "tokens_per_step": mb * T, "launches_per_step": 3,
           "flops_per_step": flops_per_step, "avg_launch_us": ev_ms * 1e3 / steps,
           "flops_per_launch": flops_per_step}
    # keep references alive until here
    res["_keep"] = (layers, d_embed, d_nn, d_m, z, h_all, c_all)
    return res


def measure_steady_state_step(ctx, steps, warmup, H=1000, mb=128, T=50, V=50000, L=4):
    """Time one more time step adds to a sweep (L nodes, one of every layer) once the layers run as a pipeline: a sweep
    over 2T time steps has T more of them than a sweep over T and the same fill and drain, so the difference of the
    two event-timed regions / T is that time."""
    long_run = bench_encoder(ctx, steps, warmup, H=H, mb=mb, T=2 * T, V=V, L=L)
    long_run.pop("_keep")
    short_run = bench_encoder(ctx, steps, warmup, H=H, mb=mb, T=T, V=V, L=L)
    short_run.pop("_keep")
    us = (long_run["event_ms"] - short_run["event_ms"]) * 1e3 / (steps * T)
    return us, L * 2.0 * 4 * H * mb * (2 * H)


PEAK_BF16_MFMA_TFLOPS = 2500.0  # MI355X dense bf16 matrix peak


def roofline_entry(kernel, bound, us, flops=None, nbytes=None, peak_tflops=PEAK_FP32_MFMA_TFLOPS, note=None):
    """One kernel (or stage) of a step against the roofline that bounds it: algorithmic flops and / or bytes, measured
    time, achieved rate and fraction of the MI355X peak."""
    e = {"kernel": kernel, "bound": bound, "us": round(us, 2)}
    if flops is not None:
        e["gflop"] = round(flops / 1e9, 3)
        e["tflops"] = round(flops / (us * 1e-6) / 1e12, 2)
    if nbytes is not None:
        e["mbytes"] = round(nbytes / 1e6, 2)
        e["gbytes_per_s"] = round(nbytes / (us * 1e-6) / 1e9, 1)
    if bound == "mfma":
        e["peak"], e["unit"], e["frac"] = peak_tflops, "TFLOP/s", round(e["tflops"] / peak_tflops, 4)
    else:
        e["peak"], e["unit"], e["frac"] = PEAK_HBM_GBS, "GB/s", round(e["gbytes_per_s"] / PEAK_HBM_GBS, 4)
    if note:
        e["note"] = note
    return e


def bench_decoder_step(ctx, steps, warmup, H=1000, mb=128, S=50, V=50000, L=4, D=50, bf16=False):
    """Config 3: gather, 4 LSTM layers (feed-input on layer 0), attention (D >= S: every source position has a
    slot), full softmax to probabilities."""
    from zoph_rnn_amd import capi, synth
    c = synth.decoder_config(H=H, mb=mb, S=S, V=V, L=L)
    layers = [Uploaded(ctx, ly, bf16=bf16) for ly in c["layers"]]
    d_embed, d_ids = ctx.array(c["embed"]), ctx.array(c["ids"])
    d_mask = ctx.array(np.ones(mb, np.int32))
    d_hp = [ctx.array(a) for a in c["h_prev"]]
    d_cp = [ctx.array(a) for a in c["c_prev"]]
    d_htp = ctx.array(c["h_tild_prev"])
    tables = [ctx.array(np.asfortranarray(c["hs"][t])) for t in range(S)]
    aw = {k: ctx.array(v) for k, v in c["attn"].items()}
    attn = ctx.attn_create(H, mb, D, aw["W_a"], aw["W_p"], aw["v_p"], aw["out_bias"], aw["W_c1"], aw["W_c2"], tables)
    d_bi = ctx.array(c["batch_info"])
    dD, dbd = ctx.array(c["D"]), ctx.array(c["b_d"])
    ctx.softmax_prepare(dD, V, H, bf16=bf16)  # one-time snapshot of D in the matrix cores' layout, not timed
    if bf16:
        ctx.attn_use_bf16_weights(attn)
    else:
        ctx.attn_prepare(attn)  # one-time snapshot of the four attention matrices, like the output layer's: not timed
    d_x = ctx.empty((H, mb))
    d_h = [ctx.empty((H, mb)) for _ in range(L)]
    d_c = [ctx.empty((H, mb)) for _ in range(L)]
    d_ht = ctx.empty((H, mb))
    d_prob = ctx.empty((V, mb))
    d_logit = ctx.empty((V * mb + 2 * mb,))

    def logits_part():
        # the logits product and the column statistics alone (what the normalisation pass comes on top of)
        ctx.softmax_forward(dD, dbd, V, H, d_ht, mb, capi.ZR_SOFTMAX_LOGITS, d_logit)

    def lstm_part():
        # all layers of the step in one call; layer 0 looks its input columns up in the embedding itself
        ctx.lstm_decoder_step([ly.w for ly in layers], d_embed, V, d_ids, d_hp, d_cp, d_mask, mb, d_h, d_c, d_htild=d_htp)

    def attn_part():
        ctx.attn_step(attn, d_bi, d_h[L - 1], d_mask, d_ht)

    def softmax_part():
        ctx.softmax_forward(dD, dbd, V, H, d_ht, mb, capi.ZR_SOFTMAX_PROB, d_prob)

    def step():
        # forward_prop_target as one call: the three parts below with their hand-overs kept in the matrix cores' layout
        ctx.decoder_step([ly.w for ly in layers], d_embed, V, d_ids, d_hp, d_cp, d_mask, mb, d_h, d_c, attn, d_bi, d_ht, dD,
                         dbd, V, capi.ZR_SOFTMAX_PROB, d_prob, d_htild_prev=d_htp)

    wall_ms, ev_ms = time_region(ctx, step, steps, warmup)
    parts = {}
    for name, fn in (("lstm_stack", lstm_part), ("attention", attn_part), ("softmax", softmax_part),
                     ("logits_and_colstats", logits_part)):
        _, ms = time_region(ctx, fn, steps, 1)
        parts[name + "_us"] = round(ms * 1e3 / steps, 2)
    f_lstm = 2.0 * 4 * H * mb * (3 * H) + (L - 1) * 2.0 * 4 * H * mb * (2 * H)
    f_attn, f_logits = 4 * 2.0 * H * H * mb, 2.0 * V * H * mb
    flops = f_lstm + f_attn + f_logits
    res = {"ms_per_step": ev_ms / steps, "wall_ms_per_step": wall_ms / steps, "tokens_per_s": mb * steps / (ev_ms * 1e-3),
           "gflop_per_step": flops / 1e9, "tflops": flops * steps / (ev_ms * 1e-3) / 1e12, "attention_D": D}
    res.update(parts)
    if not bf16:
        res["frac_of_fp32_matrix_peak"] = round(res["tflops"] / PEAK_FP32_MFMA_TFLOPS, 4)
    res["softmax_gemm_plus_normalise_tflops"] = round(2.0 * V * H * mb / (parts["softmax_us"] * 1e-6) / 1e12, 2)
    # Every stage of the step against the roofline that bounds it.  Stages are timed on their own, back to back with
    # themselves (a stage repeated alone keeps its matrices in the memory-side cache: the step's own time is the figure
    # above); bytes and flops are algorithmic.
    wb = 2 if bf16 else 4
    peak = PEAK_BF16_MFMA_TFLOPS if bf16 else PEAK_FP32_MFMA_TFLOPS
    slots = min(2 * D + 1, S)
    norm_us = max(parts["softmax_us"] - parts["logits_and_colstats_us"], 0.01)
    res["roofline"] = [
        roofline_entry("LSTM stack, %d layers (lstm_decoder_stack_kernel or one lstm_fused_kernel per layer)" % L, "mfma",
                       parts["lstm_stack_us"], flops=f_lstm, nbytes=(12 + 8 * (L - 1)) * H * H * wb, peak_tflops=peak),
        roofline_entry("attention step (attn_step_kernel, or projections + fused middle + output product)", "mfma",
                       parts["attention_us"], flops=f_attn, nbytes=4 * H * H * wb + slots * H * mb * 4, peak_tflops=peak,
                       note="a chain of dependent stages: %.0f MB of source states and matrices, %.2f GFLOP"
                            % ((4 * H * H * wb + slots * H * mb * 4) / 1e6, f_attn / 1e9)),
        roofline_entry("output-layer logits + column statistics (gemm_tall_kernel / gemm_bf16_lds_kernel, "
                       "softmax_colstats_kernel)", "hbm" if bf16 else "mfma", parts["logits_and_colstats_us"],
                       flops=f_logits, nbytes=V * H * wb + V * mb * 4, peak_tflops=peak),
        roofline_entry("softmax_normalize_kernel", "hbm", norm_us, nbytes=2.0 * V * mb * 4),
    ]
    ctx.attn_destroy(attn)
    ctx.softmax_release(dD)
    return res


def bench_training_step(ctx, steps, H=1000, mb=128, T=50, V=50000, L=4, lr=0.5, norm_clip=5.0):
    """A language-model training step at the headline shape: forward sweep keeping the gates, output-layer backward
    over all T*mb columns, back-propagation through time, weight / bias / embedding gradients and the clipped SGD
    update of every parameter (no attention, no dropout)."""
    from zoph_rnn_amd import synth
    cfg = synth.encoder_config(H=H, mb=mb, T=T, V=V, L=L)
    g = synth.rng(synth.SEED, 7)
    layers = [Uploaded(ctx, ly) for ly in cfg["layers"]]
    trains = [ctx.lstm_train_create(ly.M, ly.Wh, H) for ly in layers]
    d_embed = ctx.array(cfg["embed"])
    ids = cfg["ids"]
    n, N = H * mb, T * mb
    d_nn, d_m = ctx.empty(ids.size, np.int32), ctx.empty(ids.size, np.int32)
    ctx.vocab_prep(ctx.array(ids.reshape(-1)), ids.size, V, d_nn, d_m)
    dD, dbd = ctx.array(synth.uniform(g, (V, H))), ctx.array(synth.uniform(g, (V,)))
    ctx.softmax_prepare(dD, V, H)
    d_tgt = ctx.array(synth.zipf_ids(g, (N,), V).astype(np.int32))
    z = ctx.zeros((H, mb))
    h_all = [ctx.empty((n * T,)) for _ in range(L)]
    c_all = [ctx.empty((n * T,)) for _ in range(L)]
    g_all = [ctx.empty((4 * n * T,)) for _ in range(L)]
    dg_all = [ctx.empty((4 * n * T,)) for _ in range(L)]
    eh0, ec0 = [ctx.empty((H, mb)) for _ in range(L)], [ctx.empty((H, mb)) for _ in range(L)]
    d_err_top, d_below0, x_all = ctx.empty((n * T,)), ctx.empty((n * T,)), ctx.empty((n * T,))
    d_scr, g_D, g_bd, g_W = ctx.empty((V, N)), ctx.empty((V, H)), ctx.empty((V,)), ctx.zeros((H, V))
    g_M = [ctx.empty((4 * H, H)) for _ in range(L)]
    g_Wh = [ctx.empty((4 * H, H)) for _ in range(L)]
    g_b = [ctx.empty((4 * H,)) for _ in range(L)]
    u_M = [[ctx.empty((H, H)) for _ in range(4)] for _ in range(L)]
    u_Wh = [[ctx.empty((H, H)) for _ in range(4)] for _ in range(L)]
    ws = [ly.w for ly in layers]
    sc = 1.0 / mb

    def step():
        ctx.lstm_stack_forward_train(ws, d_embed, V, d_nn, d_m, T, mb, [z] * L, [z] * L, h_all, c_all, g_all)
        ctx.softmax_backward(dD, dbd, V, H, h_all[L - 1], N, d_tgt, d_m, d_scr, d_err_top, g_D, g_bd)
        ctx.lstm_stack_backward(trains, T, mb, d_m, [z] * L, c_all, g_all, d_err_top, dg_all, eh0, ec0,
                                d_err_below0=d_below0)
        ctx.embed_gather(d_embed, H, V, d_nn, N, x_all)
        for l in range(L):
            ctx.lstm_weight_gradients(H, T, mb, dg_all[l], x_all if l == 0 else h_all[l - 1], z, h_all[l], g_M[l], g_Wh[l],
                                      g_b[l])
        ctx.memset_zero(g_W)
        ctx.embed_gradient(H, V, d_below0, d_nn, d_m, N, g_W)
        # update_weights: every parameter, then refresh the forward / backward copies of the matrices
        ctx.sgd_update(dD, g_D, V * H, sc, norm_clip, lr)
        ctx.sgd_update(dbd, g_bd, V, sc, norm_clip, lr)
        ctx.sgd_update(d_embed, g_W, H * V, sc, norm_clip, lr)
        for l in range(L):
            ctx.unstack_gates(g_M[l], H, u_M[l])
            ctx.unstack_gates(g_Wh[l], H, u_Wh[l])
            for q in range(4):
                ctx.sgd_update(layers[l].M[q], u_M[l][q], H * H, sc, norm_clip, lr)
                ctx.sgd_update(layers[l].Wh[q], u_Wh[l][q], H * H, sc, norm_clip, lr)
                ctx.sgd_update(layers[l].b[q], g_b[l].at(q * H), H, sc, norm_clip, lr)
            ctx.lstm_weights_destroy(layers[l].w)
            layers[l].w = ctx.lstm_pack(layers[l].M, layers[l].Wh, layers[l].b, H)
            ws[l] = layers[l].w
            ctx.lstm_train_refresh(trains[l], layers[l].M, layers[l].Wh)
        ctx.softmax_prepare(dD, V, H)

    wall_ms, ev_ms = time_region(ctx, step, steps, 1)
    flops = 3 * 2.0 * 4 * H * N * (2 * H) * L + 3 * 2.0 * V * H * N  # forward + two backward products of each size
    res = {"ms_per_step": round(ev_ms / steps, 3), "tokens_per_s": round(N * steps / (ev_ms * 1e-3), 1),
           "tflops": round(flops * steps / (ev_ms * 1e-3) / 1e12, 1), "gflop_per_step": round(flops / 1e9, 1),
           "what": "4-layer H=%d LM, minibatch %d x %d steps, vocabulary %d: forward, backward, gradients, clipped SGD"
                   % (H, mb, T, V)}
    ctx.softmax_release(dD)
    for t in trains:
        ctx.lstm_train_destroy(t)
    return res


def bench_hbm_kernels(ctx, steps, H=1000, mb=128, V=50000):
    """Stand-alone HBM-bound kernels at the benchmark shape: achieved GB/s of algorithmic bytes."""
    from zoph_rnn_amd import synth
    g = synth.rng(77, 1)
    out = {}
    # embedding gather for a whole 128 x 50 minibatch in one launch (6400 columns)
    n = mb * 50
    d_W = ctx.array(synth.uniform(g, (H, V)))
    d_ids = ctx.array(synth.zipf_ids(g, (n,), V))
    d_x = ctx.empty((H, n))
    _, ms = time_region(ctx, lambda: ctx.embed_gather(d_W, H, V, d_ids, n, d_x), steps, 2)
    bytes_ = 2.0 * n * H * 4 + n * 4
    ids_host = synth.zipf_ids(synth.rng(77, 2), (n,), V)
    unique = int(np.unique(ids_host).size)
    out["embed_gather"] = {"columns": n, "us": round(ms * 1e3 / steps, 2), "algorithmic_MB": round(bytes_ / 1e6, 3),
                           "GBps": round(bytes_ * steps / (ms * 1e-3) / 1e9, 1), "cache_assisted": True,
                           "note": "Zipf(1.1) ids repeat: repeated columns are served by the caches, so this is a rate "
                                   "of algorithmic bytes, not of HBM bytes; see embed_gather_unique_ids"}
    # the same gather with 6400 DISTINCT columns: every byte read comes from memory
    d_uid = ctx.array(synth.rng(77, 3).permutation(V)[:n].astype(np.int32))
    _, ms = time_region(ctx, lambda: ctx.embed_gather(d_W, H, V, d_uid, n, d_x), steps, 2)
    out["embed_gather_unique_ids"] = {"columns": n, "us": round(ms * 1e3 / steps, 2), "algorithmic_MB": round(bytes_ / 1e6, 3),
                                      "GBps": round(bytes_ * steps / (ms * 1e-3) / 1e9, 1), "cache_assisted": False}
    del unique
    # fused gate kernel, one layer-step (4 pre-activation planes + c_prev in, c and h out)
    d_pre = ctx.array(synth.uniform(g, (4 * H * mb,), -1, 1))
    d_b = [ctx.array(synth.uniform(g, (H,))) for _ in range(4)]
    d_cp = ctx.array(synth.uniform(g, (H, mb), -1, 1))
    d_m = ctx.array(np.ones(mb, np.int32))
    d_h, d_c = ctx.empty((H, mb)), ctx.empty((H, mb))
    _, ms = time_region(ctx, lambda: ctx.lstm_gates(d_pre, d_b, d_cp, d_m, H, mb, d_h, d_c), steps, 2)
    bytes_ = 7.0 * H * mb * 4 + 4 * H * 4 + mb * 4
    out["lstm_gates"] = {"us": round(ms * 1e3 / steps, 2), "algorithmic_MB": round(bytes_ / 1e6, 3),
                         "GBps": round(bytes_ * steps / (ms * 1e-3) / 1e9, 1),
                         "note": "one layer-step of 128 columns moves 3.6 MB: bound by launch latency, not by HBM"}
    # the same kernel over a whole minibatch of nodes (6400 columns), where the bytes dominate
    mbL = n
    d_pre = ctx.array(synth.uniform(g, (4 * H * mbL,), -1, 1))
    d_cp = ctx.array(synth.uniform(g, (H, mbL), -1, 1))
    d_m = ctx.array(np.ones(mbL, np.int32))
    d_h, d_c = ctx.empty((H, mbL)), ctx.empty((H, mbL))
    _, ms = time_region(ctx, lambda: ctx.lstm_gates(d_pre, d_b, d_cp, d_m, H, mbL, d_h, d_c), steps, 2)
    bytes_ = 7.0 * H * mbL * 4 + 4 * H * 4 + mbL * 4
    out["lstm_gates_6400_columns"] = {"us": round(ms * 1e3 / steps, 2), "algorithmic_MB": round(bytes_ / 1e6, 3),
                                      "GBps": round(bytes_ * steps / (ms * 1e-3) / 1e9, 1)}
    return out


def bench_beam_decode(ctx, steps, H=1000, L=4, beam=12, n_sent=16, S=50, V=50000, D=10):
    """Config 4: batched beam decode (16 sentences x beam 12 = 192 columns), per decode step: gather, 4 LSTM layers
    with feed-input, attention (reference default width D=10), full softmax, device-side beam, state reorder."""
    from zoph_rnn_amd import capi, driver, synth
    g = synth.rng(1234, 4)
    src_layers = [synth.lstm_layer(g, H) for _ in range(L)]
    tgt_layers = [synth.lstm_layer(g, H, feed_input=(l == 0)) for l in range(L)]
    w = driver.Seq2SeqWeights(ctx, synth.uniform(g, (H, V)), src_layers, synth.uniform(g, (H, V)), tgt_layers,
                              synth.attention_weights(g, H), synth.uniform(g, (V, H)), synth.uniform(g, (V,)))
    dec = driver.BeamDecode(ctx, w, beam, n_sent, S, steps + 8, attention_D=D)
    ctx.timer_start()
    dec.encode(synth.zipf_ids(g, (S, n_sent), V), np.full(n_sent, S, np.int32))
    enc_ms = ctx.timer_stop()
    for _ in range(3):
        dec.step()
    _, ms = time_region(ctx, dec.step, steps, 0)
    res = {"columns": beam * n_sent, "ms_per_decode_step": round(ms / steps, 4),
           "hypotheses_per_s": round(beam * n_sent * steps / (ms * 1e-3), 1), "encode_ms": round(enc_ms, 3),
           "attention_D": D}
    # the beam's two launches on their own: the per-column selection on the output product's per-block pairs (folds the
    # pairs, reads only the blocks that can hold one of a column's beam + 1 largest logits) and the per-sentence merge.
    # Algorithmic bytes: the pairs (8 bytes per 32 rows and column) -- the V x columns logits are not read again.
    bm = ctx.beam_create(beam, V, n_sent, steps + 40, 0.0)
    d_w, d_b = ctx.empty(beam * n_sent, np.int32), ctx.empty(beam * n_sent, np.int32)
    ctx.beam_expand_blocks(bm, dec.logits, dec.blocks, 0, d_w, d_b)
    _, bms = time_region(ctx, lambda: ctx.beam_expand_blocks(bm, dec.logits, dec.blocks, 1, d_w, d_b), 20, 2)
    ctx.beam_destroy(bm)
    res["beam_us"] = round(bms * 1e3 / 20, 2)
    res["beam_roofline"] = roofline_entry("beam_select_blocks_kernel + beam_merge_kernel (latency-bound: two small "
                                          "launches)", "hbm", bms * 1e3 / 20,
                                          nbytes=float(capi.softmax_block_count(V)) * 8 * beam * n_sent)
    dec.close()
    return res


def vendor_sgemm_reference(iters=50):
    """Not part of the product path: times the vendor library's fp32 GEMM (through torch.bmm) on the shapes of the two
    main products -- the four node products of a full encoder diagonal and the config-3 output-layer logits -- as a
    yardstick for the hand-written kernels, which in addition fuse the gate / cell and the soft-max partial epilogues."""
    import torch
    torch.backends.cuda.matmul.allow_tf32 = False
    out = {}
    for name, (b, m, n, k) in {"encoder_full_diagonal_4x(4000x128x2000)": (4, 4000, 128, 2000),
                               "config3_logits_50000x128x1000": (1, 50000, 128, 1000)}.items():
        a = torch.randn(b, m, k, device="cuda:0", dtype=torch.float32)
        x = torch.randn(b, k, n, device="cuda:0", dtype=torch.float32)
        for _ in range(5):
            torch.bmm(a, x)
        torch.cuda.synchronize()
        t0, t1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        t0.record()
        for _ in range(iters):
            torch.bmm(a, x)
        t1.record()
        torch.cuda.synchronize()
        us = t0.elapsed_time(t1) * 1e3 / iters
        out[name] = {"us": round(us, 2), "tflops": round(2.0 * b * m * n * k / us / 1e6, 1)}
    return out


def calibrate_copy(ctx, mbytes=64):
    """Plain copies of known size (identity column gathers: n*H*4 bytes read, n*H*4 bytes written) for scaling the
    FETCH_SIZE / WRITE_SIZE counters: one with 16-byte accesses (H = 1024, column_copy_wide_kernel) and one with
    4-byte accesses (H = 1023, column_copy_kernel<false>)."""
    out = []
    for H in (1024, 1023):
        n = mbytes * 1024 * 1024 // (H * 4)
        src, dst = ctx.zeros((H, n)), ctx.empty((H, n))
        perm = ctx.array(np.arange(n, dtype=np.int32))
        for _ in range(3):
            ctx.gather_columns(src, H, perm, n, dst)
        ctx.sync()
        out.append({"kernel": "column_copy_wide_kernel" if H % 4 == 0 else "column_copy_kernel<false>", "H": H, "columns": n,
                    "KiB_read": (n * H * 4 + n * 4) / 1024.0, "KiB_written": n * H * 4 / 1024.0})
    return out


def cpu_baseline(H=1000, mb=128, V=50000, L=4, t_sample=20):
    """The oracle (float accumulation, OpenMP) on a bounded sample of the headline workload: t_sample time steps
    of the 4-layer encoder with the same shapes; per-token cost does not depend on T."""
    import oracle_lib as o
    from zoph_rnn_amd import synth
    cfg = synth.encoder_config(H=H, mb=mb, T=t_sample, V=V, L=L)
    nn, m = o.vocab_prep(cfg["ids"])
    o.lstm_stack_forward(cfg["embed"], cfg["layers"], nn[:1], m[:1], acc64=False)  # warm-up (one time step)
    reps = []
    for _ in range(3):
        t0 = time.perf_counter()
        o.lstm_stack_forward(cfg["embed"], cfg["layers"], nn, m, acc64=False)
        reps.append(time.perf_counter() - t0)
    sec = sorted(reps)[1]
    return {"value": round(mb * t_sample / sec, 1), "unit": "tokens/s", "cores": o.num_threads(), "kind": "port",
            "sample": "%d of 50 time steps of the same 4-layer H=%d mb=%d encoder (3 repetitions, median; %.2f s each)"
                      % (t_sample, H, mb, sec)}


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=20)
    ap.add_argument("--warmup", type=int, default=30,
                    help="untimed steps before the timed ones (the first 100 ms after an idle gap run 2-9 %% slower)")
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline leg")
    ap.add_argument("--no-extra", action="store_true", help="skip the config-3 and HBM-kernel measurements")
    ap.add_argument("--lstm-tn", type=int, default=0)
    ap.add_argument("--lstm-ks", type=int, default=0)
    ap.add_argument("--sweep-only", action="store_true",
                    help="run only the headline encoder sweep (one kernel launch per step) and print its time: the "
                         "command the rocprofv3 summaries under profiles/ are made with")
    ap.add_argument("--training-only", action="store_true",
                    help="only run the language-model training step measurement (for profiling) and exit")
    ap.add_argument("--vendor-gemm", action="store_true",
                    help="only time the vendor library's fp32 GEMM on the main products' shapes (a yardstick) and exit")
    ap.add_argument("--hbm-kernels-only", action="store_true",
                    help="only run the HBM-bound kernels at the benchmark shapes (embedding gather and fused gates over "
                         "6400 columns with unique token ids, a config-3 decoder step, a config-4 decode step) a few "
                         "times and exit: the command the counter summaries of those kernels under profiles/ are made with")
    ap.add_argument("--calibrate-copy", action="store_true",
                    help="only run a plain copy kernel of known size (for scaling HBM traffic counters) and exit")
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py: this build runs on one GPU; --gpus %d is not supported (no cross-GPU path exists)" % args.gpus,
              file=sys.stderr)
        sys.exit(2)

    if args.vendor_gemm:
        print(json.dumps(vendor_sgemm_reference()))
        return

    from zoph_rnn_amd import capi
    ctx = capi.Context(0)
    if args.lstm_tn:
        ctx.set_option(capi.ZR_OPT_LSTM_TN, args.lstm_tn)
    if args.lstm_ks:
        ctx.set_option(capi.ZR_OPT_LSTM_KSPLIT, args.lstm_ks)

    if args.calibrate_copy:
        print(json.dumps(calibrate_copy(ctx)))
        ctx.close()
        return
    if args.hbm_kernels_only:
        n = max(2, min(args.steps, 5))
        out = {"hbm_kernels": bench_hbm_kernels(ctx, n),
               "config3_decoder_step": {k: v for k, v in bench_decoder_step(ctx, n, 1).items() if k.endswith("_us")},
               "config4_beam_decode": bench_beam_decode(ctx, n)}
        # the config-5 step as well (single-term mode): its attention kernel streams 102 MB of source states
        ctx.set_option(capi.ZR_OPT_BF16_ACTIVATION_TERMS, 1)
        out["config5_decoder_step_bf16_single_term"] = {
            k: v for k, v in bench_decoder_step(ctx, n, 1, H=2000, mb=256, V=80000, bf16=True).items() if k.endswith("_us")}
        ctx.set_option(capi.ZR_OPT_BF16_ACTIVATION_TERMS, 2)
        print(json.dumps(out))
        ctx.close()
        return
    if args.sweep_only:
        enc = bench_encoder(ctx, args.steps, args.warmup)
        enc.pop("_keep")
        print(json.dumps({"ms_per_step": enc["event_ms"] / args.steps, "steps": args.steps}))
        ctx.close()
        return
    if args.training_only:
        print(json.dumps(bench_training_step(ctx, max(2, args.steps // 6))))
        ctx.close()
        return

    enc = bench_encoder(ctx, args.steps, args.warmup)
    enc.pop("_keep")
    ms_per_step = enc["event_ms"] / args.steps
    tokens_per_s = enc["tokens_per_step"] / (ms_per_step * 1e-3)
    launch_us = enc["avg_launch_us"]
    achieved_tflops = enc["flops_per_launch"] / (launch_us * 1e-6) / 1e12
    step_us, step_flops = measure_steady_state_step(ctx, max(2, args.steps // 4), 1)
    log("encoder: %.3f ms/step (wall %.3f), %.0f tokens/s = %.1f TFLOP/s over the launch; one more time step costs "
        "%.2f us = %.1f TFLOP/s" % (ms_per_step, enc["wall_ms"] / args.steps, tokens_per_s, achieved_tflops, step_us,
                                    step_flops / (step_us * 1e-6) / 1e12))
    # the same sweep as one launch per diagonal of the (layer, time) grid, for comparison
    ctx.set_option(capi.ZR_OPT_LSTM_SWEEP, 1)
    diag = bench_encoder(ctx, args.steps, args.warmup)
    diag.pop("_keep")
    ctx.set_option(capi.ZR_OPT_LSTM_SWEEP, 0)
    log("encoder with one launch per diagonal: %.3f ms/step" % (diag["event_ms"] / args.steps))

    extra = {}
    if not args.no_extra:
        # Sub-millisecond steps are timed over at least 0.1 s: after the host-side set-up gap in front of each of these
        # measurements the first 50-100 ms run slower (0.299 ms per config-3 step over 20 steps, 0.282 over 200, 0.274
        # over 1000 on one box), and what is wanted is the sustained rate.
        short_steps, short_warm = max(args.steps * 25, 200), max(args.warmup, 30)
        extra["config3_decoder_step"] = {k: (round(v, 4) if isinstance(v, float) else v)
                                         for k, v in bench_decoder_step(ctx, short_steps, short_warm).items()}
        extra["config3_decoder_step"]["timed_steps"] = short_steps
        log("config3:", extra["config3_decoder_step"])
        c5 = bench_decoder_step(ctx, short_steps // 2, short_warm, H=2000, mb=256, V=80000, bf16=True)
        c5["weights"] = "bf16 storage (LSTM, attention projections, output layer), fp32 activations split in two bf16 terms, fp32 accumulation"
        extra["config5_decoder_step_bf16_weights"] = {k: (round(v, 4) if isinstance(v, float) else v) for k, v in c5.items()}
        log("config5:", extra["config5_decoder_step_bf16_weights"])
        from zoph_rnn_amd import capi as _capi
        ctx.set_option(_capi.ZR_OPT_BF16_ACTIVATION_TERMS, 1)
        try:
            c5s = bench_decoder_step(ctx, short_steps // 2, short_warm, H=2000, mb=256, V=80000, bf16=True)
        finally:
            ctx.set_option(_capi.ZR_OPT_BF16_ACTIVATION_TERMS, 2)
        c5s["weights"] = "bf16 storage, activations rounded to bf16 once (single-term mode), fp32 accumulation"
        extra["config5_decoder_step_bf16_single_term"] = {k: (round(v, 4) if isinstance(v, float) else v) for k, v in c5s.items()}
        log("config5 single-term:", extra["config5_decoder_step_bf16_single_term"])
        extra["lm_training_step"] = bench_training_step(ctx, max(2, args.steps // 6))
        log("training step:", extra["lm_training_step"])
        extra["hbm_kernels"] = bench_hbm_kernels(ctx, args.steps)
        extra["config4_beam_decode"] = bench_beam_decode(ctx, max(args.steps * 5, 100))
        # its forward stages at 192 columns and the reference's window (D = 10), each against its roofline
        c4 = bench_decoder_step(ctx, short_steps // 2, short_warm, mb=192, D=10)
        extra["config4_beam_decode"]["roofline"] = c4["roofline"] + [extra["config4_beam_decode"].pop("beam_roofline")]
        extra["config4_beam_decode"]["forward_stages_ms_per_step"] = round(c4["ms_per_step"], 4)
        log("config4:", extra["config4_beam_decode"])
        # the reference decodes one sentence per pass: the same step with 12 columns
        extra["config4_single_sentence_beam12"] = bench_beam_decode(ctx, max(args.steps * 5, 100), n_sent=1)
        extra["config4_single_sentence_beam12"].pop("beam_roofline", None)
        log("config4, one sentence:", extra["config4_single_sentence_beam12"])
        log("hbm kernels:", extra["hbm_kernels"])
    cpu = None
    if not args.no_cpu:
        cpu = cpu_baseline()
        log("cpu baseline:", cpu)
    ctx.close()

    line = {
        "metric": "LSTM step tokens/sec on 1 GPU (4L H=1000 mb=128 V=50k) + % HBM/MFMA roofline",
        "value": round(tokens_per_s, 1),
        "unit": "tokens/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": round(ms_per_step, 4),
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "f32",
        "data": "synthetic",
        "config": {"workload": "config 2: 4-layer LSTM encoder forward, H=1000, minibatch 128, source length 50, "
                               "vocab 50000 (Zipf ids), fp32; one step = 200 layer-steps = 6400 tokens",
                   "tokens_per_step": enc["tokens_per_step"], "launches_per_step": enc["launches_per_step"]},
        "roofline": {"bound": "mfma", "kernel": "lstm_sweep_kernel", "achieved": round(achieved_tflops, 2),
                     "peak": PEAK_FP32_MFMA_TFLOPS, "unit": "TFLOP/s", "frac": round(achieved_tflops / PEAK_FP32_MFMA_TFLOPS, 4),
                     "traffic": LSTM_SWEEP_TRAFFIC_BYTES, "traffic_unit": "bytes per launch",
                     "launch": "whole sweep: 4 layers x 50 time steps = 200 nodes, 256 workgroups resident throughout "
                               "(the pipeline of layers fills and drains inside the launch)",
                     "avg_launch_us": round(launch_us, 2), "flops_per_launch": enc["flops_per_launch"],
                     "algorithmic_bytes_per_launch": 200 * (2 * 4 * 1000 * 1000 + 3 * 1000 * 128 + 2 * 1000 * 128) * 4,
                     "steady_state_step_us": round(step_us, 2),
                     "steady_state_tflops": round(step_flops / (step_us * 1e-6) / 1e12, 2),
                     "one_launch_per_diagonal_ms_per_step": round(diag["event_ms"] / args.steps, 4)},
        "cpu_baseline": cpu,
        "extra": extra,
    }
    print(json.dumps(line))


if __name__ == "__main__":
    main()
