"""Deterministic synthetic inputs for the benchmark configurations.

Generator: numpy Philox with a fixed seed.  Weights and biases U(-0.08, 0.08) (the reference's default init
range, src/BZ_CUDA_UTIL.h:98-99); optionally the forget-gate bias set to 1 as the reference's layers do
(src/Input_To_Hidden_Layer.hpp:33-36).  Token ids either uniform or Zipf(s) over ranks (id = rank - 1).
Everything is float32 / int32, matrices in column-major (Fortran) order.
"""
import numpy as np

SEED = 1234
INIT_RANGE = 0.08


def rng(seed=SEED, stream=0):
    return np.random.Generator(np.random.Philox(key=seed + 7919 * stream))


def uniform(g, shape, lo=-INIT_RANGE, hi=INIT_RANGE):
    a = g.random(size=shape, dtype=np.float32) * np.float32(hi - lo) + np.float32(lo)
    return np.asfortranarray(a.astype(np.float32))


def zipf_ids(g, shape, vocab, s=1.1):
    """Zipf(s) over ranks 1..vocab by inverse-CDF sampling; id = rank - 1."""
    ranks = np.arange(1, vocab + 1, dtype=np.float64)
    cdf = np.cumsum(ranks ** (-s))
    cdf /= cdf[-1]
    u = g.random(size=shape)
    return np.minimum(np.searchsorted(cdf, u), vocab - 1).astype(np.int32)


def lstm_layer(g, H, feed_input=False, forget_bias_one=False):
    ly = {"M": [uniform(g, (H, H)) for _ in range(4)], "Wh": [uniform(g, (H, H)) for _ in range(4)],
          "b": [uniform(g, (H,)) for _ in range(4)]}
    if forget_bias_one:
        ly["b"][1] = np.ones(H, dtype=np.float32)
    if feed_input:
        ly["Q"] = [uniform(g, (H, H)) for _ in range(4)]
    return ly


def attention_weights(g, H):
    return {"W_a": uniform(g, (H, H)), "W_p": uniform(g, (H, H)), "v_p": uniform(g, (H,)),
            "out_bias": uniform(g, (H,)), "W_c1": uniform(g, (H, H)), "W_c2": uniform(g, (H, H))}


def config1(seed=SEED):
    """1-layer LM forward: H=100, mb=8, T=20, V=10000, ids uniform."""
    g = rng(seed, 1)
    H, mb, T, V = 100, 8, 20, 10000
    return {"H": H, "mb": mb, "T": T, "V": V, "embed": uniform(g, (H, V)), "layers": [lstm_layer(g, H)],
            "D": uniform(g, (V, H)), "b_d": uniform(g, (V,)),
            "ids": g.integers(0, V, size=(T, mb)).astype(np.int32),
            "targets": g.integers(0, V, size=(T, mb)).astype(np.int32)}


def encoder_config(H=1000, mb=128, T=50, V=50000, L=4, seed=SEED, forget_bias_one=False):
    """Config 2: stacked encoder forward, ids Zipf(1.1)."""
    g = rng(seed, 2)
    return {"H": H, "mb": mb, "T": T, "V": V, "L": L, "embed": uniform(g, (H, V)),
            "layers": [lstm_layer(g, H, forget_bias_one=forget_bias_one) for _ in range(L)],
            "ids": zipf_ids(g, (T, mb), V)}


def decoder_config(H=1000, mb=128, S=50, V=50000, L=4, seed=SEED):
    """Config 3: one decoder step at t >= 1 with attention + feed-input and the full softmax."""
    g = rng(seed, 3)
    cfg = {"H": H, "mb": mb, "S": S, "V": V, "L": L, "embed": uniform(g, (H, V)),
           "layers": [lstm_layer(g, H, feed_input=(l == 0)) for l in range(L)],
           "attn": attention_weights(g, H), "D": uniform(g, (V, H)), "b_d": uniform(g, (V,)),
           "ids": zipf_ids(g, (mb,), V),
           "h_prev": [np.tanh(uniform(g, (H, mb), -1.0, 1.0)) * np.float32(0.5) for _ in range(L)],
           "c_prev": [uniform(g, (H, mb), -0.5, 0.5) for _ in range(L)],
           "h_tild_prev": np.tanh(uniform(g, (H, mb), -1.0, 1.0)).astype(np.float32),
           "hs": (g.standard_normal(size=(S, H, mb), dtype=np.float32) * np.float32(0.5)),
           "batch_info": np.concatenate([np.full(mb, S, np.int32), np.zeros(mb, np.int32)])}
    return cfg
