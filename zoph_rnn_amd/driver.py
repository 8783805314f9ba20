"""Host-side driver of a batched beam-search decode over the C-ABI.

It restates the reference's decode schedule (ensemble_factory::decode_file_batch, src/ensemble_factory.hpp:583-765;
neuralMT_model::forward_prop_source / forward_prop_target / swap_decoding_states, src/model.hpp:2367-2726) for
n_sent sentences side by side: columns [s*beam, (s+1)*beam) of every H x (n_sent*beam) activation belong to
sentence s.  Nothing V-sized leaves the device: the softmax output feeds zr_beam_expand directly and the
back-pointers it returns drive the state gathers.

As in the reference's decode path, every column runs with mask 1 (it passes d_ones, src/model.hpp:2573) and a dead
beam slot (-1) is fed as word 0.
"""
import numpy as np

from . import capi


class Seq2SeqWeights:
    """Device copies of one attention + feed-input translation model (weights given as numpy arrays)."""

    def __init__(self, ctx, src_embed, src_layers, tgt_embed, tgt_layers, attn, D_soft, b_soft):
        self.ctx = ctx
        self.H, self.Vs = src_embed.shape
        self.Vt = D_soft.shape[0]
        self.L = len(src_layers)
        self.src_embed = ctx.array(src_embed, np.float32)
        self.tgt_embed = ctx.array(tgt_embed, np.float32)
        self._keep = []
        self.src = [self._pack(ly) for ly in src_layers]
        self.tgt = [self._pack(ly) for ly in tgt_layers]
        self.attn = {k: ctx.array(v, np.float32) for k, v in attn.items()}
        self.D_soft = ctx.array(D_soft, np.float32)
        ctx.softmax_prepare(self.D_soft, self.Vt, self.H)
        self.b_soft = ctx.array(b_soft, np.float32)

    def _pack(self, ly):
        ctx = self.ctx
        M = [ctx.array(m, np.float32) for m in ly["M"]]
        Wh = [ctx.array(m, np.float32) for m in ly["Wh"]]
        b = [ctx.array(v, np.float32) for v in ly["b"]]
        Q = [ctx.array(m, np.float32) for m in ly["Q"]] if "Q" in ly else None
        self._keep.append((M, Wh, b, Q))
        return ctx.lstm_pack(M, Wh, b, self.H, Q)


class BeamDecode:
    """One batched decode: encode n_sent source sentences, then step the decoder with a device-side beam."""

    def __init__(self, ctx, w, beam, n_sent, src_len, max_steps, attention_D=10, penalty=0.0):
        self.ctx, self.w, self.beam, self.n_sent, self.S = ctx, w, beam, n_sent, src_len
        self.cols = n_sent * beam
        self.D = attention_D
        self.max_len = max_steps + 3
        H, cols, L = w.H, self.cols, w.L
        self.tables = [ctx.empty((H, cols)) for _ in range(src_len)]
        self.attn = ctx.attn_create(H, cols, attention_D, w.attn["W_a"], w.attn["W_p"], w.attn["v_p"],
                                    w.attn["out_bias"], w.attn["W_c1"], w.attn["W_c2"], self.tables)
        ctx.attn_prepare(self.attn)
        self.bm = ctx.beam_create(beam, w.Vt, n_sent, self.max_len, penalty)
        self.h = [[ctx.empty((H, cols)) for _ in range(L)] for _ in range(2)]  # ping-pong: previous / new state
        self.c = [[ctx.empty((H, cols)) for _ in range(L)] for _ in range(2)]
        self.h_tild = [ctx.empty((H, cols)) for _ in range(2)]
        self.x = ctx.empty((H, cols))
        # the logits and, behind them, the output product's (max, sum exp) pair per 32-row block and column
        # (ZR_SOFTMAX_LOGITS_BLOCKS): the beam folds the pairs itself, reads only the blocks that can hold one of a
        # column's beam + 1 largest entries and normalises only what it selects -- no probability matrix is written,
        # and the logits are not read again as a whole
        off = capi.softmax_blocks_offset(w.Vt, cols)
        self.logits = ctx.empty((off + 2 * capi.softmax_block_count(w.Vt) * cols,))
        self.blocks = self.logits.at(off)
        self.d_words = ctx.array(np.zeros(cols, np.int32))  # <START> = 0
        self.d_words_nn = ctx.array(np.zeros(cols, np.int32))
        ctx.beam_set_input_ids(self.bm, self.d_words_nn)
        self.d_back = ctx.empty(cols, np.int32)
        self.d_ones = ctx.array(np.ones(cols, np.int32))
        self.cur = 0
        self.step_index = 0
        self.history = []

    def encode(self, src_ids, src_lens):
        """src_ids: (S, n_sent) time-major, reversed and left padded with -1 as the reference lays sources out."""
        ctx, w, S, n_sent, beam = self.ctx, self.w, self.S, self.n_sent, self.beam
        H, L = w.H, w.L
        ids = np.ascontiguousarray(src_ids, np.int32)
        d_nn, d_m = ctx.empty(ids.size, np.int32), ctx.empty(ids.size, np.int32)
        ctx.vocab_prep(ctx.array(ids.reshape(-1)), ids.size, w.Vs, d_nn, d_m)
        z = ctx.zeros((H, n_sent))
        h_all = [ctx.empty((H * n_sent * S,)) for _ in range(L)]
        c_all = [ctx.empty((H * n_sent * S,)) for _ in range(L)]
        ctx.lstm_stack_forward(w.src, w.src_embed, w.Vs, d_nn, d_m, S, n_sent, [z] * L, [z] * L, h_all, c_all)
        # every sentence's states replicated over its beam columns (forward_prop_source, src/model.hpp:2394-2445,
        # and transfer_decoding_states_GPU for the final state of each layer)
        rep = ctx.array(np.repeat(np.arange(n_sent, dtype=np.int32), beam))
        n = H * n_sent
        for t in range(S):
            ctx.gather_columns(h_all[L - 1].at(t * n), H, rep, self.cols, self.tables[t])
        for l in range(L):
            ctx.gather_columns(h_all[l].at((S - 1) * n), H, rep, self.cols, self.h[0][l])
            ctx.gather_columns(c_all[l].at((S - 1) * n), H, rep, self.cols, self.c[0][l])
        lens = np.repeat(np.asarray(src_lens, np.int32), beam)
        self.d_batch_info = ctx.array(np.concatenate([lens, S - lens]).astype(np.int32))
        ctx.sync()
        self._enc_keep = (h_all, c_all, d_nn, d_m, z, rep)

    def _forward(self):
        """forward_prop_target (src/model.hpp:2573-2688): new state into the other ping-pong half, logits and their per-block pairs."""
        ctx, w, cols = self.ctx, self.w, self.cols
        H, L = w.H, w.L
        p, q = self.cur, 1 - self.cur
        # (the input ids -- the words of the last step with a dead slot's -1 turned into 0 -- come from the beam itself)
        feed = self.h_tild[p] if self.step_index > 0 else None
        ctx.decoder_step(w.tgt, w.tgt_embed, w.Vt, self.d_words_nn, self.h[p], self.c[p], self.d_ones, cols, self.h[q],
                         self.c[q], self.attn, self.d_batch_info, self.h_tild[q], w.D_soft, w.b_soft, w.Vt,
                         capi.ZR_SOFTMAX_LOGITS_BLOCKS, self.logits, d_htild_prev=feed)

    def step(self, record=False):
        """One decode step: forward, expand the beam, reorder the states by the back-pointers."""
        ctx, w, cols = self.ctx, self.w, self.cols
        H, L = w.H, w.L
        self._forward()
        ctx.beam_expand_blocks(self.bm, self.logits, self.blocks, self.step_index, self.d_words, self.d_back)
        # swap_decoding_states + target_copy_prev_states (src/model.hpp:2691-2726): the new state, permuted, becomes
        # the previous state of the next step
        p, q = self.cur, 1 - self.cur
        ctx.gather_columns_multi(self.h[q] + self.c[q] + [self.h_tild[q]], H, self.d_back, cols, cols,
                                 self.h[p] + self.c[p] + [self.h_tild[p]])
        self.step_index += 1
        if record:
            ctx.sync()
            self.history.append((self.d_words.get().copy(), self.d_back.get().copy()))

    def finish(self):
        """Last forward step and forced <EOF> on every live hypothesis (src/ensemble_factory.hpp:727-743)."""
        self._forward()
        self.ctx.beam_finish_blocks(self.bm, self.logits, self.blocks)
        self.ctx.sync()

    def hypotheses(self, sentence, cap=256):
        hyps, n = self.ctx.beam_hypotheses(self.bm, sentence, cap, self.max_len)
        return hyps

    def close(self):
        self.ctx.attn_destroy(self.attn)
        self.ctx.beam_destroy(self.bm)
