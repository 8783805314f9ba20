// The whole attention step of attention_node::forward_prop (src/attention_node.hpp:73-394) in ONE launch.
//
// As three launches the step is a chain of short kernels -- the two projections of h_t, the per-column window / score /
// soft-max / context kernel, the output product -- each of which is mostly launch, ramp-up and drain.  Here every
// workgroup is resident for the whole step and the stages hand over through device memory and arrival counters (the
// mechanism of lstm_sweep_kernel and lstm_decoder_stack_kernel in zr_lstm.hip):
//   phase P   all workgroups: the 32 x 32 tiles of  pre = W_p h_t  and  q = W_a^T h_t  (K split over the 8 waves),
//             stored into padded columns, one arrival per tile on the counter of the tile's 32-column group;
//   role M    one workgroup per batch column: waits for the 2 * ceil(H/32) tiles of its column group, then p_t, the
//             window, the scores of the valid source states (held in registers: read once), the reference's soft-max
//             whose maximum starts at 0 times the Gaussian, and the context vector, which it also leaves k-interleaved
//             for the output product; one arrival per column on the context counter of the column group;
//   role O    one workgroup per 32 x 32 tile of h~: W_c2 h_t straight away (it needs nothing of this step), the weights
//             of W_c1 requested, then the wait for the 32 contexts of its column group, W_c1 c into the same accumulators,
//             tanh, bias and mask.
// Role O's first product and role M's chain of dependent latencies overlap.  Progress: the launch must be wholly resident
// (the host checks), P never waits, M waits for P only, O for M only.  Every wait is bounded; a workgroup that runs out
// of polls marks every counter, raises the status flag and leaves NaN in the h~ tile or context column it owed.
#include <math.h>

#include "zr_internal.h"
#include "zr_mfma_core.h"

namespace {

constexpr int kGaveUp = 1 << 28;
constexpr int kCtrStride = 32;  // ints between counters: one 128-byte line each

struct AttnStep {
  const float* wpack;  // k-interleaved W_p, W_a^T, W_c1, W_c2, `per` floats apart
  long long per;
  int ldp;             // rows per k-block of those (H rounded up to 32)
  const float* hpack;  // h_t k-interleaved [H/4][mb][4]
  float* pre;          // W_p h_t before the tanh, column b at pre + b * ldp
  float* q;            // W_a^T h_t, likewise
  float* cpad;         // the context vectors for the output product: column b at cpad + b * ldp ...
  float* cpack;        // ... or, when ctx_packed, k-interleaved [H/4][mb][4] (the output product's K loop takes 2.3 us
                       // on that against 3.7 us on plain columns at 128 columns of H = 1000)
  int ctx_packed;
  int prefetch;        // role O touches the source states ahead of role M (see there)
  const float* const* table;
  const float* v_p;
  const int* batch_info;
  const int* mask01;
  const float* out_bias;
  float* p_t;
  int* indices;
  float* align;
  float* ctx_out;
  float* htild;
  float* htild_pack;   // may be null
  int* counters;       // [n_tiles] projection arrivals, then [n_tiles] context arrivals, kCtrStride apart
  int* departures;
  int* status;
  int* flags;
  int H, mb, D, longest, j_tiles, n_tiles, n_o, n_o_pad, spin_limit;
  int m_first;  // 1: the per-column workgroups have the lowest ids (see the kernel)
  int fence;  // 1: consumers invalidate their caches after a wait.  Not needed: every column of pre, q and cpad starts a
              // 128-byte line, so a line has one producer and is first read after the wait for it (and the caches are
              // clean when the launch starts).  An acquire costs 13 us of the launch's 27 at 128 columns of H = 1000:
              // it empties the die's L2 of the weights its other workgroups are streaming.
  float sigma_sq;
#ifdef ZR_ATTN_STAMPS
  unsigned long long* stamps;  // [workgroup][16]
#endif
};

#ifdef ZR_ATTN_STAMPS
#define ZR_STAMP(i)                                                                          \
  do {                                                                                       \
    if (threadIdx.x == 0) P.stamps[(size_t)blockIdx.x * 16 + (i)] = __builtin_amdgcn_s_memrealtime(); \
  } while (0)
#else
#define ZR_STAMP(i) \
  do {              \
  } while (0)
#endif

__device__ __forceinline__ float wave_sum64(float v) {
#pragma unroll
  for (int off = 32; off > 0; off >>= 1) v += __shfl_xor(v, off, 64);
  return v;
}

__device__ __forceinline__ float wave_max64(float v) {
#pragma unroll
  for (int off = 32; off > 0; off >>= 1) v = fmaxf(v, __shfl_xor(v, off, 64));
  return v;
}

// Sums over the 64 lanes of N values held one per register (N a power of two, at most 32).  Every step sends half of a
// lane's remaining values to the lane `s` away and keeps the other half, so N values cost N - 1 + log2(64 / N) cross-lane
// moves instead of 6 N.  Returns the total of value  lane >> (6 - log2 N).
template <int N, int S>
__device__ __forceinline__ float wave_sum_scatter_step(float (&v)[N > 1 ? N : 1], int lane) {
  if constexpr (N == 1) {
    float r = v[0];
#pragma unroll
    for (int s = S; s > 0; s >>= 1) r += __shfl_xor(r, s, 64);
    return r;
  } else {
    const bool up = (lane & S) != 0;
    float w[N / 2 > 1 ? N / 2 : 1];
#pragma unroll
    for (int k = 0; k < N / 2; ++k) {
      const float send = up ? v[k] : v[k + N / 2];
      const float keep = up ? v[k + N / 2] : v[k];
      w[k] = keep + __shfl_xor(send, S, 64);
    }
    return wave_sum_scatter_step<N / 2, S / 2>(w, lane);
  }
}

constexpr int ilog2(int n) { return n <= 1 ? 0 : 1 + ilog2(n / 2); }

// All threads of the workgroup call this.  False: leave (the caller poisons what it owed).
__device__ __forceinline__ bool step_wait(const AttnStep& P, int* ctr, int target, int* s_go, int nap) {
  if (threadIdx.x == 0) {
    int v = __hip_atomic_load(ctr, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    for (int spins = 0; v < target && spins < P.spin_limit; ++spins) {
      if (nap == 2)
        __builtin_amdgcn_s_sleep(2);
      else
        __builtin_amdgcn_s_sleep(6);
      v = __hip_atomic_load(ctr, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    }
    const bool ok = v >= target && !(v & kGaveUp);
    if (!ok) {
      if (!(v & kGaveUp))
        for (int i = 0; i < 2 * P.n_tiles; ++i) atomicOr(P.counters + i * kCtrStride, kGaveUp);
      __hip_atomic_store(P.status, 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    }
    *s_go = ok ? 1 : 0;
  }
  __syncthreads();
  const bool go = *s_go != 0;
  if (go && P.fence) __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "agent");
  return go;
}

// NJ: window slots per thread of role M (the 512 threads are two sets of 256: set 0 takes the even slots, set 1 the odd
// ones; a thread owns four consecutive rows of H <= 1024): up to 2 * NJ slots.
template <int NJ>
__global__ void __launch_bounds__(512) attn_step_kernel(AttnStep P) {
  constexpr int KS = 8;
  constexpr int PF = 6;
  __shared__ __align__(16) float red[KS * 16 * 64];
  __shared__ float s_red[8];
  __shared__ float s_part[8][NJ];
  __shared__ __align__(16) float s_val[2][NJ];  // alignment weights: [slot parity][slot / 2]
  __shared__ __align__(16) float s_ctx[1024];
  __shared__ int s_go[3];
  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int H = P.H, mb = P.mb;
  const int id = blockIdx.x;
  const int n_wg = gridDim.x;
  const int jl = lane & 31, half = lane >> 5;

  ZR_STAMP(0);
  auto work = [&]() {
    // ---- phase P: tiles of the two projections, dealt so that workgroup ids congruent mod 8 (one die, one L2) take
    // neighbouring tiles: the column tiles of a row tile read the same weights
    {
      const int n_p = 2 * P.n_o;
      const int n_p8 = (n_p + 7) >> 3;
      for (int slot = id; slot < 8 * n_p8; slot += n_wg) {
        const int tile = (slot & 7) * n_p8 + (slot >> 3);
        if (tile >= n_p) continue;
        const int pr = tile / P.n_o;
        const int rem = tile - pr * P.n_o;
        const int jt = rem / P.n_tiles, nt = rem - jt * P.n_tiles;
        const int j0 = jt * 32, n0 = nt * 32;
        zr_f32x16 acc[1][1];
#pragma unroll
        for (int r = 0; r < 16; ++r) acc[0][0][r] = 0.0f;
        const int col = n0 + jl < mb ? n0 + jl : mb - 1;
        const unsigned wsoff[1] = {0u};
        const unsigned xoffb[1] = {16u * (unsigned)(col + half * mb)};
        const unsigned woffb = 16u * (unsigned)(j0 + jl + half * P.ldp);
        zr_mma_segment_ring<1, 1, KS, PF>(acc, zr_make_rsrc(P.wpack + (long long)pr * P.per), wsoff, woffb,
                                       32u * (unsigned)P.ldp, zr_make_rsrc(P.hpack), xoffb, 32u * (unsigned)mb, H, wave);
        float* out = pr == 0 ? P.pre : P.q;
        zr_reduce_visit<1, 1, KS>(acc, red, wave, lane, [&](const float(&v)[1], int, int r, int) {
          const int n = n0 + 8 * (r >> 2) + 4 * half + (r & 3);
          if (n < mb)
            __hip_atomic_store(out + (long long)n * P.ldp + j0 + jl, v[0], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        });
        zr_publish_barrier();
        if (tid == 0) atomicAdd(P.counters + nt * kCtrStride, 1);
      }
    }
    ZR_STAMP(1);

    // Roles by id: the output tiles first and the columns behind them, or (m_first) the columns first -- workgroups are
    // dealt to compute units in id order, so when there are more workgroups than compute units the role that comes
    // first has a compute unit each and the other role doubles up
    const int mb8 = (mb + 7) & ~7;
    const bool is_m = P.m_first ? id < mb8 : id >= P.n_o_pad;
    const int oid = P.m_first ? id - mb8 : id;
    if (is_m) {
      // ---- role M: one batch column
      const int b = P.m_first ? id : id - P.n_o_pad;
      if (b >= mb) return;
      const int W = 2 * P.D + 1;
      const int H4 = H >> 2;
      const int k4r = tid & 255;
      const int par = wave >> 2;
      const bool mine = k4r < H4;
      const int k4 = mine ? k4r : 0;
      typedef zr_f32x4 f4;
      const f4 zero4 = {0.0f, 0.0f, 0.0f, 0.0f};
      // what does not depend on the projections goes out before the wait
      const f4 vp = (mine && par == 0) ? ((const f4*)P.v_p)[k4] : zero4;
      const int len = P.batch_info[b], off = P.batch_info[mb + b];
      const bool live = P.mask01[b] == 1;
      const bool small_table = P.longest <= 128;
      unsigned tab_lo[2] = {0u, 0u}, tab_hi[2] = {0u, 0u};
      if (small_table) {
#pragma unroll
        for (int c = 0; c < 2; ++c) {
          const int t = lane + 64 * c < P.longest ? lane + 64 * c : P.longest - 1;
          const unsigned long long pv = (unsigned long long)P.table[t];
          tab_lo[c] = (unsigned)pv, tab_hi[c] = (unsigned)(pv >> 32);
        }
      }
      auto poison = [&]() {
        const float nan = __builtin_nanf("");
        for (int k = tid; k < H; k += 512) P.ctx_out[(long long)b * H + k] = nan;
      };
      if (!step_wait(P, P.counters + (b >> 5) * kCtrStride, 2 * P.j_tiles, &s_go[0], 2)) {
        poison();
        return;
      }
      ZR_STAMP(2);
      const f4 qv = mine ? ((const f4*)(P.q + (long long)b * P.ldp))[k4] : zero4;
      float part = 0.0f;
      if (mine && par == 0) {
        const f4 t = ((const f4*)(P.pre + (long long)b * P.ldp))[k4];
        part = vp.x * tanhf(t.x) + vp.y * tanhf(t.y) + vp.z * tanhf(t.z) + vp.w * tanhf(t.w);
      }
      part = wave_sum64(part);
      if (lane == 0) s_red[wave] = part;
      __syncthreads();
      ZR_STAMP(3);
      const float sdot = ((s_red[0] + s_red[1]) + s_red[2]) + s_red[3];
      // sigmoid in double as the reference's sigmoid_kernel (src/custom_kernels.h:1583-1590): p_t feeds a truncation
      const float sig = (float)(1.0 / (1.0 + exp(-1.0 * (double)sdot)));
      const float p = (float)len * sig;
      const int ip = (int)p;
      const int lo = (0 > ip - P.D) ? 0 : (ip - P.D);
      const int hi = ((len - 1) < ip + P.D) ? (len - 1) : (ip + P.D);
      int nvalid = live ? hi - lo + 1 : 0;
      nvalid = nvalid < 0 ? 0 : (nvalid > W ? W : nvalid);
      nvalid = nvalid > 2 * NJ ? 2 * NJ : nvalid;  // the host picks NJ with 2 * NJ >= min(W, longest)
      // The table pointers of the window's slots.  Looked up slot by slot (from memory, from LDS or through the scalar
      // cache) every fetch waits for its own pointer and the 2 * NJ fetches leave one round trip after the other (3.3 us
      // of the step at 50 slots).  Instead every lane holds one table entry -- the whole table, fetched before the wait,
      // when it has at most 128 rows, else the window's rows fetched here -- and a slot's pointer is read out of its
      // lane (the row index is wave-uniform by construction).
      const int nv = __builtin_amdgcn_readfirstlane(nvalid);
      const int tb = __builtin_amdgcn_readfirstlane(len - 1 - lo + off);  // table row of slot 0; slot j sits at tb - j
      if (!small_table) {
        int t = tb - lane;
        t = t < 0 ? 0 : (t >= P.longest ? P.longest - 1 : t);
        const unsigned long long pv = (unsigned long long)P.table[t];
        tab_lo[0] = (unsigned)pv, tab_hi[0] = (unsigned)(pv >> 32);
      }
      const float* hp[NJ];
#pragma unroll
      for (int jj = 0; jj < NJ; ++jj) {
        const int j = 2 * jj + par;
        int e = j;  // entry of this slot in the lanes' copies: row tb - j of the whole table, or entry j of the window
        if (small_table) {
          e = tb - j;
          e = e < 0 ? 0 : (e >= P.longest ? P.longest - 1 : e);
        }
        const int c = e >> 6, ln = e & 63;
        const unsigned plo = __builtin_amdgcn_readlane(c ? tab_lo[1] : tab_lo[0], ln);
        const unsigned phi = __builtin_amdgcn_readlane(c ? tab_hi[1] : tab_hi[0], ln);
        hp[jj] = (const float*)(((unsigned long long)phi << 32) | plo);
      }
      f4 x[NJ];
#pragma unroll
      for (int jj = 0; jj < NJ; ++jj) {
        x[jj] = zero4;
        if (2 * jj + par < nv && mine) x[jj] = ((const f4*)(hp[jj] + (long long)b * H))[k4];
      }
      ZR_STAMP(4);
      if (tid == 0) P.p_t[b] = p;
      for (int j = tid; j < W; j += 512) P.indices[b + (long long)mb * j] = j < nvalid ? lo + j : -1;
      if (tid < nvalid) {
        const int t = len - 1 - (lo + tid) + off;
        if (t < 0 || t >= P.longest) atomicAdd(&P.flags[1], 1);
      }
      float d[NJ];
#pragma unroll
      for (int jj = 0; jj < NJ; ++jj) d[jj] = x[jj].x * qv.x + x[jj].y * qv.y + x[jj].z * qv.z + x[jj].w * qv.w;
      {
        const float tot = wave_sum_scatter_step<NJ, 32>(d, lane);
        constexpr int SH = 6 - ilog2(NJ);
        if ((lane & ((1 << SH) - 1)) == 0) s_part[wave][lane >> SH] = tot;
      }
      __syncthreads();
      ZR_STAMP(5);
      if (wave == 0) {
        // alignment_reduction_kernel (src/custom_kernels.h:1752-1794): the maximum starts at 0
        const bool v = lane < nvalid;
        float sc = 0.0f;
        if (v) {
          const int w0 = 4 * (lane & 1), jj = lane >> 1;
          sc = (s_part[w0][jj] + s_part[w0 + 1][jj]) + (s_part[w0 + 2][jj] + s_part[w0 + 3][jj]);
        }
        const float max_val = wave_max64(v ? fmaxf(sc, 0.0f) : 0.0f);
        const float e = v ? expf(sc - max_val) : 0.0f;
        const float sum = wave_sum64(e);
        float a = 0.0f;
        if (v) {
          const float dd = p - (float)(lo + lane);
          const float g = expf((-1.0f * dd * dd) / (2.0f * P.sigma_sq));
          a = sum != 0.0f ? (e / sum) * g : e;
        }
        if (lane < 2 * NJ) s_val[lane & 1][lane >> 1] = a;
        for (int j = lane; j < W; j += 64) P.align[b + (long long)mb * j] = j == lane ? a : 0.0f;
      }
      __syncthreads();
      ZR_STAMP(6);
      f4 acc = zero4;
      {
        float av[NJ];
#pragma unroll
        for (int q4 = 0; q4 < NJ / 4; ++q4) {
          const f4 a4 = ((const f4*)s_val[par])[q4];
#pragma unroll
          for (int c = 0; c < 4; ++c) av[4 * q4 + c] = a4[c];
        }
#pragma unroll
        for (int jj = 0; jj < NJ; ++jj) acc += av[jj] * x[jj];  // (slots beyond the window hold zeros on both sides)
      }
      if (par == 1 && mine) ((f4*)s_ctx)[k4] = acc;
      __syncthreads();
      if (par == 0 && mine) {
        acc += ((const f4*)s_ctx)[k4];
        if (P.ctx_packed)
          zr_store16_device(P.cpack + ((long long)k4 * mb + b) * 4, acc);
        else
          zr_store16_device(P.cpad + (long long)b * P.ldp + 4 * k4, acc);
        ((f4*)(P.ctx_out + (long long)b * H))[k4] = acc;
      }
      ZR_STAMP(7);
      zr_publish_barrier();
      if (tid == 0) atomicAdd(P.counters + (P.n_tiles + (b >> 5)) * kCtrStride, 1);
      ZR_STAMP(8);
      return;
    }

    // ---- role O: one 32 x 32 tile of h~ = tanh(W_c1 c + W_c2 h + b) * mask
    {
      const int n_o8 = P.n_o_pad >> 3;
      const int tile = (oid & 7) * n_o8 + (oid >> 3);
      if (tile >= P.n_o) return;
      const int jt = tile / P.n_tiles, nt = tile - jt * P.n_tiles;
      const int j0 = jt * 32, n0 = nt * 32;
      const int m = j0 + jl;
      const bool m_ok = m < H;
      const float bias = P.out_bias[m_ok ? m : H - 1];
      float mask_v[2];
#pragma unroll
      for (int i = 0; i < 2; ++i) {
        const int slot = wave + KS * i;
        const int n = n0 + 8 * (slot >> 2) + 4 * half + (slot & 3);
        mask_v[i] = (float)P.mask01[n < mb ? n : mb - 1];
      }
      // The source states of one batch column (the one whose role-M workgroup runs on this die) are touched here, one
      // 4-byte load per 128-byte line, so that they sit in the die's L2 when that workgroup asks for its window: all
      // columns ask at the same moment, and 128 columns of 50 states of H = 1000 are 25.6 MB from memory in one burst.
      // This workgroup has the time: its second product cannot start before the contexts are there.
      float touched[4] = {0.0f, 0.0f, 0.0f, 0.0f};
      if (P.prefetch) {
        const int lines = (H * 4 + 127) >> 7;
        for (int c = oid; c < mb; c += P.n_o_pad) {
          const int len = P.batch_info[c], off = P.batch_info[mb + c];
          const int total = len * lines;
          if (total > 4 * 512 || P.mask01[c] != 1) continue;
#pragma unroll
          for (int i = 0; i < 4; ++i) {
            const int l = tid + 512 * i;
            if (l < total) {
              const int r = l / lines, cl = l - r * lines;
              int t = off + r;
              t = t < 0 ? 0 : (t >= P.longest ? P.longest - 1 : t);
              const int k = cl * 32 < H ? cl * 32 : H - 1;
              touched[i] += P.table[t][(long long)c * H + k];
            }
          }
        }
      }
      zr_f32x16 acc[1][1];
#pragma unroll
      for (int r = 0; r < 16; ++r) acc[0][0][r] = 0.0f;
      const int col = n0 + jl < mb ? n0 + jl : mb - 1;
      const unsigned wsoff[1] = {0u};
      const unsigned xoffb[1] = {16u * (unsigned)(col + half * mb)};
      const unsigned woffb = 16u * (unsigned)(j0 + jl + half * P.ldp);
      const unsigned wstep = 32u * (unsigned)P.ldp, xstep = 32u * (unsigned)mb;
      zr_mma_segment_ring<1, 1, KS, PF>(acc, zr_make_rsrc(P.wpack + 3 * P.per), wsoff, woffb, wstep, zr_make_rsrc(P.hpack),
                                     xoffb, xstep, H, wave);
      ZR_STAMP(9);
#pragma unroll
      for (int i = 0; i < 4; ++i) asm volatile("" ::"v"(touched[i]));  // (the loads above are not dead)
      ZrFrag<1, 1> ring[PF + 1];
      const __amdgpu_buffer_rsrc_t w1 = zr_make_rsrc(P.wpack + 2 * P.per);
      zr_preload_w<1, 1, KS, PF>(ring, w1, wsoff, woffb, wstep, H, wave);
      const int want = mb - n0 < 32 ? mb - n0 : 32;
      if (!step_wait(P, P.counters + (P.n_tiles + nt) * kCtrStride, want, &s_go[1], 6)) {
        const float nan = __builtin_nanf("");
        for (int e = tid; e < 32 * 32; e += 512) {
          const int mm = j0 + (e & 31), n = n0 + (e >> 5);
          if (mm < H && n < mb) {
            P.htild[(long long)n * H + mm] = nan;
            if (P.htild_pack) P.htild_pack[((long long)(mm >> 2) * mb + n) * 4 + (mm & 3)] = nan;
          }
        }
        return;
      }
      ZR_STAMP(10);
      const unsigned coffb[1] = {P.ctx_packed ? xoffb[0] : 4u * ((unsigned)col * (unsigned)P.ldp + 4u * (unsigned)half)};
      zr_mma_segment_u<1, 1, KS, PF, true>(acc, w1, wsoff, woffb, wstep, zr_make_rsrc(P.ctx_packed ? P.cpack : P.cpad), coffb,
                                           P.ctx_packed ? xstep : 32u, H, wave, ring);
      ZR_STAMP(11);
      zr_reduce_visit<1, 1, KS>(acc, red, wave, lane, [&](const float(&v)[1], int, int r, int i) {
        const int n = n0 + 8 * (r >> 2) + 4 * half + (r & 3);
        if (m_ok && n < mb) {
          const float t = tanhf(v[0] + bias) * mask_v[i];
          P.htild[(long long)n * H + m] = t;
          if (P.htild_pack) P.htild_pack[((long long)(m >> 2) * mb + n) * 4 + (m & 3)] = t;
        }
      });
    }
  };
  work();
  ZR_STAMP(12);

  // Departure.  The last workgroup out returns the counters to zero for the next launch.
  __syncthreads();
  if (tid == 0) {
    const int before = __hip_atomic_fetch_add(P.departures, 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    s_go[2] = before == n_wg - 1 ? 1 : 0;
  }
  __syncthreads();
  if (!s_go[2]) return;
  for (int i = tid; i < 2 * P.n_tiles; i += 512)
    __hip_atomic_store(P.counters + i * kCtrStride, 0, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
  if (tid == 0) __hip_atomic_store(P.departures, 0, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}

template <int NJ>
int capacity_of(int device, int* cus_out) {
  int cus = 0, per_cu = 0;
  if (hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, device) != hipSuccess ||
      hipOccupancyMaxActiveBlocksPerMultiprocessor(&per_cu, attn_step_kernel<NJ>, 512, 0) != hipSuccess) {
    (void)hipGetLastError();
    return -1;
  }
  *cus_out = cus;
  return cus * per_cu > 0 ? cus * per_cu : -1;
}

}  // namespace

#ifdef ZR_ATTN_STAMPS
static unsigned long long* g_attn_stamps = nullptr;
extern "C" int zr_debug_attn_stamps(unsigned long long* h_out, int n_wg) {
  if (!g_attn_stamps) return 1;
  return hipMemcpy(h_out, g_attn_stamps, (size_t)n_wg * 16 * 8, hipMemcpyDeviceToHost) == hipSuccess ? 0 : 2;
}
#endif

int zr_attn_step_single_launch(zr_ctx* ctx, zr_attn* a, const int* d_batch_info, const int* d_mask01, float* d_htild,
                               float* d_htild_pack, float* align, int* idx, float* pt, float* cctx, int* took) {
  *took = 0;
  const int H = a->H, mb = a->mb, D = a->D, W = 2 * D + 1;
  const int max_slots = W < a->longest_sent ? W : a->longest_sent;
  if (!a->d_pack32 || a->d_bf16 || H % 8 != 0 || H > 1024 || H < 32 || max_slots > 64 || 
      !a->tables_aligned || ((((uintptr_t)cctx | (uintptr_t)a->v_p) & 15u) != 0) || !a->d_pq || ctx->lstm_sweep == 1)
    return ZR_OK;
  const int nj = max_slots <= 16 ? 8 : (max_slots <= 32 ? 16 : 32);
  int& cached = ctx->attn_step_capacity[nj == 8 ? 0 : (nj == 16 ? 1 : 2)];
  if (cached == 0) {
    int cus = 0;
    cached = nj == 8 ? capacity_of<8>(ctx->device, &cus) : (nj == 16 ? capacity_of<16>(ctx->device, &cus)
                                                                       : capacity_of<32>(ctx->device, &cus));
    if (cached > 0) ctx->cu_count = cus;
  }
  const int cap = cached > 0 ? cached : 0;
  const int j_tiles = (H + 31) / 32, n_tiles = (mb + 31) / 32;
  const int n_o = j_tiles * n_tiles, n_o_pad = (n_o + 7) / 8 * 8;
  // one workgroup per output tile and one per column; with few columns, further workgroups that only take projection
  // tiles, so that the 2 * n_o of those are one round (12 columns of H = 1000: 64 tiles on 44 workgroups otherwise)
  long long wgs = (long long)n_o_pad + ((mb + 7) & ~7);  // (the columns rounded up: they may come first in id order)
  {
    const long long p_tiles = (2LL * n_o + 7) / 8 * 8;
    const long long want = p_tiles < cap ? p_tiles : cap;
    if (wgs < want) wgs = want;
  }
  const bool alone = zr_live_contexts(ctx->device) == 1 && ctx->stream == ctx->own_stream;
  const long long lim = 1LL << 32;
  const bool offsets_fit = 4LL * a->kp32 * a->ldp32 * 4 < lim && (long long)a->ldp32 * mb * 4 < lim;
  if (cap <= 0 || wgs > cap || !alone || !offsets_fit || 2 * n_tiles * kCtrStride >= ZR_MAX_COUNTERS - 1) return ZR_OK;
  AttnStep P = {};
  P.wpack = a->d_pack32;
  P.per = (long long)a->kp32 * a->ldp32;
  P.ldp = a->ldp32;
  P.hpack = a->d_hpack;
  P.pre = a->d_pq;
  P.q = a->d_pq + (size_t)a->ldp32 * mb;
  P.cpad = a->d_pq + 2 * (size_t)a->ldp32 * mb;
  P.table = a->d_table;
  P.v_p = a->v_p;
  P.batch_info = d_batch_info;
  P.mask01 = d_mask01;
  P.out_bias = a->out_bias;
  P.p_t = pt;
  P.indices = idx;
  P.align = align;
  P.ctx_out = cctx;
  P.htild = d_htild;
  P.htild_pack = d_htild_pack;
  P.counters = ctx->d_counters;
  P.departures = ctx->d_counters + (ZR_MAX_COUNTERS - 1);
  P.status = ctx->d_flags + 2;
  P.flags = ctx->d_flags;
  P.H = H;
  P.mb = mb;
  P.D = D;
  P.longest = a->longest_sent;
  P.j_tiles = j_tiles;
  P.n_tiles = n_tiles;
  P.n_o = n_o;
  P.n_o_pad = n_o_pad;
  // more workgroups than compute units (192 columns of H = 1000: 384): the per-column workgroups, which stream the
  // source states through their compute unit's L1, get a compute unit each (41.4 -> 40.4 us)
  P.m_first = (long long)n_o_pad + mb > (ctx->cu_count > 0 ? ctx->cu_count : 256) ? 1 : 0;
  P.spin_limit = ctx->sweep_spin > 0 ? ctx->sweep_spin : (1 << 20);
  P.fence = 0;
  P.cpack = a->d_cpack;
  // the k-interleaved copy has one producing column group per cache line only when lines do not straddle its rows
  P.ctx_packed = mb % 8 == 0 ? 1 : 0;
  P.prefetch = 1;
  P.sigma_sq = (float)((D * D) / 4.0);  // attention_node.hpp:50
#ifdef ZR_ATTN_STAMPS
  static unsigned long long* d_stamps = nullptr;
  if (!d_stamps) (void)hipMalloc((void**)&d_stamps, 8 * 16 * 4096);
  P.stamps = d_stamps;
  g_attn_stamps = d_stamps;
#endif
  if (nj == 8)
    attn_step_kernel<8><<<(unsigned)wgs, 512, 0, ctx->stream>>>(P);
  else if (nj == 16)
    attn_step_kernel<16><<<(unsigned)wgs, 512, 0, ctx->stream>>>(P);
  else
    attn_step_kernel<32><<<(unsigned)wgs, 512, 0, ctx->stream>>>(P);
  ZR_LAUNCH_CHECK("attn_step_kernel");
  *took = 1;
  return ZR_OK;
}
