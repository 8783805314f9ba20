// Generic multi-segment fp32 GEMM on MFMA:  C = sum_s op(A_s) * B_s  followed by a fused epilogue.
// Serves the softmax logits (with per-block max / sum-exp partials), the attention projections (tanh, bias,
// mask fused) and the plain cublasSgemm replacement.  See zr_mfma_core.h for the operand mapping.
#include <math.h>

#include "zr_internal.h"
#include "zr_mfma_core.h"

namespace {

struct GemmArgs {
  int M, N, nseg;
  int K[3];
  const float* A[3];
  long long lda[3];
  const float* B[3];
  int ldb[3];
  float* C;
  int ldc;
  long long strideA, strideC, strideBias;
  const float* bias;
  const int* mask;
  float* partials;
  float* Cpack;          // ZR_EPI_TANH_BIAS_MASK: second, k-interleaved copy of the result (null: none)
  unsigned short* Chi;   // ZR_EPI_TANH_BIAS_MASK: the result as bf16 terms, [M/8][N][8] (null: none); Clo may be null
  unsigned short* Clo;
  int m_tiles, n_tiles;  // wave tiles along M and N
  int b_pack4;           // B segments are k-interleaved copies: element (k, n) at ((k/4)*N + n)*4 + k%4
  // bf16 weights: B[s] is the bf16 "hi" array and Blo[s] the "lo" array of the split activations, both
  // k-interleaved by 8 ([K/8][N][8]); see zr_split_pack_multi_kernel
  const unsigned short* Blo[3];
  int accum;  // ZR_EPI_STORE only: C += result instead of C = result
  int stream_a;  // the weights are fetched with the streaming hint (ZrGemmDesc::stream_a)
  // groups > 0: blockIdx.z = group * batch + batch index; the group picks A, B and C from these tables
  int groups, batch;
  const float* gA[8];
  const float* gB[8];
  float* gC[8];
};

template <int... I>
struct zr_int_seq {};
template <int N, int... I>
struct zr_make_int_seq_t : zr_make_int_seq_t<N - 1, N - 1, I...> {};
template <int... I>
struct zr_make_int_seq_t<0, I...> {
  typedef zr_int_seq<I...> type;
};
template <int N>
using zr_make_int_seq = typename zr_make_int_seq_t<N>::type;

// largest divisor c of nv with c * tm <= 32
constexpr int stats_chunk(int nv, int tm) {
  int best = 1;
  for (int c = 1; c <= nv; ++c)
    if (nv % c == 0 && c * tm <= 32) best = c;
  return best;
}

// Soft-max-partial epilogue of a wave that holds a whole 32*TM x 32*TN tile (no K split): logits = acc + bias stored to
// C, and (max, sum exp) of every 32-row block and column to a.partials.  Four columns (accumulator registers) of every
// row sub-tile at a time, so that their cross-lane reductions run interleaved.  One instantiation per 32-column block
// (a loop over them is not unrolled at eight blocks, and an accumulator array indexed by a variable lives in memory).
template <int TM, int TN, int TNI, bool FULL>
__device__ __forceinline__ void softmax_partial_epilogue_block(const GemmArgs& a, float* C,
                                                               const zr_f32x16 (&acc)[TM][TN], const float (&bias_v)[TM],
                                                               int m0, int n0, bool active, int lane) {
  const int jl = lane & 31;
  const int half = lane >> 5;
  auto store = [&](int n, int tm, bool okv, float val, float mxv, float sev) {
    const int m = m0 + tm * 32 + jl;
    if (FULL || okv) C[(long long)n * a.ldc + m] = val;
    const int prow = (m0 >> 5) + tm;  // 32-row block index
    if (jl == 0 && (FULL || (active && n < a.N && prow * 32 < a.M))) {
      typedef float zr_f32x2 __attribute__((ext_vector_type(2)));
      *(zr_f32x2*)(a.partials + ((long long)n * ((a.M + 31) >> 5) + prow) * 2) = zr_f32x2{mxv, sev};
    }
  };
#pragma unroll
  for (int rg = 0; rg < 4; ++rg) {
    float v[4 * TM], mx[4 * TM], se[4 * TM];
    bool ok[4 * TM];
#pragma unroll
    for (int i = 0; i < 4; ++i)
#pragma unroll
      for (int tm = 0; tm < TM; ++tm) {
        const int n = n0 + TNI * 32 + 8 * rg + 4 * half + i;
        v[i * TM + tm] = acc[tm][TNI][4 * rg + i] + bias_v[tm];
        ok[i * TM + tm] = FULL || (active && n < a.N && (m0 + tm * 32 + jl) < a.M);
      }
    zr_half_wave_softmax_stats<4 * TM>(v, ok, mx, se);
#pragma unroll
    for (int i = 0; i < 4; ++i)
#pragma unroll
      for (int tm = 0; tm < TM; ++tm)
        store(n0 + TNI * 32 + 8 * rg + 4 * half + i, tm, ok[i * TM + tm], v[i * TM + tm], mx[i * TM + tm],
              se[i * TM + tm]);
  }
}

template <int TM, int TN, bool FULL, int... TNI>
__device__ __forceinline__ void softmax_partial_epilogue_blocks(const GemmArgs& a, float* C,
                                                                const zr_f32x16 (&acc)[TM][TN], const float (&bias_v)[TM],
                                                                int m0, int n0, bool active, int lane,
                                                                zr_int_seq<TNI...>) {
  (softmax_partial_epilogue_block<TM, TN, TNI, FULL>(a, C, acc, bias_v, m0, n0, active, lane), ...);
}

template <int TM, int TN>
__device__ __forceinline__ void softmax_partial_epilogue(const GemmArgs& a, float* C, const zr_f32x16 (&acc)[TM][TN],
                                                         const float (&bias_v)[TM], int m0, int n0, bool active,
                                                         int lane) {
  // FULL: the whole tile lies inside the matrix (uniform over the wave): no masks, no branches around the stores
  if (active && m0 + 32 * TM <= a.M && n0 + 32 * TN <= a.N)
    softmax_partial_epilogue_blocks<TM, TN, true>(a, C, acc, bias_v, m0, n0, active, lane, zr_make_int_seq<TN>{});
  else
    softmax_partial_epilogue_blocks<TM, TN, false>(a, C, acc, bias_v, m0, n0, active, lane, zr_make_int_seq<TN>{});
}

// One output tile of 32*TM rows x 32*TN columns at (m0, n0), computed by the KS waves that call this together
// (kslice = this wave's K slice, redp = their KS*TN*16*64 floats of LDS): all segments, the split-K sum and the
// epilogue.  `active` false: same control flow (barriers), nothing stored.  PF = prefetch distance in k-groups.
// BUF (k-interleaved fp32 operands on both sides, K % 8 == 0, every row and column of the tile in range, operands below
// 4 GiB): the K loop fetches through buffer descriptors with the pinned schedule of zr_mma_segment_u.
template <int TM, int TN, int KS, int AMODE, bool VEC, int EPI, int PF, bool BUF = false, int WAUX = 0>
__device__ __forceinline__ void gemm_tile(const GemmArgs& a, int m0, int n0, bool active, int z, float* redp,
                                          int kslice, int lane) {
  const int jl = lane & 31;
  const int half = lane >> 5;
  int rows[TM];
#pragma unroll
  for (int tm = 0; tm < TM; ++tm) {
    const int r = m0 + tm * 32 + jl;
    rows[tm] = r < a.M ? r : a.M - 1;
  }
  int cols[TN];
#pragma unroll
  for (int tn = 0; tn < TN; ++tn) {
    const int c = n0 + tn * 32 + jl;
    cols[tn] = c < a.N ? c : a.N - 1;
  }

  zr_f32x16 acc[TM][TN];
#pragma unroll
  for (int tm = 0; tm < TM; ++tm)
#pragma unroll
    for (int tn = 0; tn < TN; ++tn)
#pragma unroll
      for (int r = 0; r < 16; ++r) acc[tm][tn][r] = 0.0f;

  // several problems in one launch: the group picks the operands, z becomes the batch index inside the group
  const float* grpA = nullptr;
  const float* grpB = nullptr;
  float* grpC = nullptr;
  if (a.groups) {
    const int grp = z / a.batch;
    z -= grp * a.batch;
    grpA = a.gA[grp];
    grpB = a.gB[grp];
    grpC = a.gC[grp];
  }

  // epilogue operands go out ahead of the K loop
  const float* bias = a.bias ? a.bias + (long long)z * a.strideBias : nullptr;
  float bias_v[TM];
  if (EPI == ZR_EPI_SOFTMAX_PARTIAL) {
#pragma unroll
    for (int tm = 0; tm < TM; ++tm) bias_v[tm] = bias[rows[tm]];
  }

  for (int s = 0; s < a.nseg; ++s) {
    if constexpr (BUF) {
      unsigned wsoff[TM], xoffb[TN];
#pragma unroll
      for (int tm = 0; tm < TM; ++tm) wsoff[tm] = 512u * (unsigned)tm;  // 32 rows of 16 bytes
#pragma unroll
      for (int tn = 0; tn < TN; ++tn) xoffb[tn] = 16u * (unsigned)(cols[tn] + half * a.N);
      const unsigned woffb = 16u * (unsigned)(m0 + jl + half * (int)a.lda[s]);
      zr_mma_segment_ring<TM, TN, KS, PF, WAUX>(acc, zr_make_rsrc(a.A[s]), wsoff, woffb, 32u * (unsigned)a.lda[s],
                                       zr_make_rsrc(a.B[s]), xoffb, 32u * (unsigned)a.N, a.K[s], kslice);
    } else if constexpr (zr_is_bf16_mode(AMODE)) {
      const unsigned short* wbase[TM];
      unsigned woff[TM];
      const float* xcol[TN];
#pragma unroll
      for (int tm = 0; tm < TM; ++tm) {
        wbase[tm] = (const unsigned short*)a.A[s] + (long long)z * a.strideA;  // (strideA counts bf16 elements here)
        woff[tm] = (unsigned)(8LL * rows[tm] + 8LL * half * a.lda[s]);
      }
      const unsigned short* xlo[TN];
#pragma unroll
      for (int tn = 0; tn < TN; ++tn) {
        const long long off = 8LL * (cols[tn] + (long long)half * a.N);
        xcol[tn] = (const float*)((const unsigned short*)a.B[s] + off);
        xlo[tn] = a.Blo[s] + off;
      }
      zr_mma_segment_bf16<TM, TN, KS, PF, true, AMODE == ZR_A_PACK8_BF16>(acc, wbase, woff, a.lda[s], xcol, a.K[s], kslice,
                                                                          xlo, a.N);
    } else {
      const float* A = (grpA ? grpA : a.A[s]) + (long long)z * a.strideA;
      const float* Bs = grpB ? grpB : a.B[s];
      const float* wbase[TM];
      unsigned woff[TM];
      const float* xcol[TN];
#pragma unroll
      for (int tm = 0; tm < TM; ++tm) {
        wbase[tm] = A;
        woff[tm] = AMODE == ZR_A_PACK4   ? (unsigned)(4LL * rows[tm] + 4LL * half * a.lda[s])
                   : AMODE == ZR_A_TRANS ? (unsigned)((long long)rows[tm] * a.lda[s] + 4 * half)
                                         : (unsigned)(rows[tm] + 4LL * half * a.lda[s]);
      }
#pragma unroll
      for (int tn = 0; tn < TN; ++tn)
        xcol[tn] = (AMODE == ZR_A_PACK4 && a.b_pack4) ? Bs + 4LL * cols[tn] + 4LL * half * a.N
                                                     : Bs + (long long)cols[tn] * a.ldb[s] + 4 * half;
      zr_mma_segment<TM, TN, KS, PF, AMODE, VEC>(acc, wbase, woff, a.lda[s], xcol, a.K[s], kslice, half,
                                                 (AMODE == ZR_A_PACK4 && a.b_pack4) ? a.N : 1);
    }
  }

  float* C = (grpC ? grpC : a.C) + (long long)z * a.strideC;

  if (EPI == ZR_EPI_SOFTMAX_PARTIAL) {
    // logits = acc + bias, plus (max, sum exp) of every 32-row block and column.  The values of all visits are
    // collected first so that their cross-lane reductions run interleaved, then everything is stored.
    auto store = [&](int n, int tm, bool okv, float val, float mxv, float sev) {
      const int m = m0 + tm * 32 + jl;
      if (okv) C[(long long)n * a.ldc + m] = val;
      const int prow = (m0 >> 5) + tm;  // 32-row block index
      if (jl == 0 && active && n < a.N && prow * 32 < a.M) {
        typedef float zr_f32x2 __attribute__((ext_vector_type(2)));
        *(zr_f32x2*)(a.partials + ((long long)n * ((a.M + 31) >> 5) + prow) * 2) = zr_f32x2{mxv, sev};
      }
    };
    if (KS == 1) {
      softmax_partial_epilogue<TM, TN>(a, C, acc, bias_v, m0, n0, active, lane);
    } else {
      constexpr int NV = zr_visit_count<TN, KS>();
      float v[NV * TM];
      bool ok[NV * TM];
      int nn[NV];
      zr_reduce_visit<TM, TN, KS>(acc, redp, kslice, lane, [&](const float(&vals)[TM], int tn, int r, int i) {
        const int n = n0 + tn * 32 + 8 * (r >> 2) + 4 * half + (r & 3);
        nn[i] = n;
#pragma unroll
        for (int tm = 0; tm < TM; ++tm) {
          v[i * TM + tm] = vals[tm] + bias_v[tm];
          ok[i * TM + tm] = active && n < a.N && (m0 + tm * 32 + jl) < a.M;
        }
      });
      // at most 32 butterflies at a time (register budget)
      constexpr int CH = stats_chunk(NV, TM);
#pragma unroll
      for (int c0 = 0; c0 < NV; c0 += CH) {
        float cv[CH * TM], cmx[CH * TM], cse[CH * TM];
        bool cok[CH * TM];
#pragma unroll
        for (int j = 0; j < CH * TM; ++j) {
          cv[j] = v[c0 * TM + j];
          cok[j] = ok[c0 * TM + j];
        }
        zr_half_wave_softmax_stats<CH * TM>(cv, cok, cmx, cse);
#pragma unroll
        for (int i = 0; i < CH; ++i)
#pragma unroll
          for (int tm = 0; tm < TM; ++tm)
            store(nn[c0 + i], tm, cok[i * TM + tm], cv[i * TM + tm], cmx[i * TM + tm], cse[i * TM + tm]);
      }
    }
    return;
  }

  zr_reduce_visit<TM, TN, KS>(acc, redp, kslice, lane, [&](const float(&vals)[TM], int tn, int r, int) {
    const int n = n0 + tn * 32 + 8 * (r >> 2) + 4 * half + (r & 3);
    const bool n_ok = active && n < a.N;
#pragma unroll
    for (int tm = 0; tm < TM; ++tm) {
      const int m = m0 + tm * 32 + jl;
      const bool ok = n_ok && m < a.M;
      float v = vals[tm];
      if (EPI == ZR_EPI_STORE) {
        if (ok) {
          if (bias) v += bias[m];
          float* cp = C + (long long)n * a.ldc + m;
          *cp = a.accum ? *cp + v : v;
        }
      } else if (EPI == ZR_EPI_TANH) {
        if (ok) C[(long long)n * a.ldc + m] = tanhf(v);
      } else {  // ZR_EPI_TANH_BIAS_MASK
        if (ok) {
          const float t = tanhf(v + bias[m]) * (float)a.mask[n];
          C[(long long)n * a.ldc + m] = t;
          if (a.Cpack) a.Cpack[((long long)(m >> 2) * a.N + n) * 4 + (m & 3)] = t;
          if (a.Chi) {  // the split of zr_split_bf16_pair, element by element
            const __bf16 hb = (__bf16)t;
            const long long o = ((long long)(m >> 3) * a.N + n) * 8 + (m & 7);
            a.Chi[o] = __builtin_bit_cast(unsigned short, hb);
            if (a.Clo) a.Clo[o] = __builtin_bit_cast(unsigned short, (__bf16)(t - (float)hb));
          }
        }
      }
    }
  });
}

// Workgroup = 64*KS*WPB threads: WPB independent wave tiles, each shared by KS waves that split K.
// AMODE is the weight layout (ZR_A_NN / ZR_A_TRANS / ZR_A_PACK4).  The packed variant is built for two workgroups
// per CU (at most 256 registers per wave): with several workgroups per CU in sequence, the prologue and epilogue
// of one overlap the K loop of the other.
template <int TM, int TN, int KS, int WPB, int AMODE, bool VEC, int EPI, int OCC = 1>
__global__ void __launch_bounds__(64 * KS * WPB, OCC) gemm_kernel(GemmArgs a) {
  __shared__ float red[KS > 1 ? WPB * KS * TN * 16 * 64 : 1];
  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);  // wave-uniform by construction
  const int kslice = wave % KS;
  const int sub = wave / KS;  // which wave tile of the workgroup
  const int z = blockIdx.z;

  long long tile = (long long)blockIdx.x * WPB + sub;
  const long long ntiles = (long long)a.m_tiles * a.n_tiles;
  bool active = tile < ntiles;
  int mt, nt;
  if (AMODE == ZR_A_PACK4 || zr_is_bf16_mode(AMODE)) {
    // Workgroup ids congruent modulo 8 run on the same XCD.  Each XCD gets a contiguous range of row tiles and
    // runs the column tiles of one row tile back to back (in neighbouring waves of a workgroup when WPB > 1), so a
    // weight tile leaves memory once.
    const int r8 = (int)(blockIdx.x & 7);
    const int q = (int)(blockIdx.x >> 3) * WPB + sub;   // wave-tile slot within the XCD's range
    const int mpx = (a.m_tiles + 7) >> 3;
    nt = q % a.n_tiles;
    mt = r8 * mpx + q / a.n_tiles;
    active = (q / a.n_tiles < mpx) && (mt < a.m_tiles);
    if (!active) mt = a.m_tiles - 1;
  } else {
    // wave tile id -> (mt, nt), m fastest so that neighbouring waves stream neighbouring weight rows
    if (!active) tile = ntiles - 1;  // keep the wave in step with the workgroup barriers; results discarded
    mt = (int)(tile % a.m_tiles);
    nt = (int)(tile / a.m_tiles);
  }
  constexpr int PF = zr_is_bf16_mode(AMODE) ? 4
                     : AMODE == ZR_A_PACK4    ? (OCC == 1 ? (TM + TN <= 4 ? 8 : 6) : (TM + TN == 4 ? 6 : 4))
                                              : zr_prefetch_depth(TM, TN);
  float* redp = KS > 1 ? red + (size_t)sub * KS * TN * 16 * 64 : red;
  gemm_tile<TM, TN, KS, AMODE, VEC, EPI, PF>(a, mt * 32 * TM, nt * 32 * TN, active, z, redp, kslice, lane);
}

// Row-range variant for a tall weight matrix in the k-interleaved layout (the softmax logits: tens of thousands
// of rows, a minibatch of columns).  With one tile per workgroup the number of workgroups is rarely a multiple of
// the number of CUs and the last, partly filled round costs as much as a full one.  Here the grid is one
// workgroup per CU (or fewer): each takes an equal share of the 32-row blocks for one column tile and walks it in
// passes of up to four blocks; the few blocks that do not divide evenly are split into 32-column pieces over the
// workgroups.  Every CU finishes at about the same time and each weight element is read by exactly one workgroup
// per column tile (by up to TN for the left-over blocks).
template <int TN, int EPI, int AMODE = ZR_A_PACK4>
__global__ void __launch_bounds__(256) gemm_rows_kernel(GemmArgs a, int row_chunks) {
  __shared__ float red[4 * TN * 16 * 64];
  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int kslice = __builtin_amdgcn_readfirstlane(tid >> 6);
  // ids congruent modulo 8 share an XCD: give each XCD a contiguous range of row chunks, column tiles adjacent
  const int r8 = blockIdx.x & 7;
  const int q = blockIdx.x >> 3;
  const int cpx = (row_chunks + 7) >> 3;
  const int nt = q % a.n_tiles;
  const int chunk = r8 * cpx + q / a.n_tiles;
  if (q / a.n_tiles >= cpx || chunk >= row_chunks) return;
  // Every chunk takes the same number of 32-row blocks; the blocks left over (fewer than row_chunks) are dealt out
  // afterwards in 32-column pieces, one piece per workgroup, so that no workgroup carries a whole extra block.
  // (Only when that is at most one piece per workgroup; with more left over, shares of +-1 block cost less.)
  const int blocks = (a.M + 31) >> 5;
  const int per_chunk = blocks / row_chunks;
  const int left = blocks - per_chunk * row_chunks;
  const bool pieces = left * TN <= row_chunks;
  int b = pieces ? chunk * per_chunk : (int)((long long)blocks * chunk / row_chunks);
  const int b_end = pieces ? b + per_chunk : (int)((long long)blocks * (chunk + 1) / row_chunks);
  const int n0 = nt * 32 * TN;
  // at most 192 accumulator registers per wave: four blocks per pass up to 96 columns, three at 128
  constexpr int TMAX = TN <= 3 ? 4 : 3;
  constexpr int PF4 = zr_is_bf16_mode(AMODE) ? 2 : (TN <= 2 ? 6 : (TN == 3 ? 4 : 3));
  while (b < b_end) {
    const int nb = b_end - b < TMAX ? b_end - b : TMAX;  // uniform over the workgroup
    if (TMAX == 4 && nb == 4)
      gemm_tile<TMAX, TN, 4, AMODE, true, EPI, PF4>(a, b * 32, n0, true, 0, red, kslice, lane);
    else if (nb == 3)
      gemm_tile<3, TN, 4, AMODE, true, EPI, PF4 + 1>(a, b * 32, n0, true, 0, red, kslice, lane);
    else if (nb == 2)
      gemm_tile<2, TN, 4, AMODE, true, EPI, PF4 + 2>(a, b * 32, n0, true, 0, red, kslice, lane);
    else
      gemm_tile<1, TN, 4, AMODE, true, EPI, PF4 + 2>(a, b * 32, n0, true, 0, red, kslice, lane);
    b += nb;
    __syncthreads();  // the next pass reuses the reduction buffer
  }
  for (int u = chunk; pieces && u < left * TN; u += row_chunks) {
    const int blk = per_chunk * row_chunks + u / TN, sub = u % TN;
    if (n0 + sub * 32 < a.N)
      gemm_tile<1, 1, 4, AMODE, true, EPI, PF4 + 2>(a, blk * 32, n0 + sub * 32, true, 0, red, kslice, lane);
    __syncthreads();
  }
}

// Tall weight matrix (k-interleaved) times at most 32 columns: the output layer at the width the reference decodes at
// (one sentence, minibatch = beam).  The product is a stream of the matrix through the chip -- 200 MB for 1.2 GFLOP at
// 50 000 x 1000 x 12 -- so what matters is bytes in flight and how memory sees the fetches.  K split over the waves of a
// workgroup means a cross-wave sum through LDS and a ramp per pass (the row-range kernel: 50 us, 3.9 TB/s).  Here every
// WAVE takes two neighbouring 32-row blocks over all of K on its own, a ring of 10 fetch stages deep, two workgroups per
// compute unit: no LDS, no barrier, and the soft-max partials of a block are the wave's own rows.  Measured at
// 50 000 x 12 x 1000 (kernel time): one block per wave, ring of 12: 49.6 us; two blocks, ring of 10: 40.2 us (5.0 TB/s;
// a wave's two weight fetches of a stage are 1 KB of contiguous memory instead of 512 bytes); two blocks, ring of 14:
// 51.9; three blocks, ring of 8: 57.4; four blocks, ring of 6: 73.3 (too few bytes in flight).
// K % 8 == 0, k-interleaved activations.
template <int EPI, int WAUX>
__global__ void __launch_bounds__(256, 2) gemm_stream_kernel(GemmArgs a) {
  constexpr int PF = 10;
  const int lane = threadIdx.x & 63;
  const int wave = __builtin_amdgcn_readfirstlane((int)(blockIdx.x * 4 + (threadIdx.x >> 6)));
  const int n_waves = (int)gridDim.x * 4;
  const int blocks = (a.M + 31) >> 5;  // (the packed matrix holds exactly these rows: nothing beyond them is fetched)
  const int pairs = blocks >> 1;
  for (int b = wave; b < pairs; b += n_waves)
    gemm_tile<2, 1, 1, ZR_A_PACK4, true, EPI, PF, true, WAUX>(a, b * 64, 0, true, 0, nullptr, 0, lane);
  if ((blocks & 1) && wave == pairs % n_waves)  // an odd block at the end, on its own
    gemm_tile<1, 1, 1, ZR_A_PACK4, true, EPI, PF, true, WAUX>(a, (blocks - 1) * 32, 0, true, 0, nullptr, 0, lane);
}

// Tall weight matrix (k-interleaved) times a minibatch that is a multiple of 128 columns wide, balanced over the
// CUs without a persistent loop.  A workgroup takes one 64-row x 128-column tile; two workgroups share a CU (256
// registers each: 128 accumulators and a two-deep operand ring), so that the epilogue of one tile -- cross-wave sum,
// soft-max partials, stores: a fifth of a tile's time -- and the ramp-up of the next overlap the other workgroup's K
// loop instead of leaving the matrix pipe idle.  The number of such tiles is rarely a multiple of the number of CUs,
// and a last, mostly empty round costs as much as a full one.  So only as many
// 64-row tiles as fill whole rounds are taken that way (workgroups [0, n_big)); the rows left over go to the
// workgroups behind them as 32 x 32 tiles, which the hardware hands out as the CUs run dry, and whose round lasts an
// eighth of a big one.  Workgroup ids congruent modulo 8 share an XCD: each XCD takes a contiguous range of big row
// tiles and the column tiles of one row tile run side by side on it.
// Big tile of gemm_tall_kernel: 32*TM rows x 32*TN columns, operand ring PF deep, OCC workgroups per CU.  Measured on the 50000 x 128 x 1000 logits product (kernel time, us): one workgroup per CU with a six-deep
// ring (all 512 registers) 134-136; two per CU with a ring of two 119, of three 122, of one 122; 32 x 128 tiles at two
// per CU 123; 64 x 64 tiles at three per CU 123.  Giving every resident workgroup the same share of the rows (512
// workgroups of one 64-row and one 32-row tile each, all resident from start to end, instead of 768 tiles of which the
// last 256 run one to a CU) changed nothing: 123.9 us for the whole output layer either way.
// Minibatches that are a multiple of 64 but not of 128 columns wide (192 beam columns) take 64 x 64 tiles at three
// workgroups per CU.
template <int EPI, int TM, int TN, int PF, int OCC, int WAUX>
__global__ void __launch_bounds__(256, OCC) gemm_tall_kernel(GemmArgs a, int big_rows, int n_col_tiles, int n_big) {
  __shared__ float red[4 * TN * 16 * 64];
  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int kslice = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int bid = blockIdx.x;
  if (bid < n_big) {
    const int r8 = bid & 7, q = bid >> 3;
    const int mpx = big_rows >> 3;  // big_rows is a multiple of 8
    const int nt = q % n_col_tiles;
    const int mt = r8 * mpx + q / n_col_tiles;
    gemm_tile<TM, TN, 4, ZR_A_PACK4, true, EPI, PF, true, WAUX>(a, mt * 32 * TM, nt * 32 * TN, true, 0, red, kslice, lane);
  } else {
    const int idx = bid - n_big;
    const int n32 = (a.N + 31) >> 5;
    const int blk = big_rows * TM + idx / n32;
    gemm_tile<1, 1, 4, ZR_A_PACK4, true, EPI, 8>(a, blk * 32, (idx % n32) * 32, true, 0, red, kslice, lane);
  }
}

// Soft-max-partial epilogue for accumulators held the other way round: lane = column (n0 + 32*tn + lane % 32),
// register r = row m0 + 32*tm + 8*(r/4) + 4*(lane/32) + r%4.  A 32-row block's maximum and sum of exponentials are then
// 15 in-lane operations and one exchange between the half-waves each (against five cross-lane stages per VALUE when a
// lane holds one row), and a lane's four consecutive rows leave as one 16-byte store.  VEC: C + n*ldc is 16-byte aligned
// for every column and the tile lies wholly inside the matrix.
template <int TM, int TN, int TNI, bool VEC>
__device__ __forceinline__ void softmax_partial_epilogue_t_block(const GemmArgs& a, const zr_f32x16 (&acc)[TM][TN], int m0,
                                                                 int n0, int lane) {
  const int jl = lane & 31, half = lane >> 5;
  const int n = n0 + TNI * 32 + jl;
  const int nblocks = (a.M + 31) >> 5;
#pragma unroll
  for (int tm = 0; tm < TM; ++tm) {
    const int mb0 = m0 + tm * 32 + 4 * half;  // this lane's rows: mb0 + 8*q + i
    float v[16];
    bool ok[16];
#pragma unroll
    for (int q = 0; q < 4; ++q) {
      zr_f32x4 b4;
      if (VEC) {
        b4 = *(const zr_f32x4*)(a.bias + mb0 + 8 * q);
      } else {
        b4.x = a.bias[min(mb0 + 8 * q, a.M - 1)];
        b4.y = a.bias[min(mb0 + 8 * q + 1, a.M - 1)];
        b4.z = a.bias[min(mb0 + 8 * q + 2, a.M - 1)];
        b4.w = a.bias[min(mb0 + 8 * q + 3, a.M - 1)];
      }
      v[4 * q] = acc[tm][TNI][4 * q] + b4.x;
      v[4 * q + 1] = acc[tm][TNI][4 * q + 1] + b4.y;
      v[4 * q + 2] = acc[tm][TNI][4 * q + 2] + b4.z;
      v[4 * q + 3] = acc[tm][TNI][4 * q + 3] + b4.w;
#pragma unroll
      for (int i = 0; i < 4; ++i) ok[4 * q + i] = VEC || (mb0 + 8 * q + i < a.M && n < a.N);
    }
    float mx = -INFINITY;
#pragma unroll
    for (int r = 0; r < 16; ++r) mx = fmaxf(mx, ok[r] ? v[r] : -INFINITY);
    mx = fmaxf(mx, __shfl_xor(mx, 32, 64));
    float se = 0.0f;
#pragma unroll
    for (int r = 0; r < 16; ++r) se += ok[r] ? __builtin_amdgcn_exp2f((v[r] - mx) * 1.4426950408889634f) : 0.0f;
    se += __shfl_xor(se, 32, 64);
    float* cp = a.C + (long long)(n < a.N ? n : a.N - 1) * a.ldc + mb0;
#pragma unroll
    for (int q = 0; q < 4; ++q) {
      if (VEC) {
        *(zr_f32x4*)(cp + 8 * q) = zr_f32x4{v[4 * q], v[4 * q + 1], v[4 * q + 2], v[4 * q + 3]};
      } else {
#pragma unroll
        for (int i = 0; i < 4; ++i)
          if (ok[4 * q + i]) cp[8 * q + i] = v[4 * q + i];
      }
    }
    const int prow = (m0 >> 5) + tm;
    if (half == 0 && n < a.N && prow * 32 < a.M) {
      typedef float zr_f32x2 __attribute__((ext_vector_type(2)));
      *(zr_f32x2*)(a.partials + ((long long)n * nblocks + prow) * 2) = zr_f32x2{mx, se};
    }
  }
}

template <int TM, int TN, bool VEC, int... TNI>
__device__ __forceinline__ void softmax_partial_epilogue_t_blocks(const GemmArgs& a, const zr_f32x16 (&acc)[TM][TN],
                                                                  int m0, int n0, int lane, zr_int_seq<TNI...>) {
  (softmax_partial_epilogue_t_block<TM, TN, TNI, VEC>(a, acc, m0, n0, lane), ...);
}

template <int TM, int TN>
__device__ __forceinline__ void softmax_partial_epilogue_t(const GemmArgs& a, const zr_f32x16 (&acc)[TM][TN], int m0,
                                                           int n0, int lane) {
  const bool vec = m0 + 32 * TM <= a.M && n0 + 32 * TN <= a.N && (a.ldc & 3) == 0 && (m0 & 3) == 0 &&
                   (((uintptr_t)a.C | (uintptr_t)a.bias) & 15u) == 0;  // uniform
  if (vec)
    softmax_partial_epilogue_t_blocks<TM, TN, true>(a, acc, m0, n0, lane, zr_make_int_seq<TN>{});
  else
    softmax_partial_epilogue_t_blocks<TM, TN, false>(a, acc, m0, n0, lane, zr_make_int_seq<TN>{});
}

// ---------------------------------------------------------------------------------------------------------
// Tall bf16 weight matrix (k-interleaved by 8) times a minibatch of exactly 32*NB columns whose activations were
// rounded to bf16 once (single-term mode) or split into two bf16 terms, soft-max-partial epilogue: the output-layer
// product of the bf16 model.
// In bf16 a 32 x 32 x 16 matrix instruction takes 32 cycles for two 1 KB operands, so a K loop that fetches both
// operands of every wave from L2 is bound by that traffic, not by the matrix pipe.  Here
//   * the activations go through LDS: per 64-k chunk the workgroup copies 8 k-groups x 32*NB columns (a contiguous
//     4*NB KB of the packed array) into one of two LDS buffers with loads that write LDS directly (no staging
//     registers, no LDS store instructions), and every wave reads its operands from there;
//   * the four waves of a workgroup take DIFFERENT rows (64 each) and ALL the columns, so a weight element is
//     fetched by exactly one wave of the launch, straight into registers, one chunk ahead;
//   * one barrier per chunk, behind a wait for the chunk's fetches: the chunk after the current one lands in the other
//     buffer while the current one is multiplied.
// 64 x 256 accumulators per wave are 256 registers, which leaves the launch at one workgroup per CU, and the number of
// 64-row blocks is rarely a multiple of four per CU.  So only whole rounds of such workgroups are taken (ids below
// n_main); every 64-row block left over goes to one further workgroup whose four waves split the columns instead
// (the same staging; the weights of those few blocks are fetched by four waves each).
// ---------------------------------------------------------------------------------------------------------
// LO: two-term mode -- the activations come as two bf16 arrays (hi and lo, see zr_split_pack_multi_kernel) and every weight
// operand is multiplied with both (a chunk then holds CG k-groups of each term).
// PD: how many chunks ahead the weight fetches run (a ring of PD + 1 register sets; 1 with the LDS double buffer).
template <int TM, int TNW, int NB, int CG, bool LO, int PD>
__device__ __forceinline__ void bf16_lds_tile(const GemmArgs& a, zr_u32x4* sB, int m0, int nb0, int tid) {
  constexpr int STEPS = CG / 2;          // 16-k steps per chunk of CG k-groups of 8
  constexpr int NT = LO ? 2 : 1;         // activation terms
  constexpr int NP1 = NB * CG / 8;       // 4 KB pieces of one packed activation array per chunk, one 16-byte load each
  constexpr int NP = NP1 * NT;
  constexpr int N = 32 * NB;
  constexpr int BUF = NT * CG * N;       // 16-byte elements per LDS buffer: [term][k-group][column]
  const int lane = tid & 63, jl = lane & 31, half = lane >> 5;
  int rows[TM];
#pragma unroll
  for (int tm = 0; tm < TM; ++tm) {
    const int r = m0 + tm * 32 + jl;
    rows[tm] = r < a.M ? r : a.M - 1;
  }
  zr_f32x16 acc[TM][TNW];
#pragma unroll
  for (int tm = 0; tm < TM; ++tm)
#pragma unroll
    for (int tn = 0; tn < TNW; ++tn)
#pragma unroll
      for (int r = 0; r < 16; ++r) acc[tm][tn][r] = 0.0f;

  const unsigned lda16 = 16u * (unsigned)a.lda[0];
  const int kgroups = a.K[0] >> 3;
  const int nchunks = (kgroups + CG - 1) / CG;
  const __amdgpu_buffer_rsrc_t arsrc = __builtin_amdgcn_make_buffer_rsrc(const_cast<float*>(a.A[0]), 0,
                                                                         (unsigned)kgroups * lda16, 0x00020000);
  const __amdgpu_buffer_rsrc_t brsrc = __builtin_amdgcn_make_buffer_rsrc(const_cast<float*>(a.B[0]), 0,
                                                                         (unsigned)kgroups * (16u * N), 0x00020000);
  const __amdgpu_buffer_rsrc_t blrsrc = __builtin_amdgcn_make_buffer_rsrc(
      const_cast<unsigned short*>(LO ? a.Blo[0] : (const unsigned short*)a.B[0]), 0, (unsigned)kgroups * (16u * N), 0x00020000);
  unsigned aoff[TM];
#pragma unroll
  for (int tm = 0; tm < TM; ++tm) aoff[tm] = 16u * (unsigned)rows[tm] + (unsigned)half * lda16;
  const unsigned boff = 16u * (unsigned)tid;

  // Both operands are fetched through descriptors that end at k = K, with the whole offset in the per-lane part (the
  // part the bounds check looks at): the steps of the last chunk that lie past the end of K read zeros, so the loop needs
  // neither a tail nor a branch around its matrix instructions (which would turn every accumulator into a merge of two
  // values) nor selects behind its loads (which would make each load wait for its data where it is issued).
  auto load_a = [&](zr_u32x4 (&ar)[STEPS][TM], int c) {
#pragma unroll
    for (int st = 0; st < STEPS; ++st) {
      const unsigned koff = (unsigned)(c * CG + 2 * st) * lda16;  // uniform
#pragma unroll
      for (int tm = 0; tm < TM; ++tm)
        ar[st][tm] =
            __builtin_bit_cast(zr_u32x4, __builtin_amdgcn_raw_buffer_load_b128(arsrc, (int)(aoff[tm] + koff), 0, 0));
    }
  };
  // activations: straight from memory into LDS (each lane's 16 bytes land at the wave's base + 16 * lane)
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  auto load_b = [&](int c, int buf) {
#pragma unroll
    for (int i = 0; i < NP; ++i) {
      const unsigned off = boff + (unsigned)(c * NP1 + i % NP1) * 4096u;
      __builtin_amdgcn_raw_ptr_buffer_load_lds(i < NP1 ? brsrc : blrsrc,
                                               (__attribute__((address_space(3))) void*)(sB + buf * BUF + i * 256 + wave * 64),
                                               16, (int)off, 0, 0, 0);
    }
  };
  // one pass per (16-k step, term): the same weight operands against the hi octets, then against the lo octets
  auto compute = [&](const zr_u32x4 (&ar)[STEPS][TM], int buf) {
    const zr_u32x4* sb = sB + buf * BUF + half * N + nb0 * 32 + jl;
    constexpr int PASSES = STEPS * NT;
    auto frag = [&](int ps, int tn) { return sb[(ps % NT) * (CG * N) + 2 * (ps / NT) * N + tn * 32]; };
    zr_u32x4 bq[2][TNW];
#pragma unroll
    for (int tn = 0; tn < TNW; ++tn) bq[0][tn] = frag(0, tn);
#pragma unroll
    for (int ps = 0; ps < PASSES; ++ps) {
      if (ps + 1 < PASSES) {
#pragma unroll
        for (int tn = 0; tn < TNW; ++tn) bq[(ps + 1) & 1][tn] = frag(ps + 1, tn);
      }
#pragma unroll
      for (int tn = 0; tn < TNW; ++tn)
#pragma unroll
        for (int tm = 0; tm < TM; ++tm)
          // weights first: a lane ends up with one column and sixteen rows of each 32 x 32 block
          acc[tm][tn] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(zr_bf16x8, ar[ps / NT][tm]),
                                                                __builtin_bit_cast(zr_bf16x8, bq[ps & 1][tn]), acc[tm][tn],
                                                                0, 0, 0);
    }
  };

  // Ring of R = PD + 1 register sets for the weights and the staged activations.  One chunk ahead everywhere: two ahead
  // measured no faster for the row-split workgroups (95.8 against 93.1 us at 65536 rows), three ahead no faster for the
  // column-split ones (41.2 against 38.0 us for the 226 left-over blocks of 80000 rows), and neither did giving those
  // two row blocks each (49.7 us) or 128-k chunks (41.6 us).
  constexpr int R = PD + 1;
  static_assert(PD == 1, "the LDS double buffer is written one chunk ahead");
  zr_u32x4 ar[R][STEPS][TM];
  load_b(0, 0);
  load_a(ar[0], 0);
  __builtin_amdgcn_s_waitcnt(0x0F70);  // vmcnt(0): the LDS loads have landed
  __syncthreads();
  for (int c0 = 0; c0 < nchunks; c0 += R) {
#pragma unroll
    for (int u = 0; u < R; ++u) {
      const int c = c0 + u;
      // the fetches go out before this chunk's matrix work and stay there; the other LDS buffer was last read in chunk
      // c - 1, behind the barrier that ended it
      load_b(c + 1, (u + 1) & 1);
      load_a(ar[(u + 1) % R], c + 1);
      __builtin_amdgcn_sched_barrier(0);
      compute(ar[u], u & 1);
      __builtin_amdgcn_sched_barrier(0);
      __builtin_amdgcn_s_waitcnt(0x0F70);  // vmcnt(0)
      __syncthreads();
    }
  }
  softmax_partial_epilogue_t<TM, TNW>(a, acc, m0, nb0 * 32, lane);
}

template <int NB, bool LO>
__global__ void __launch_bounds__(256) gemm_bf16_lds_kernel(GemmArgs a, int n_main) {
  // chunks of 64 k (of each term); measured at 80000 x 256 x 2000: 128-k chunks no faster in single-term mode (126 us
  // either way), 32-k chunks of each term slower in two-term mode (212 against 195 us)
  constexpr int CG = 8;
  __shared__ zr_u32x4 sB[2 * (LO ? 2 : 1) * CG * 32 * NB];
  const int tid = threadIdx.x;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int bid = blockIdx.x;
  if (bid < n_main)
    bf16_lds_tile<2, NB, NB, CG, LO, 1>(a, sB, (bid * 4 + wave) * 64, 0, tid);
  else
    bf16_lds_tile<2, NB / 4, NB, CG, LO, 1>(a, sB, (n_main * 4 + (bid - n_main)) * 64, wave * (NB / 4), tid);
}

// ---------------------------------------------------------------------------------------------------------
// Large-M variant: weight rows staged through LDS and shared by all waves of the workgroup.
//
// A workgroup owns 32*TMR rows x 32*NWV columns; wave w owns columns [32w, 32w+32) and all TMR row sub-tiles, so
// every weight chunk (32 k x 32*TMR rows) is read from L2 once per workgroup with 16-byte coalesced loads,
// parked in LDS (double buffered, one barrier per chunk) and multiplied by every wave, while each wave fetches
// only its own 32 activation columns.  Against one 32x32 tile per wave this cuts the bytes pulled through the
// CU's L1 per flop by about TMR, which is what limited the softmax-logits GEMM (V x H times H x mb).
// Loads are unconditional (see zr_mfma_core.h on why) buffer loads whose descriptors end at the last valid element,
// so out-of-range weights read as zeros.  Requires: no transpose, one K segment, K a multiple of 8, M, lda, ldb
// multiples of 4, 16-byte aligned bases, both operands below 4 GiB.
// ---------------------------------------------------------------------------------------------------------
template <int TMR, int NWV, int EPI>
__global__ void __launch_bounds__(64 * NWV) gemm_lds_kernel(GemmArgs a) {
  constexpr int KC = 32;
  constexpr int NTHR = 64 * NWV;
  constexpr int F4 = KC * TMR * 8;                 // float4 per weight chunk
  constexpr int WLD = (F4 + NTHR - 1) / NTHR;      // float4 loads per thread per chunk
  __shared__ zr_f32x4 Ws4[2][F4];
  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int jl = lane & 31;
  const int half = lane >> 5;
  const int mt = blockIdx.x % a.m_tiles;
  const int nt = blockIdx.x / a.m_tiles;
  const int m0 = mt * 32 * TMR;
  const int n0 = nt * 32 * NWV + wave * 32;
  const int M = a.M, K = a.K[0];
  const long long lda = a.lda[0];
  const float* A = a.A[0];
  const int n_chunks = (K + KC - 1) / KC;

  int col = n0 + jl;
  col = col < a.N ? col : a.N - 1;
  // Operands come through buffer descriptors: address = base + a scalar byte offset that advances with the chunk +
  // a per-thread byte offset fixed for the whole loop, so the loop holds no vector address arithmetic.  The
  // descriptors end exactly at the last valid element: a read past it (the K tail of the last chunk, the dummy chunk
  // of an odd chunk count) returns zeros, which is what those weights must be.  Rows past M are clamped to valid
  // rows instead; what they produce lands in output rows that are never stored.  Requires K % 8 == 0 (host-checked).
  const __amdgpu_buffer_rsrc_t wrsrc = __builtin_amdgcn_make_buffer_rsrc(
      const_cast<float*>(A), 0, (int)(unsigned)((((long long)K - 1) * lda + M) * 4), 0x00020000);
  const __amdgpu_buffer_rsrc_t xrsrc = __builtin_amdgcn_make_buffer_rsrc(
      const_cast<float*>(a.B[0]), 0, (int)(unsigned)((((long long)a.N - 1) * a.ldb[0] + K) * 4), 0x00020000);
  const unsigned xoffb = 4u * ((unsigned)col * (unsigned)a.ldb[0] + 4u * (unsigned)half);

  unsigned woffb[WLD];
#pragma unroll
  for (int u = 0; u < WLD; ++u) {
    const int f = tid + NTHR * u;
    const int fc = f < F4 ? f : F4 - 1;
    const int j4 = fc & 7, tm = (fc >> 3) % TMR, kk = fc / (8 * TMR);
    const int row = m0 + 32 * tm + 4 * j4;
    woffb[u] = 4u * ((unsigned)(row < M ? row : M - 4) + (unsigned)kk * (unsigned)lda);
  }

  zr_f32x16 acc[TMR];
#pragma unroll
  for (int tm = 0; tm < TMR; ++tm)
#pragma unroll
    for (int r = 0; r < 16; ++r) acc[tm][r] = 0.0f;

  zr_u32x4v wreg[WLD];
  zr_f32x4 xf[2][4];
  // gload only issues loads (the values stay in registers while the current chunk is multiplied) so that several
  // loads stay in flight.
  auto gload = [&](int c, zr_f32x4 (&xdst)[4]) {
    const unsigned wso = (unsigned)c * (unsigned)(KC * 4) * (unsigned)lda;
#pragma unroll
    for (int u = 0; u < WLD; ++u)  // the scalar-offset operand is exempt from the range check: add it on the vector side
      wreg[u] = __builtin_amdgcn_raw_buffer_load_b128(wrsrc, (int)(woffb[u] + wso), 0, 0);
#pragma unroll
    for (int gq = 0; gq < 4; ++gq) {
      int kx = c * KC + 8 * gq;
      kx = kx + 8 <= K ? kx : K - 8;  // wave-uniform: the weights of the k values this replaces are zeros
      const zr_u32x4v v = __builtin_amdgcn_raw_buffer_load_b128(xrsrc, (int)(xoffb + (unsigned)kx * 4u), 0, 0);
      xdst[gq].x = __uint_as_float(v.x);
      xdst[gq].y = __uint_as_float(v.y);
      xdst[gq].z = __uint_as_float(v.z);
      xdst[gq].w = __uint_as_float(v.w);
    }
  };
  auto lds_store = [&](int buf, int) {
#pragma unroll
    for (int u = 0; u < WLD; ++u) {
      const int f = tid + NTHR * u;
      zr_f32x4 v;
      v.x = __uint_as_float(wreg[u].x);
      v.y = __uint_as_float(wreg[u].y);
      v.z = __uint_as_float(wreg[u].z);
      v.w = __uint_as_float(wreg[u].w);
      if (f < F4) Ws4[buf][f] = v;
    }
  };
  auto compute = [&](int buf, const zr_f32x4 (&xs)[4]) {
    // chunk layout in LDS: [kk][tm][32 rows]
    const float* Ws = (const float*)&Ws4[buf][0] + (4 * half * TMR) * 32 + jl;
    float wf[2][4][TMR];
    auto lds_frag = [&](float (&dst)[4][TMR], int gq) {
#pragma unroll
      for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int tm = 0; tm < TMR; ++tm) dst[i][tm] = Ws[((8 * gq + i) * TMR + tm) * 32];
    };
    lds_frag(wf[0], 0);
#pragma unroll
    for (int gq = 0; gq < 4; ++gq) {
      if (gq + 1 < 4) lds_frag(wf[(gq + 1) & 1], gq + 1);
#pragma unroll
      for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int tm = 0; tm < TMR; ++tm)
          acc[tm] = __builtin_amdgcn_mfma_f32_32x32x2f32(xs[gq][i], wf[gq & 1][i][tm], acc[tm], 0, 0, 0);
      // issue order within this group: one LDS read of the next fragment behind each MFMA, so that the reads hide
      // under the matrix pipe instead of stalling it in a burst (and never slide down to just before their use)
#pragma unroll
      for (int j = 0; j < 4 * TMR; ++j) {
        __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);  // one MFMA
        __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);  // one LDS read
      }
      __builtin_amdgcn_sched_barrier(0);
    }
  };

  gload(0, xf[0]);
  lds_store(0, 0);
  __syncthreads();
  for (int c = 0; c < n_chunks; c += 2) {
    gload(c + 1, xf[1]);
    compute(0, xf[0]);
    lds_store(1, c + 1);
    __syncthreads();
    gload(c + 2, xf[0]);
    compute(1, xf[1]);
    lds_store(0, c + 2);
    __syncthreads();
  }

  float bias_v[TMR];
#pragma unroll
  for (int tm = 0; tm < TMR; ++tm) {
    const int m = m0 + tm * 32 + jl;
    bias_v[tm] = a.bias ? a.bias[m < M ? m : M - 1] : 0.0f;
  }
  if (EPI == ZR_EPI_STORE) {
#pragma unroll
    for (int r = 0; r < 16; ++r) {
      const int n = n0 + 8 * (r >> 2) + 4 * half + (r & 3);
#pragma unroll
      for (int tm = 0; tm < TMR; ++tm) {
        const int m = m0 + tm * 32 + jl;
        if (n < a.N && m < M) {
          float* cp = a.C + (long long)n * a.ldc + m;
          const float v = acc[tm][r] + bias_v[tm];
          *cp = a.accum ? *cp + v : v;
        }
      }
    }
  } else {  // ZR_EPI_SOFTMAX_PARTIAL: four columns (accumulator registers) of all row sub-tiles at a time
#pragma unroll
    for (int rg = 0; rg < 4; ++rg) {
      float v[4 * TMR], mx[4 * TMR], se[4 * TMR];
      bool ok[4 * TMR];
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        const int n = n0 + 8 * rg + 4 * half + i;
#pragma unroll
        for (int tm = 0; tm < TMR; ++tm) {
          v[i * TMR + tm] = acc[tm][4 * rg + i] + bias_v[tm];
          ok[i * TMR + tm] = n < a.N && (m0 + tm * 32 + jl) < M;
        }
      }
      zr_half_wave_softmax_stats<4 * TMR>(v, ok, mx, se);
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        const int n = n0 + 8 * rg + 4 * half + i;
#pragma unroll
        for (int tm = 0; tm < TMR; ++tm) {
          const int m = m0 + tm * 32 + jl;
          if (ok[i * TMR + tm]) a.C[(long long)n * a.ldc + m] = v[i * TMR + tm];
          const int prow = (m0 >> 5) + tm;
          if (jl == 0 && n < a.N && prow * 32 < M) {
            float* p = a.partials + ((long long)n * ((a.M + 31) >> 5) + prow) * 2;
            p[0] = mx[i * TMR + tm];
            p[1] = se[i * TMR + tm];
          }
        }
      }
    }
  }
}

template <int TMR, int NWV>
int launch_lds(zr_ctx* ctx, GemmArgs& ga, int epi) {
  ga.m_tiles = (ga.M + 32 * TMR - 1) / (32 * TMR);
  ga.n_tiles = (ga.N + 32 * NWV - 1) / (32 * NWV);
  const unsigned grid = (unsigned)ga.m_tiles * ga.n_tiles;
  if (epi == ZR_EPI_STORE)
    gemm_lds_kernel<TMR, NWV, ZR_EPI_STORE><<<grid, 64 * NWV, 0, ctx->stream>>>(ga);
  else
    gemm_lds_kernel<TMR, NWV, ZR_EPI_SOFTMAX_PARTIAL><<<grid, 64 * NWV, 0, ctx->stream>>>(ga);
  ZR_LAUNCH_CHECK("gemm_lds_kernel");
  return ZR_OK;
}

template <int NWV>
int launch_lds_rows(zr_ctx* ctx, GemmArgs& ga, int epi) {
  // row sub-tiles per workgroup: the choice that needs fewer rounds of 256 workgroups per unit of tile height
  const int blocks = (ga.M + 31) / 32;
  const int ncol = (ga.N + 32 * NWV - 1) / (32 * NWV);
  const long long wg7 = (long long)((blocks + 6) / 7) * ncol, wg4 = (long long)((blocks + 3) / 4) * ncol;
  const long long cost7 = ((wg7 + 255) / 256) * 7, cost4 = ((wg4 + 255) / 256) * 4;
  // 7 row sub-tiles need 112 accumulator registers: only with 4 waves per workgroup (one per SIMD) is the full
  // register file available to a wave
  if (NWV == 4 && cost7 <= cost4) return launch_lds<7, 4>(ctx, ga, epi);
  return launch_lds<4, NWV>(ctx, ga, epi);
}

template <int TM, int TN, int KS, int WPB, int AMODE, bool VEC, int OCC = 1>
int launch_epi(zr_ctx* ctx, const GemmArgs& ga, int batch, int epi) {
  long long ntiles = (long long)ga.m_tiles * ga.n_tiles;
  dim3 grid((unsigned)((ntiles + WPB - 1) / WPB), 1, batch);
  if (AMODE == ZR_A_PACK4 || zr_is_bf16_mode(AMODE)) {
    // XCD-major id space: 8 ranges of ceil(m_tiles/8) row tiles x n_tiles wave tiles, WPB wave tiles per workgroup
    const long long per_xcd = (long long)((ga.m_tiles + 7) / 8) * ga.n_tiles;
    grid.x = (unsigned)(((per_xcd + WPB - 1) / WPB) * 8);
  }
  dim3 block(64 * KS * WPB);
  switch (epi) {
    case ZR_EPI_STORE:
      gemm_kernel<TM, TN, KS, WPB, AMODE, VEC, ZR_EPI_STORE, OCC><<<grid, block, 0, ctx->stream>>>(ga);
      break;
    case ZR_EPI_TANH:
      gemm_kernel<TM, TN, KS, WPB, AMODE, VEC, ZR_EPI_TANH, OCC><<<grid, block, 0, ctx->stream>>>(ga);
      break;
    case ZR_EPI_TANH_BIAS_MASK:
      gemm_kernel<TM, TN, KS, WPB, AMODE, VEC, ZR_EPI_TANH_BIAS_MASK, OCC><<<grid, block, 0, ctx->stream>>>(ga);
      break;
    default:
      gemm_kernel<TM, TN, KS, WPB, AMODE, VEC, ZR_EPI_SOFTMAX_PARTIAL, OCC><<<grid, block, 0, ctx->stream>>>(ga);
      break;
  }
  ZR_LAUNCH_CHECK("gemm_kernel");
  return ZR_OK;
}

template <int TM, int TN, int KS, int WPB>
int launch_cfg(zr_ctx* ctx, GemmArgs& ga, int batch, int epi, bool trans_a, bool vec) {
  ga.m_tiles = (ga.M + 32 * TM - 1) / (32 * TM);
  ga.n_tiles = (ga.N + 32 * TN - 1) / (32 * TN);
  if (trans_a) {
    if (vec) return launch_epi<TM, TN, KS, WPB, ZR_A_TRANS, true>(ctx, ga, batch, epi);
    return launch_epi<TM, TN, KS, WPB, ZR_A_TRANS, false>(ctx, ga, batch, epi);
  }
  if (vec) return launch_epi<TM, TN, KS, WPB, ZR_A_NN, true>(ctx, ga, batch, epi);
  return launch_epi<TM, TN, KS, WPB, ZR_A_NN, false>(ctx, ga, batch, epi);
}

// k-interleaved weights: one wave tile per workgroup, K split over its 4 waves
template <int TM, int TN, int OCC>
int launch_pack4(zr_ctx* ctx, GemmArgs& ga, int epi, bool vec, int zcount) {
  ga.m_tiles = (ga.M + 32 * TM - 1) / (32 * TM);
  ga.n_tiles = (ga.N + 32 * TN - 1) / (32 * TN);
  if (vec) return launch_epi<TM, TN, 4, 1, ZR_A_PACK4, true, OCC>(ctx, ga, zcount, epi);
  return launch_epi<TM, TN, 4, 1, ZR_A_PACK4, false, OCC>(ctx, ga, zcount, epi);
}

// Activations X (K x N, column n at src + n*ld) into [K/4][N][4]; K % 4 == 0.  One thread per float4.
__global__ void __launch_bounds__(256) pack4_x_kernel(const float* __restrict__ src, int K, int N, int ld,
                                                      float* __restrict__ dst) {
  const int i = blockIdx.x * 256 + threadIdx.x;  // float4 index in the source order: (n, k/4)
  const int kb = K >> 2;
  if (i >= kb * N) return;
  const int n = i / kb, b = i - n * kb;
  const zr_f32x4 v = *(const zr_f32x4*)(src + (long long)n * ld + 4 * b);
  *(zr_f32x4*)(dst + ((long long)b * N + n) * 4) = v;
}

template <int TN, int AMODE = ZR_A_PACK4>
int launch_rows(zr_ctx* ctx, GemmArgs& ga, int epi, int n_tiles) {
  ga.n_tiles = n_tiles;
  ga.m_tiles = 0;
  const int blocks = (ga.M + 31) / 32;
  int row_chunks = 256 / n_tiles;  // one workgroup per CU
  if (row_chunks > blocks) row_chunks = blocks;
  const unsigned grid = (unsigned)((row_chunks + 7) / 8) * 8 * n_tiles;
  if (epi == ZR_EPI_STORE)
    gemm_rows_kernel<TN, ZR_EPI_STORE, AMODE><<<grid, 256, 0, ctx->stream>>>(ga, row_chunks);
  else
    gemm_rows_kernel<TN, ZR_EPI_SOFTMAX_PARTIAL, AMODE><<<grid, 256, 0, ctx->stream>>>(ga, row_chunks);
  ZR_LAUNCH_CHECK("gemm_rows_kernel");
  return ZR_OK;
}

// gemm_bf16_lds_kernel: whole rounds of four-block workgroups, one further workgroup per 64-row block left over.
template <int NB, bool LO>
int launch_bf16_lds(zr_ctx* ctx, GemmArgs& ga) {
  const int nb64 = (ga.M + 63) / 64;
  const int cus = ctx->cu_count > 0 ? ctx->cu_count : 256;
  const int n_main = nb64 / (4 * cus) * cus;
  const int rest = nb64 - 4 * n_main;
  ga.m_tiles = ga.n_tiles = 0;
  gemm_bf16_lds_kernel<NB, LO><<<(unsigned)(n_main + rest), 256, 0, ctx->stream>>>(ga, n_main);
  ZR_LAUNCH_CHECK("gemm_bf16_lds_kernel");
  return ZR_OK;
}

// gemm_tall_kernel: N a multiple of 128, fp32 k-interleaved A.  Returns false when the shape is better served by the
// row-range kernel (too many rows would be left to the small tiles).
template <int TM, int TN, int PF, int OCC>
bool launch_tall_v(zr_ctx* ctx, GemmArgs& ga, int epi, int* rc) {
  const int blocks = (ga.M + 31) / 32;
  const int n_col_tiles = ga.N / (32 * TN);
  const int n32 = ga.N / 32;
  const long long row_tiles = blocks / TM;  // whole big row tiles
  // as many big row tiles as fill whole rounds of 256 workgroups, a multiple of 8 of them
  long long big_rows = (row_tiles * n_col_tiles / 256) * 256 / n_col_tiles;
  big_rows = big_rows / 8 * 8;
  const long long small = (long long)(blocks - TM * big_rows) * n32;
  const bool offsets_fit = (long long)ga.K[0] * ga.lda[0] * 4 + 4096 < (1LL << 32) && (long long)ga.K[0] * ga.N * 4 < (1LL << 32);
  if (big_rows == 0 || small > 1024 || !offsets_fit) {
    // the left-over rows would be more than four rounds of small tiles: leave the shape to the row-range kernel
    return false;
  }
  ga.m_tiles = ga.n_tiles = 0;
  const int n_big = (int)(big_rows * n_col_tiles);
  const unsigned grid = (unsigned)(n_big + small);
  if (epi == ZR_EPI_STORE)
    gemm_tall_kernel<ZR_EPI_STORE, TM, TN, PF, OCC, 0><<<grid, 256, 0, ctx->stream>>>(ga, (int)big_rows, n_col_tiles, n_big);
  else if (ga.stream_a)
    gemm_tall_kernel<ZR_EPI_SOFTMAX_PARTIAL, TM, TN, PF, OCC, ZR_AUX_STREAM><<<grid, 256, 0, ctx->stream>>>(
        ga, (int)big_rows, n_col_tiles, n_big);
  else
    gemm_tall_kernel<ZR_EPI_SOFTMAX_PARTIAL, TM, TN, PF, OCC, 0><<<grid, 256, 0, ctx->stream>>>(ga, (int)big_rows,
                                                                                               n_col_tiles, n_big);
  hipError_t e = hipGetLastError();
  *rc = e == hipSuccess ? ZR_OK : zr_set_error(ZR_EHIP, "launch of gemm_tall_kernel failed: %s", hipGetErrorString(e));
  return true;
}

// gemm_tall_kernel: N a multiple of 128, 96 or 64 (column tiles of that width: two workgroups per CU at 128, three
// below), fp32 k-interleaved A.  Returns false when the shape is better served by the row-range kernel (too many rows
// would be left to the small tiles).  Measured at 50000 x 192 x 1000: row ranges 201 us, 64 x 64 tiles 190, 64 x 96 182.
bool launch_tall(zr_ctx* ctx, GemmArgs& ga, int epi, int* rc) {
  if (ga.N % 128 == 0) return launch_tall_v<2, 4, 2, 2>(ctx, ga, epi, rc);
  if (ga.N % 96 == 0) return launch_tall_v<2, 3, 2, 3>(ctx, ga, epi, rc);
  return launch_tall_v<2, 2, 2, 3>(ctx, ga, epi, rc);
}

// Activations X (K x N fp32, column n at src + n*ld, K % 8 == 0) -> two bf16 arrays hi and lo with x = hi + lo up
// to 2^-16 |x|, each k-interleaved by 8: element (k, n) at ((k/8)*N + n)*8 + k%8.
// A workgroup takes 16 columns x 16 k-groups, one per thread, and turns them through LDS: it reads with 16 consecutive
// lanes on 16 consecutive k-groups of one column (512 bytes contiguous) and writes with 16 consecutive lanes on 16
// consecutive columns of one k-group (256 bytes contiguous); small tiles, because a single 2000 x 256 array must still
// spread over the chip (250 workgroups).  With one thread per k-group writing its 16 bytes where they belong, consecutive
// lanes stored 16-byte pieces N*16 bytes apart: 11 us for the six 2000 x 256 arrays of a config-5 step.
// Up to kSplitMultiMax matrices of one shape per launch (blockIdx.z picks the matrix): a decoder step splits the previous
// state of every layer, the previous attention output and the embedding columns of the current words at its start, and
// each of them as a launch of its own costs more in launch latency than in work.  Matrix i goes to hi + i*stride
// (lo + i*stride); ids (or null) turns matrix 0 into a gather, column n read from src[0] + ids[n]*ld (ids outside
// [0, V) are clamped, as the gather kernel does).
constexpr int kSplitMultiMax = 12;
struct SplitMulti {
  const float* src[kSplitMultiMax];
  const int* ids;
  int V;
};
__global__ void __launch_bounds__(256) zr_split_pack_multi_kernel(SplitMulti m, int K, int N, int ld,
                                                                  unsigned short* __restrict__ hi,
                                                                  unsigned short* __restrict__ lo, long long stride) {
  __shared__ zr_u32x4 s_hi[16][17], s_lo[16][17];  // [column][k-group], a row padded by one item
  const int tid = threadIdx.x;
  const int kb = K >> 3;
  const int b0 = blockIdx.x * 16, n0 = blockIdx.y * 16;
  const int which = blockIdx.z;
  const int lx = tid & 15, ly = tid >> 4;
  {
    const int n = n0 + ly, b = b0 + lx;
    if (n < N && b < kb) {
      long long col = n;
      if (which == 0 && m.ids) {
        const int v = m.ids[n];
        col = v < 0 ? 0 : (v >= m.V ? m.V - 1 : v);
      }
      const float* src = m.src[which] + col * ld + 8 * b;
      const zr_f32x4 v0 = *(const zr_f32x4*)src;
      const zr_f32x4 v1 = *(const zr_f32x4*)(src + 4);
      zr_u32x4 h, l;
      unsigned x, y;
      zr_split_bf16_pair(v0.x, v0.y, x, y); h.x = x; l.x = y;
      zr_split_bf16_pair(v0.z, v0.w, x, y); h.y = x; l.y = y;
      zr_split_bf16_pair(v1.x, v1.y, x, y); h.z = x; l.z = y;
      zr_split_bf16_pair(v1.z, v1.w, x, y); h.w = x; l.w = y;
      s_hi[ly][lx] = h;
      if (lo) s_lo[ly][lx] = l;
    }
  }
  __syncthreads();
  {
    const int n = n0 + lx, b = b0 + ly;
    if (n < N && b < kb) {
      const long long o = which * stride + ((long long)b * N + n) * 8;
      *(zr_u32x4*)(hi + o) = s_hi[lx][ly];
      if (lo) *(zr_u32x4*)(lo + o) = s_lo[lx][ly];  // null: single-term mode, the residues are dropped
    }
  }
}

__global__ void __launch_bounds__(256) pack4_kernel(const float* __restrict__ src, int M, int K, long long ld,
                                                    int ldp, int kp, float* __restrict__ dst) {
  const long long i = (long long)blockIdx.x * 256 + threadIdx.x;
  if (i >= (long long)kp * ldp) return;
  const int k4 = (int)(i & 3);
  const long long t = i >> 2;
  const int row = (int)(t % ldp);
  const int k = (int)(t / ldp) * 4 + k4;
  dst[i] = (row < M && k < K) ? src[row + (long long)k * ld] : 0.0f;
}

// The same for the TRANSPOSE of the source: element (row, k) of the packed matrix is src[k + row*ld].
__global__ void __launch_bounds__(256) pack4_trans_kernel(const float* __restrict__ src, int M, int K, long long ld,
                                                          int ldp, int kp, float* __restrict__ dst) {
  const long long i = (long long)blockIdx.x * 256 + threadIdx.x;
  if (i >= (long long)kp * ldp) return;
  const int k4 = (int)(i & 3);
  const long long t = i >> 2;
  const int row = (int)(t % ldp);
  const int k = (int)(t / ldp) * 4 + k4;
  dst[i] = (row < M && k < K) ? src[k + (long long)row * ld] : 0.0f;
}

__global__ void __launch_bounds__(256) pack8_bf16_kernel(const float* __restrict__ src, int M, int K, long long ld,
                                                         int ldp, int kp, unsigned short* __restrict__ dst, int trans) {
  const long long i = (long long)blockIdx.x * 256 + threadIdx.x;
  if (i >= (long long)kp * ldp) return;
  const int k8 = (int)(i & 7);
  const long long t = i >> 3;
  const int row = (int)(t % ldp);
  const int k = (int)(t / ldp) * 8 + k8;
  const float v = (row < M && k < K) ? (trans ? src[k + (long long)row * ld] : src[row + (long long)k * ld]) : 0.0f;
  dst[i] = __builtin_bit_cast(unsigned short, (__bf16)v);
}

}  // namespace

int zr_pack8_bf16_launch(zr_ctx* ctx, const float* src, int M, int K, long long ld, int ldp, int kp,
                         unsigned short* dst, int trans) {
  const long long total = (long long)kp * ldp;
  pack8_bf16_kernel<<<(unsigned)((total + 255) / 256), 256, 0, ctx->stream>>>(src, M, K, ld, ldp, kp, dst, trans);
  ZR_LAUNCH_CHECK("pack8_bf16_kernel");
  return ZR_OK;
}

int zr_split_pack_multi_launch(zr_ctx* ctx, int n_src, const float* const* srcs, const int* d_ids, int V, int K, int N,
                               int ld, unsigned short* hi, unsigned short* lo, long long stride) {
  if (n_src < 1 || n_src > kSplitMultiMax) return zr_set_error(ZR_EINVAL, "split: %d matrices in one launch", n_src);
  SplitMulti m = {};
  for (int i = 0; i < n_src; ++i) m.src[i] = srcs[i];
  m.ids = d_ids;
  m.V = V;
  const dim3 grid((unsigned)((K / 8 + 15) / 16), (unsigned)((N + 15) / 16), (unsigned)n_src);
  if (grid.y > 65535) return zr_set_error(ZR_EINVAL, "split: %d columns", N);
  zr_split_pack_multi_kernel<<<grid, 256, 0, ctx->stream>>>(m, K, N, ld, hi, lo, stride);
  ZR_LAUNCH_CHECK("zr_split_pack_multi_kernel");
  return ZR_OK;
}

int zr_split_pack_x_launch(zr_ctx* ctx, const float* src, int K, int N, int ld, unsigned short* hi,
                           unsigned short* lo) {
  const float* srcs[1] = {src};
  return zr_split_pack_multi_launch(ctx, 1, srcs, nullptr, 0, K, N, ld, hi, lo, 0);
}

int zr_pack4_launch(zr_ctx* ctx, const float* src, int M, int K, long long ld, int ldp, int kp, float* dst) {
  const long long total = (long long)kp * ldp;
  pack4_kernel<<<(unsigned)((total + 255) / 256), 256, 0, ctx->stream>>>(src, M, K, ld, ldp, kp, dst);
  ZR_LAUNCH_CHECK("pack4_kernel");
  return ZR_OK;
}

int zr_pack4_x_launch(zr_ctx* ctx, const float* src, int K, int N, int ld, float* dst) {
  const int f4 = (K / 4) * N;
  pack4_x_kernel<<<(f4 + 255) / 256, 256, 0, ctx->stream>>>(src, K, N, ld, dst);
  ZR_LAUNCH_CHECK("pack4_x_kernel");
  return ZR_OK;
}

int zr_pack4_trans_launch(zr_ctx* ctx, const float* src, int M, int K, long long ld, int ldp, int kp, float* dst) {
  const long long total = (long long)kp * ldp;
  pack4_trans_kernel<<<(unsigned)((total + 255) / 256), 256, 0, ctx->stream>>>(src, M, K, ld, ldp, kp, dst);
  ZR_LAUNCH_CHECK("pack4_trans_kernel");
  return ZR_OK;
}

int zr_gemm_launch(zr_ctx* ctx, const ZrGemmDesc& d) {
  ZR_CHECK_ARG(d.M > 0 && d.N > 0, "gemm: M = %d, N = %d", d.M, d.N);
  ZR_CHECK_ARG(d.nseg >= 1 && d.nseg <= 3, "gemm: nseg = %d", d.nseg);
  ZR_CHECK_ARG((d.groups > 0 || d.C != nullptr) && d.ldc >= d.M, "gemm: C null or ldc %d < M %d", d.ldc, d.M);
  ZR_CHECK_ARG(d.batch >= 1 && d.batch <= 65535, "gemm: batch = %d", d.batch);
  ZR_CHECK_ARG(d.groups >= 0 && d.groups <= 8, "gemm: groups = %d", d.groups);
  if (d.groups > 0) {
    ZR_CHECK_ARG(d.nseg == 1 && d.epilogue == ZR_EPI_STORE && !d.bias && d.a_pack != 2 && d.batch * d.groups <= 65535,
                 "gemm: grouped problems take one segment, the plain store epilogue, no bias and fp32 operands");
    for (int g = 0; g < d.groups; ++g)
      ZR_CHECK_ARG(d.gA[g] && d.gB[g] && d.gC[g], "gemm: null operand in group %d", g);
  }
  GemmArgs ga;
  ga.groups = d.groups;
  ga.batch = d.batch;
  for (int g = 0; g < 8; ++g) {
    ga.gA[g] = g < d.groups ? d.gA[g] : nullptr;
    ga.gB[g] = g < d.groups ? d.gB[g] : nullptr;
    ga.gC[g] = g < d.groups ? d.gC[g] : nullptr;
  }
  const int zcount = d.batch * (d.groups > 0 ? d.groups : 1);  // grid depth
  ga.M = d.M;
  ga.N = d.N;
  ga.nseg = d.nseg;
  bool vec = true;
  long long flops = 0;
  for (int s = 0; s < 3; ++s) {
    if (s < d.nseg) {
      ZR_CHECK_ARG(d.K[s] > 0, "gemm: K[%d] = %d", s, d.K[s]);
      ZR_CHECK_ARG(d.groups > 0 || (d.A[s] && d.B[s]), "gemm: null operand in segment %d", s);
      ZR_CHECK_ARG(d.lda[s] >= (d.trans_a ? d.K[s] : d.M), "gemm: lda[%d] = %d too small", s, d.lda[s]);
      ZR_CHECK_ARG(!d.a_pack || (!d.trans_a && d.lda[s] % 32 == 0 && 8LL * d.lda[s] + 8LL * d.M < (1LL << 31)),
                   "gemm: packed operand A of segment %d: needs no transpose, lda a multiple of 32", s);
      // a batch over bf16 matrices: one segment, plain store, and a shape the tile kernel serves (strideA in bf16 elements)
      ZR_CHECK_ARG(d.a_pack != 2 || d.batch == 1 ||
                       (d.nseg == 1 && d.epilogue == ZR_EPI_STORE && d.M < 8192 && d.strideA % 8 == 0),
                   "gemm: a batch of bf16 products needs one segment, the store epilogue and M < 8192");
      ZR_CHECK_ARG(d.a_pack != 2 || d.K[s] % 16 == 0, "gemm: bf16 operand A needs K %% 16 == 0 (K[%d] = %d)", s, d.K[s]);
      ZR_CHECK_ARG(d.ldb[s] >= d.K[s], "gemm: ldb[%d] = %d < K = %d", s, d.ldb[s], d.K[s]);
      // per-lane weight offsets are 32-bit element indices
      ZR_CHECK_ARG(d.trans_a ? ((long long)d.M * d.lda[s] + 8 < (1LL << 31)) : (d.M + 8LL * d.lda[s] < (1LL << 31)),
                   "gemm: operand A of segment %d is too large for 32-bit offsets", s);
      ga.K[s] = d.K[s];
      ga.A[s] = d.A[s];
      ga.lda[s] = d.lda[s];
      ga.B[s] = d.B[s];
      ga.ldb[s] = d.ldb[s];
      vec = vec && (d.ldb[s] % 4 == 0) && (((uintptr_t)d.B[s] & 15u) == 0);
      for (int g = 0; g < d.groups; ++g) vec = vec && (((uintptr_t)d.gB[g] & 15u) == 0);
      if (d.trans_a) {
        vec = vec && (d.lda[s] % 4 == 0) && (((uintptr_t)d.A[s] & 15u) == 0) && (d.strideA % 4 == 0);
        for (int g = 0; g < d.groups; ++g) vec = vec && (((uintptr_t)d.gA[g] & 15u) == 0);
      }
      flops += 2LL * d.M * d.N * d.K[s];
    } else {
      ga.K[s] = 0;
      ga.A[s] = nullptr;
      ga.lda[s] = 0;
      ga.B[s] = nullptr;
      ga.ldb[s] = 0;
    }
  }
  ga.C = d.C;
  ga.ldc = d.ldc;
  ga.strideA = d.strideA;
  ga.strideC = d.strideC;
  ga.strideBias = d.strideBias;
  ga.bias = d.bias;
  ga.mask = d.mask;
  ga.partials = d.partials;
  ga.Cpack = d.Cpack;
  ga.Chi = d.Chi;
  ga.Clo = d.Clo;
  ZR_CHECK_ARG(!d.Chi || (d.epilogue == ZR_EPI_TANH_BIAS_MASK && d.batch <= 1 && d.groups == 0 && d.M % 8 == 0),
               "gemm: bf16 terms of the result need the tanh-bias-mask epilogue, one batch and M %% 8 == 0");
  ZR_CHECK_ARG(!d.Clo || d.Chi, "gemm: Clo without Chi");
  ZR_CHECK_ARG(!d.Cpack || (d.epilogue == ZR_EPI_TANH_BIAS_MASK && d.batch <= 1 && d.groups == 0),
               "gemm: a k-interleaved second result needs the tanh-bias-mask epilogue and a single problem");
  ga.accum = d.accumulate;
  ga.stream_a = d.stream_a;
  if (d.epilogue == ZR_EPI_TANH_BIAS_MASK) ZR_CHECK_ARG(d.bias && d.mask, "gemm: bias/mask required");
  ZR_CHECK_ARG(!d.accumulate || d.epilogue == ZR_EPI_STORE, "gemm: accumulate needs the plain store epilogue");
  if (d.epilogue == ZR_EPI_SOFTMAX_PARTIAL) ZR_CHECK_ARG(d.bias && d.partials, "gemm: bias/partials required");

  ga.b_pack4 = 0;
  for (int s = 0; s < 3; ++s) ga.Blo[s] = nullptr;
  if (d.a_pack == 2) {
    ZR_CHECK_ARG(vec, "gemm: bf16 operand A needs 16-byte aligned activations with ldb %% 4 == 0");
    const bool one_term = ctx->bf16_terms == 1;
    {
      // split the fp32 activations into bf16 hi + lo once, k-interleaved, instead of in every workgroup's K loop
      size_t elems = 0;
      for (int s = 0; s < d.nseg; ++s) elems += (size_t)d.K[s] * d.N;
      void* p = nullptr;
      int rc = zr_ctx_scratch(ctx, 0, sizeof(unsigned short) * 2 * elems, &p);
      if (rc) return rc;
      unsigned short* hi = (unsigned short*)p;
      for (int s = 0; s < d.nseg; ++s) {
        const size_t e = (size_t)d.K[s] * d.N;
        const bool lo = !one_term;
        if (d.Bhi[s] && (one_term || d.Blo[s])) {  // the caller has split this segment already
          ga.B[s] = (const float*)d.Bhi[s];
          ga.Blo[s] = lo ? d.Blo[s] : nullptr;
          continue;
        }
        rc = zr_split_pack_x_launch(ctx, d.B[s], d.K[s], d.N, d.ldb[s], hi, lo ? hi + e : nullptr);
        if (rc) return rc;
        ga.B[s] = (const float*)hi;
        ga.Blo[s] = lo ? hi + e : nullptr;
        hi += 2 * e;
      }
    }
    if (d.nseg == 1 && d.M >= 8192 && d.N > 32 && d.N <= 1024 &&
        (d.epilogue == ZR_EPI_STORE || d.epilogue == ZR_EPI_SOFTMAX_PARTIAL)) {
      const int n32 = (d.N + 31) / 32;
      const int n_tiles = (n32 + 3) / 4;
      const int tn = (n32 + n_tiles - 1) / n_tiles;
      // logits at 256 or 128 columns: activations through LDS, every weight element fetched by one wave
      if (d.epilogue == ZR_EPI_SOFTMAX_PARTIAL && ctx->gemm_cfg == 0 && (d.N == 256 || d.N == 128) && d.K[0] >= 64 &&
          (long long)(d.K[0] / 8 + 32) * d.lda[0] * 16 < (1LL << 32)) {
        if (one_term) return d.N == 256 ? launch_bf16_lds<8, false>(ctx, ga) : launch_bf16_lds<4, false>(ctx, ga);
        return d.N == 256 ? launch_bf16_lds<8, true>(ctx, ga) : launch_bf16_lds<4, true>(ctx, ga);
      }
      if (one_term) {
        if (tn <= 2) return launch_rows<2, ZR_A_PACK8_BF16_1T>(ctx, ga, d.epilogue, n_tiles);
        if (tn == 3) return launch_rows<3, ZR_A_PACK8_BF16_1T>(ctx, ga, d.epilogue, n_tiles);
        return launch_rows<4, ZR_A_PACK8_BF16_1T>(ctx, ga, d.epilogue, n_tiles);
      }
      if (tn <= 2) return launch_rows<2, ZR_A_PACK8_BF16>(ctx, ga, d.epilogue, n_tiles);
      if (tn == 3) return launch_rows<3, ZR_A_PACK8_BF16>(ctx, ga, d.epilogue, n_tiles);
      return launch_rows<4, ZR_A_PACK8_BF16>(ctx, ga, d.epilogue, n_tiles);
    }
    // 64 x 32 tiles for a narrow batch, and where 64 x 64 tiles would leave more than a third of the chip idle (the
    // attention output product at 2000 x 256: 128 tiles of 64 x 64 against 256 of 64 x 32)
    const long long wide_tiles = (long long)((ga.M + 63) / 64) * ((ga.N + 63) / 64) * d.batch;
    const int cus = ctx->cu_count > 0 ? ctx->cu_count : 256;
    if (d.N <= 32 || wide_tiles * 3 <= 2LL * cus) {
      ga.m_tiles = (ga.M + 63) / 64;
      ga.n_tiles = (ga.N + 31) / 32;
      if (one_term) return launch_epi<2, 1, 4, 1, ZR_A_PACK8_BF16_1T, true, 2>(ctx, ga, d.batch, d.epilogue);
      return launch_epi<2, 1, 4, 1, ZR_A_PACK8_BF16, true, 2>(ctx, ga, d.batch, d.epilogue);
    }
    ga.m_tiles = (ga.M + 63) / 64;
    ga.n_tiles = (ga.N + 63) / 64;
    if (one_term) return launch_epi<2, 2, 4, 1, ZR_A_PACK8_BF16_1T, true, 2>(ctx, ga, d.batch, d.epilogue);
    return launch_epi<2, 2, 4, 1, ZR_A_PACK8_BF16, true, 2>(ctx, ga, d.batch, d.epilogue);
  }
  if (d.a_pack) {
    // Activations too: a k-interleaved copy in scratch turns their loads (16 bytes from each of 32 lines per
    // half-wave) into contiguous ones.  Worth a small extra kernel once the weight matrix is large.
    if (d.b_packed) {
      ZR_CHECK_ARG(d.a_pack == 1 && vec, "gemm: a k-interleaved B needs a k-interleaved fp32 A and 16-byte alignment");
      for (int s = 0; s < d.nseg; ++s)
        ZR_CHECK_ARG(d.K[s] % 8 == 0, "gemm: a k-interleaved B needs K %% 8 == 0 (K[%d] = %d)", s, d.K[s]);
      ga.b_pack4 = 1;
    }
    bool xpack = vec && d.M >= 2048 && d.groups == 0 && !d.b_packed;
    size_t xfloats = 0;
    for (int s = 0; s < d.nseg; ++s) {
      xpack = xpack && (d.K[s] % 8 == 0);
      xfloats += (size_t)d.K[s] * d.N;
    }
    if (xpack) {
      void* p = nullptr;
      int rc = zr_ctx_scratch(ctx, 0, sizeof(float) * xfloats, &p);
      if (rc) return rc;
      float* xp = (float*)p;
      for (int s = 0; s < d.nseg; ++s) {
        const int f4 = (d.K[s] / 4) * d.N;
        pack4_x_kernel<<<(f4 + 255) / 256, 256, 0, ctx->stream>>>(d.B[s], d.K[s], d.N, d.ldb[s], xp);
        ZR_LAUNCH_CHECK("pack4_x_kernel");
        ga.B[s] = xp;
        xp += (size_t)d.K[s] * d.N;
      }
      ga.b_pack4 = 1;
    }
    // tall matrices: equal row ranges per CU, column tiles of equal width (at most 128 columns each)
    if (vec && d.nseg == 1 && zcount == 1 && d.M >= 8192 && d.N <= 1024 && ctx->gemm_cfg != 11 &&
        (d.epilogue == ZR_EPI_STORE || d.epilogue == ZR_EPI_SOFTMAX_PARTIAL)) {
      const int n32 = (d.N + 31) / 32;
      if ((d.N % 64 == 0 || d.N % 96 == 0) && ga.b_pack4 && ctx->gemm_cfg == 0) {
        int rc = ZR_OK;
        if (launch_tall(ctx, ga, d.epilogue, &rc)) return rc;
      }
      if (d.N <= 32 && ga.b_pack4 && d.K[0] % 8 == 0 && ctx->gemm_cfg == 0 &&
          (long long)d.K[0] * ga.lda[0] * 4 + 4096 < (1LL << 32)) {
        // one 32-row block per wave while there are waves (three workgroups per compute unit), more beyond that
        // two neighbouring 32-row blocks per wave (their fetches are 1 KB of contiguous memory), two workgroups per
        // compute unit, one pair per wave while there are waves
        const int pairs = ((d.M + 31) / 32 + 1) / 2;
        const int cus = ctx->cu_count > 0 ? ctx->cu_count : 256;
        int wgs = (pairs + 3) / 4;
        if (wgs > 2 * cus) wgs = 2 * cus;
        ga.m_tiles = ga.n_tiles = 0;
        if (d.epilogue == ZR_EPI_STORE)
          gemm_stream_kernel<ZR_EPI_STORE, 0><<<wgs, 256, 0, ctx->stream>>>(ga);
        else if (ga.stream_a)
          gemm_stream_kernel<ZR_EPI_SOFTMAX_PARTIAL, ZR_AUX_STREAM><<<wgs, 256, 0, ctx->stream>>>(ga);
        else
          gemm_stream_kernel<ZR_EPI_SOFTMAX_PARTIAL, 0><<<wgs, 256, 0, ctx->stream>>>(ga);
        ZR_LAUNCH_CHECK("gemm_stream_kernel");
        return ZR_OK;
      }
      const int n_tiles = (n32 + 3) / 4;
      const int tn = (n32 + n_tiles - 1) / n_tiles;
      if (tn == 1) return launch_rows<1>(ctx, ga, d.epilogue, n_tiles);
      if (tn <= 2) return launch_rows<2>(ctx, ga, d.epilogue, n_tiles);
      if (tn == 3) return launch_rows<3>(ctx, ga, d.epilogue, n_tiles);
      return launch_rows<4>(ctx, ga, d.epilogue, n_tiles);
    }
    // Small outputs (the attention projections: about a thousand rows by a minibatch of columns): 32 x 32 tiles with K
    // split over the eight waves of a workgroup, so that a few hundred workgroups share the chip and each wave's chain
    // of dependent matrix instructions is short.
    {
      const long long t32 = (long long)((d.M + 31) / 32) * ((d.N + 31) / 32) * zcount;
      long long ktot = 0;
      for (int s = 0; s < d.nseg; ++s) ktot += d.K[s];
      if (ctx->gemm_cfg == 0 && d.groups == 0 && t32 <= 768 && ktot >= 512) {
        ga.m_tiles = (ga.M + 31) / 32;
        ga.n_tiles = (ga.N + 31) / 32;
        if (vec) return launch_epi<1, 1, 8, 1, ZR_A_PACK4, true, 1>(ctx, ga, zcount, d.epilogue);
        return launch_epi<1, 1, 8, 1, ZR_A_PACK4, false, 1>(ctx, ga, zcount, d.epilogue);
      }
    }
    if (ctx->gemm_cfg == 12) return launch_pack4<4, 2, 1>(ctx, ga, d.epilogue, vec, zcount);
    if (ctx->gemm_cfg == 13) return launch_pack4<2, 2, 1>(ctx, ga, d.epilogue, vec, zcount);
    if (ctx->gemm_cfg == 14) return launch_pack4<2, 4, 1>(ctx, ga, d.epilogue, vec, zcount);
    if (d.N <= 32) return launch_pack4<2, 1, 2>(ctx, ga, d.epilogue, vec, zcount);
    return launch_pack4<2, 2, 2>(ctx, ga, d.epilogue, vec, zcount);
  }
  // Large, untransposed, single-segment products with a wide batch (the softmax logits): LDS-shared weights.
  const bool lds_ok = !d.trans_a && d.nseg == 1 && zcount == 1 && vec && (d.M % 4 == 0) && (d.lda[0] % 4 == 0) &&
                      (((uintptr_t)d.A[0] & 15u) == 0) && d.K[0] >= 8 && d.K[0] % 8 == 0 && d.M >= 2048 && d.N >= 96 &&
                      ((long long)d.K[0] + 64) * d.lda[0] * 4 < (1LL << 32) && (long long)d.N * d.ldb[0] * 4 < (1LL << 32) &&
                      (d.epilogue == ZR_EPI_STORE || d.epilogue == ZR_EPI_SOFTMAX_PARTIAL);
  if (lds_ok && ctx->gemm_cfg == 10) return launch_lds<4, 4>(ctx, ga, d.epilogue);
  if (lds_ok && (ctx->gemm_cfg == 0 || ctx->gemm_cfg == 9)) {
    if (d.N <= 128 || d.N > 256) return launch_lds_rows<4>(ctx, ga, d.epilogue);
    if (d.N <= 192) return launch_lds_rows<6>(ctx, ga, d.epilogue);
    return launch_lds_rows<8>(ctx, ga, d.epilogue);
  }
  // Tile choice.  The chip has 1024 SIMDs; a wave tile is 32*TM x 32*TN outputs.  Prefer the largest tile that
  // still yields about two waves per SIMD, and split K inside the workgroup when the output is too small to
  // fill the chip otherwise.
  const bool trans_a = d.trans_a != 0;
  int cfg = ctx->gemm_cfg;
  if (cfg == 0) {
    const long long sub32 = (long long)((d.M + 31) / 32) * ((d.N + 31) / 32) * zcount;  // 32x32 output blocks
    if (sub32 >= 8 * 2048)
      cfg = 1;  // 64 x 128 wave tiles
    else if (sub32 >= 4 * 2048)
      cfg = 2;  // 32 x 128
    else if (sub32 >= 2 * 1024)
      cfg = 3;  // 32 x 64
    else if (sub32 >= 1024)
      cfg = 4;  // 32 x 32
    else if (sub32 <= 256 && d.K[0] >= 512)
      cfg = 6;  // 32 x 32, K split over 8 waves: at most one tile per CU, the K loop is all there is to shorten
    else
      cfg = 5;  // 32 x 32, K split over 4 waves
    if (d.N <= 32 && cfg < 4) cfg = 4;
    else if (d.N <= 64 && cfg < 3) cfg = 3;
  }
  (void)flops;
  switch (cfg) {
    case 1:
      return launch_cfg<2, 4, 1, 4>(ctx, ga, zcount, d.epilogue, trans_a, vec);
    case 2:
      return launch_cfg<1, 4, 1, 4>(ctx, ga, zcount, d.epilogue, trans_a, vec);
    case 3:
      return launch_cfg<1, 2, 1, 4>(ctx, ga, zcount, d.epilogue, trans_a, vec);
    case 4:
      return launch_cfg<1, 1, 1, 4>(ctx, ga, zcount, d.epilogue, trans_a, vec);
    case 5:
      return launch_cfg<1, 1, 4, 1>(ctx, ga, zcount, d.epilogue, trans_a, vec);
    case 6:
      return launch_cfg<1, 1, 8, 1>(ctx, ga, zcount, d.epilogue, trans_a, vec);
    case 7:
      return launch_cfg<2, 2, 1, 4>(ctx, ga, zcount, d.epilogue, trans_a, vec);
    default:
      return launch_cfg<1, 2, 4, 1>(ctx, ga, zcount, d.epilogue, trans_a, vec);
  }
}

extern "C" int zr_gemm(zr_ctx* ctx, int trans_a, int M, int N, int K, const float* d_A, int lda, const float* d_B,
                       int ldb, float* d_C, int ldc) {
  int rc = zr_bind_device(ctx);
  if (rc) return rc;
  ZrGemmDesc d = {};
  d.M = M;
  d.N = N;
  d.nseg = 1;
  d.K[0] = K;
  d.A[0] = d_A;
  d.lda[0] = lda;
  d.trans_a = trans_a;
  d.B[0] = d_B;
  d.ldb[0] = ldb;
  d.C = d_C;
  d.ldc = ldc;
  d.batch = 1;
  d.epilogue = ZR_EPI_STORE;
  return zr_gemm_launch(ctx, d);
}
