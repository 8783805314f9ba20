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
  int m_tiles, n_tiles;  // wave tiles along M and N
};

// Workgroup = 64*KS*WPB threads: WPB independent wave tiles, each shared by KS waves that split K.
template <int TM, int TN, int KS, int WPB, bool TRANS_A, bool VEC, int EPI>
__global__ void __launch_bounds__(64 * KS * WPB) gemm_kernel(GemmArgs a) {
  __shared__ float red[KS > 1 ? WPB * KS * TN * 16 * 64 : 1];
  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);  // wave-uniform by construction
  const int kslice = wave % KS;
  const int sub = wave / KS;  // which wave tile of the workgroup
  const int jl = lane & 31;
  const int half = lane >> 5;
  const int z = blockIdx.z;

  // wave tile id -> (mt, nt), m fastest so that neighbouring waves stream neighbouring weight rows
  long long tile = (long long)blockIdx.x * WPB + sub;
  const long long ntiles = (long long)a.m_tiles * a.n_tiles;
  const bool active = tile < ntiles;
  if (!active) tile = ntiles - 1;  // keep the wave in step with the workgroup barriers; results discarded
  const int mt = (int)(tile % a.m_tiles);
  const int nt = (int)(tile / a.m_tiles);
  const int m0 = mt * 32 * TM;
  const int n0 = nt * 32 * TN;

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

  for (int s = 0; s < a.nseg; ++s) {
    const float* A = a.A[s] + (long long)z * a.strideA;
    const float* wbase[TM];
    unsigned woff[TM];
    const float* xcol[TN];
#pragma unroll
    for (int tm = 0; tm < TM; ++tm) {
      wbase[tm] = A;
      woff[tm] = TRANS_A ? (unsigned)((long long)rows[tm] * a.lda[s] + 4 * half)
                         : (unsigned)(rows[tm] + 4LL * half * a.lda[s]);
    }
#pragma unroll
    for (int tn = 0; tn < TN; ++tn) xcol[tn] = a.B[s] + (long long)cols[tn] * a.ldb[s] + 4 * half;
    zr_mma_segment<TM, TN, KS, zr_prefetch_depth(TM, TN), TRANS_A ? ZR_A_TRANS : ZR_A_NN, VEC>(acc, wbase, woff, a.lda[s], xcol, a.K[s],
                                                                        kslice, half);
  }

  float* C = a.C + (long long)z * a.strideC;
  const float* bias = a.bias ? a.bias + (long long)z * a.strideBias : nullptr;
  float* redp = KS > 1 ? red + (size_t)sub * KS * TN * 16 * 64 : red;

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
          C[(long long)n * a.ldc + m] = v;
        }
      } else if (EPI == ZR_EPI_TANH) {
        if (ok) C[(long long)n * a.ldc + m] = tanhf(v);
      } else if (EPI == ZR_EPI_TANH_BIAS_MASK) {
        if (ok) C[(long long)n * a.ldc + m] = tanhf(v + bias[m]) * (float)a.mask[n];
      } else {  // ZR_EPI_SOFTMAX_PARTIAL
        if (ok) {
          v += bias[m];
          C[(long long)n * a.ldc + m] = v;
        }
        // (max, sum exp) over the 32 rows of this sub-tile for column n: reduce across the 32 lanes of a half
        float mx = ok ? v : -INFINITY;
#pragma unroll
        for (int off = 16; off > 0; off >>= 1) mx = fmaxf(mx, __shfl_xor(mx, off, 64));
        float e = ok ? expf(v - mx) : 0.0f;
#pragma unroll
        for (int off = 16; off > 0; off >>= 1) e += __shfl_xor(e, off, 64);
        const int prow = (m0 >> 5) + tm;  // 32-row block index
        if (jl == 0 && n_ok && prow * 32 < a.M) {
          float* p = a.partials + ((long long)prow * a.N + n) * 2;
          p[0] = mx;
          p[1] = e;
        }
      }
    }
  });
}


// ---------------------------------------------------------------------------------------------------------
// Large-M variant: weight rows staged through LDS and shared by all waves of the workgroup.
//
// A workgroup owns 32*TMR rows x 32*NWV columns; wave w owns columns [32w, 32w+32) and all TMR row sub-tiles, so
// every weight chunk (32 k x 32*TMR rows) is read from L2 once per workgroup with 16-byte coalesced loads,
// parked in LDS (double buffered, one barrier per chunk) and multiplied by every wave, while each wave fetches
// only its own 32 activation columns.  Against one 32x32 tile per wave this cuts the bytes pulled through the
// CU's L1 per flop by about TMR, which is what limited the softmax-logits GEMM (V x H times H x mb).
// Loads are unconditional with clamped addresses (see zr_mfma_core.h on why); out-of-range weights are zeroed
// by multiplication.  Requires: no transpose, one K segment, M, lda, ldb multiples of 4, 16-byte aligned bases.
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
  const float* xcol = a.B[0] + (long long)col * a.ldb[0];

  const float* wsrc[WLD];
  float wkeep[WLD];
  int wkk[WLD];
#pragma unroll
  for (int u = 0; u < WLD; ++u) {
    const int f = tid + NTHR * u;
    const int fc = f < F4 ? f : F4 - 1;
    const int j4 = fc & 7, tm = (fc >> 3) % TMR, kk = fc / (8 * TMR);
    const int row = m0 + 32 * tm + 4 * j4;
    wkeep[u] = (row < M && f < F4) ? 1.0f : 0.0f;
    wkk[u] = kk;
    wsrc[u] = A + (row < M ? row : M - 4);
  }

  zr_f32x16 acc[TMR];
#pragma unroll
  for (int tm = 0; tm < TMR; ++tm)
#pragma unroll
    for (int r = 0; r < 16; ++r) acc[tm][r] = 0.0f;

  zr_f32x4 wreg[WLD];
  zr_f32x4 xf[2][4];
  // gload only issues loads (raw values stay in registers while the current chunk is multiplied); the zeroing of
  // out-of-range weights happens in lds_store, so that no instruction consumes a loaded value right after its
  // load and several loads stay in flight.
  auto gload = [&](int c, zr_f32x4 (&xdst)[4]) {
    const int cc = c < n_chunks ? c : n_chunks - 1;
#pragma unroll
    for (int u = 0; u < WLD; ++u) {
      const int k = cc * KC + wkk[u];
      const int kc = k < K ? k : K - 1;
      wreg[u] = *(const zr_f32x4*)(wsrc[u] + (long long)kc * lda);
    }
#pragma unroll
    for (int gq = 0; gq < 4; ++gq) {
      int kx = cc * KC + 8 * gq + 4 * half;
      kx = (kx + 4 <= K) ? kx : K - 4;
      xdst[gq] = *(const zr_f32x4*)(xcol + kx);
    }
  };
  auto lds_store = [&](int buf, int c) {
    const float chunk_keep = c < n_chunks ? 1.0f : 0.0f;  // dummy chunk of an odd chunk count: all zeros
    const int cc = c < n_chunks ? c : n_chunks - 1;
#pragma unroll
    for (int u = 0; u < WLD; ++u) {
      const int f = tid + NTHR * u;
      const float keep = ((cc * KC + wkk[u]) < K ? wkeep[u] : 0.0f) * chunk_keep;
      zr_f32x4 v = wreg[u];
      v.x *= keep;
      v.y *= keep;
      v.z *= keep;
      v.w *= keep;
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
      __builtin_amdgcn_sched_barrier(0);  // keep the LDS reads ahead of the MFMAs that consume them
#pragma unroll
      for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int tm = 0; tm < TMR; ++tm)
          acc[tm] = __builtin_amdgcn_mfma_f32_32x32x2f32(xs[gq][i], wf[gq & 1][i][tm], acc[tm], 0, 0, 0);
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

#pragma unroll
  for (int r = 0; r < 16; ++r) {
    const int n = n0 + 8 * (r >> 2) + 4 * half + (r & 3);
    const bool n_ok = n < a.N;
#pragma unroll
    for (int tm = 0; tm < TMR; ++tm) {
      const int m = m0 + tm * 32 + jl;
      const bool ok = n_ok && m < M;
      float v = acc[tm][r];
      if (EPI == ZR_EPI_STORE) {
        if (ok) {
          if (a.bias) v += a.bias[m];
          a.C[(long long)n * a.ldc + m] = v;
        }
      } else {  // ZR_EPI_SOFTMAX_PARTIAL
        if (ok) {
          v += a.bias[m];
          a.C[(long long)n * a.ldc + m] = v;
        }
        float mx = ok ? v : -INFINITY;
#pragma unroll
        for (int off = 16; off > 0; off >>= 1) mx = fmaxf(mx, __shfl_xor(mx, off, 64));
        float e = ok ? expf(v - mx) : 0.0f;
#pragma unroll
        for (int off = 16; off > 0; off >>= 1) e += __shfl_xor(e, off, 64);
        const int prow = (m0 >> 5) + tm;
        if (jl == 0 && n_ok && prow * 32 < M) {
          float* p = a.partials + ((long long)prow * a.N + n) * 2;
          p[0] = mx;
          p[1] = e;
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

template <int TM, int TN, int KS, int WPB, bool TRANS_A, bool VEC>
int launch_epi(zr_ctx* ctx, const GemmArgs& ga, int batch, int epi) {
  const long long ntiles = (long long)ga.m_tiles * ga.n_tiles;
  dim3 grid((unsigned)((ntiles + WPB - 1) / WPB), 1, batch);
  dim3 block(64 * KS * WPB);
  switch (epi) {
    case ZR_EPI_STORE:
      gemm_kernel<TM, TN, KS, WPB, TRANS_A, VEC, ZR_EPI_STORE><<<grid, block, 0, ctx->stream>>>(ga);
      break;
    case ZR_EPI_TANH:
      gemm_kernel<TM, TN, KS, WPB, TRANS_A, VEC, ZR_EPI_TANH><<<grid, block, 0, ctx->stream>>>(ga);
      break;
    case ZR_EPI_TANH_BIAS_MASK:
      gemm_kernel<TM, TN, KS, WPB, TRANS_A, VEC, ZR_EPI_TANH_BIAS_MASK><<<grid, block, 0, ctx->stream>>>(ga);
      break;
    default:
      gemm_kernel<TM, TN, KS, WPB, TRANS_A, VEC, ZR_EPI_SOFTMAX_PARTIAL><<<grid, block, 0, ctx->stream>>>(ga);
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
    if (vec) return launch_epi<TM, TN, KS, WPB, true, true>(ctx, ga, batch, epi);
    return launch_epi<TM, TN, KS, WPB, true, false>(ctx, ga, batch, epi);
  }
  if (vec) return launch_epi<TM, TN, KS, WPB, false, true>(ctx, ga, batch, epi);
  return launch_epi<TM, TN, KS, WPB, false, false>(ctx, ga, batch, epi);
}

}  // namespace

int zr_gemm_launch(zr_ctx* ctx, const ZrGemmDesc& d) {
  ZR_CHECK_ARG(d.M > 0 && d.N > 0, "gemm: M = %d, N = %d", d.M, d.N);
  ZR_CHECK_ARG(d.nseg >= 1 && d.nseg <= 3, "gemm: nseg = %d", d.nseg);
  ZR_CHECK_ARG(d.C != nullptr && d.ldc >= d.M, "gemm: C null or ldc %d < M %d", d.ldc, d.M);
  ZR_CHECK_ARG(d.batch >= 1 && d.batch <= 65535, "gemm: batch = %d", d.batch);
  GemmArgs ga;
  ga.M = d.M;
  ga.N = d.N;
  ga.nseg = d.nseg;
  bool vec = true;
  long long flops = 0;
  for (int s = 0; s < 3; ++s) {
    if (s < d.nseg) {
      ZR_CHECK_ARG(d.K[s] > 0, "gemm: K[%d] = %d", s, d.K[s]);
      ZR_CHECK_ARG(d.A[s] && d.B[s], "gemm: null operand in segment %d", s);
      ZR_CHECK_ARG(d.lda[s] >= (d.trans_a ? d.K[s] : d.M), "gemm: lda[%d] = %d too small", s, d.lda[s]);
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
      if (d.trans_a) vec = vec && (d.lda[s] % 4 == 0) && (((uintptr_t)d.A[s] & 15u) == 0) && (d.strideA % 4 == 0);
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
  if (d.epilogue == ZR_EPI_TANH_BIAS_MASK) ZR_CHECK_ARG(d.bias && d.mask, "gemm: bias/mask required");
  if (d.epilogue == ZR_EPI_SOFTMAX_PARTIAL) ZR_CHECK_ARG(d.bias && d.partials, "gemm: bias/partials required");

  // Large, untransposed, single-segment products with a wide batch (the softmax logits): LDS-shared weights.
  const bool lds_ok = !d.trans_a && d.nseg == 1 && d.batch == 1 && vec && (d.M % 4 == 0) && (d.lda[0] % 4 == 0) &&
                      (((uintptr_t)d.A[0] & 15u) == 0) && d.K[0] >= 8 && d.M >= 4096 && d.N >= 96 &&
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
    const long long sub32 = (long long)((d.M + 31) / 32) * ((d.N + 31) / 32) * d.batch;  // 32x32 output blocks
    if (sub32 >= 8 * 2048)
      cfg = 1;  // 64 x 128 wave tiles
    else if (sub32 >= 4 * 2048)
      cfg = 2;  // 32 x 128
    else if (sub32 >= 2 * 1024)
      cfg = 3;  // 32 x 64
    else if (sub32 >= 1024)
      cfg = 4;  // 32 x 32
    else
      cfg = 5;  // 32 x 32, K split over 4 waves
    if (d.N <= 32 && cfg < 4) cfg = 4;
    else if (d.N <= 64 && cfg < 3) cfg = 3;
  }
  (void)flops;
  switch (cfg) {
    case 1:
      return launch_cfg<2, 4, 1, 4>(ctx, ga, d.batch, d.epilogue, trans_a, vec);
    case 2:
      return launch_cfg<1, 4, 1, 4>(ctx, ga, d.batch, d.epilogue, trans_a, vec);
    case 3:
      return launch_cfg<1, 2, 1, 4>(ctx, ga, d.batch, d.epilogue, trans_a, vec);
    case 4:
      return launch_cfg<1, 1, 1, 4>(ctx, ga, d.batch, d.epilogue, trans_a, vec);
    case 5:
      return launch_cfg<1, 1, 4, 1>(ctx, ga, d.batch, d.epilogue, trans_a, vec);
    case 6:
      return launch_cfg<1, 1, 8, 1>(ctx, ga, d.batch, d.epilogue, trans_a, vec);
    case 7:
      return launch_cfg<2, 2, 1, 4>(ctx, ga, d.batch, d.epilogue, trans_a, vec);
    default:
      return launch_cfg<1, 2, 4, 1>(ctx, ga, d.batch, d.epilogue, trans_a, vec);
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
