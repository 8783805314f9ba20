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
    zr_mma_segment<TM, TN, KS, zr_prefetch_depth(TM, TN), TRANS_A, VEC>(acc, wbase, woff, a.lda[s], xcol, a.K[s],
                                                                        kslice, half);
  }

  float* C = a.C + (long long)z * a.strideC;
  const float* bias = a.bias ? a.bias + (long long)z * a.strideBias : nullptr;
  float* redp = KS > 1 ? red + (size_t)sub * KS * TN * 16 * 64 : red;

  zr_reduce_visit<TM, TN, KS>(acc, redp, kslice, lane, [&](const float(&vals)[TM], int tn, int r) {
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
