// LSTM node forward on MFMA with the gate / cell maths fused into the GEMM epilogue.
//
// One launch covers a set of independent (layer, time-step) units.  For each unit it computes, for every hidden
// row j and batch column n,
//     z_g[j,n] = sum_k M_g[j,k] in[k,n] + sum_k Wh_g[j,k] h_prev[k,n] (+ sum_k Q_g[j,k] h~[k,n]),  g = i,f,c,o
// and immediately turns the four z_g of a (j,n) pair -- which land in the same accumulator register of the
// same lane because each wave owns the four gate sub-tiles of its 32 rows -- into c_t and h_t.  The
// pre-activations never touch memory.
//
// Work decomposition: a workgroup owns 32 hidden rows x 32*TN batch columns (all four gates) and its KS waves
// split K; weights stream from HBM/L2 straight into MFMA operand registers (full 128-byte lines), the
// activations are fetched with 16-byte loads along K.  See zr_mfma_core.h.
#include "zr_internal.h"
#include "zr_math.h"
#include "zr_mfma_core.h"

namespace {

constexpr int kMaxUnits = 8;

struct LstmUnit {
  const float* W;           // [nseg][4][H*H]
  const float* bias;        // [4][H]
  const float* in[3];       // segment inputs, H x mb (ld = H)
  const int* gather_ids;    // non-null: column n of segment 0 is in[0] + ids[n]*H (embedding gather)
  const float* cprev;
  const int* mask01;
  float* h;
  float* c;
  float* gates[4];          // all null or all non-null
  int nseg;
  int V;                    // rows of the gather source (ids are clamped to [0,V))
};

struct LstmLaunch {
  LstmUnit u[kMaxUnits];
  int n_units;
  int H, mb;
  float clip;
  int j_tiles, n_tiles;
};

template <int TN, int KS, bool VEC>
__global__ void __launch_bounds__(64 * KS) lstm_fused_kernel(LstmLaunch L) {
  __shared__ float red[KS * TN * 16 * 64];
  // Workgroups that share a weight tile (same unit and row tile, different column tile) get ids that are
  // congruent modulo 8, so the round-robin workgroup->XCD dispatch puts them on the same XCD and its L2.
  const int id = blockIdx.x;
  const int r8 = id & 7;
  const int q = id >> 3;
  const int nt = q % L.n_tiles;
  const int group = (q / L.n_tiles) * 8 + r8;
  if (group >= L.n_units * L.j_tiles) return;
  const int unit = group / L.j_tiles;
  const int jt = group % L.j_tiles;
  const LstmUnit& U = L.u[unit];

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int kslice = __builtin_amdgcn_readfirstlane(tid >> 6);  // wave-uniform by construction
  const int jl = lane & 31;
  const int half = lane >> 5;
  const int H = L.H;
  const int j0 = jt * 32;
  const int n0 = nt * 32 * TN;
  const int j = j0 + jl;
  const int jc = j < H ? j : H - 1;

  int cols[TN];
#pragma unroll
  for (int tn = 0; tn < TN; ++tn) {
    const int c = n0 + tn * 32 + jl;
    cols[tn] = c < L.mb ? c : L.mb - 1;
  }

  zr_f32x16 acc[4][TN];
#pragma unroll
  for (int g = 0; g < 4; ++g)
#pragma unroll
    for (int tn = 0; tn < TN; ++tn)
#pragma unroll
      for (int r = 0; r < 16; ++r) acc[g][tn][r] = 0.0f;

  const long long HH = (long long)H * H;
  for (int s = 0; s < U.nseg; ++s) {
    const float* wbase[4];
    unsigned woff[4];
    const float* xcol[TN];
#pragma unroll
    for (int g = 0; g < 4; ++g) {
      wbase[g] = U.W + ((long long)s * 4 + g) * HH;
      woff[g] = (unsigned)(jc + 4 * half * H);
    }
#pragma unroll
    for (int tn = 0; tn < TN; ++tn) {
      long long c = cols[tn];
      if (s == 0 && U.gather_ids) {
        int idv = U.gather_ids[cols[tn]];
        idv = idv < 0 ? 0 : (idv >= U.V ? U.V - 1 : idv);
        c = idv;
      }
      xcol[tn] = U.in[s] + c * H + 4 * half;
    }
    zr_mma_segment<4, TN, KS, zr_prefetch_depth(4, TN), false, VEC>(acc, wbase, woff, (long long)H, xcol, H, kslice,
                                                                    half);
  }

  const float bi = U.bias[jc], bf = U.bias[H + jc], bc = U.bias[2 * H + jc], bo = U.bias[3 * H + jc];
  const bool j_ok = j < H;
  zr_reduce_visit<4, TN, KS>(acc, red, kslice, lane, [&](const float(&z)[4], int tn, int r) {
    const int n = n0 + tn * 32 + 8 * (r >> 2) + 4 * half + (r & 3);
    if (j_ok && n < L.mb) {
      const long long ix = (long long)n * H + j;
      float gi, gf, gc, go, c, h;
      zr_lstm_cell(z[0] + bi, z[1] + bf, z[2] + bc, z[3] + bo, U.cprev[ix], (float)U.mask01[n], L.clip, gi, gf, gc,
                   go, c, h);
      U.c[ix] = c;
      U.h[ix] = h;
      if (U.gates[0]) {
        U.gates[0][ix] = gi;
        U.gates[1][ix] = gf;
        U.gates[2][ix] = gc;
        U.gates[3][ix] = go;
      }
    }
  });
}

template <int TN, int KS>
int launch_fused_v(zr_ctx* ctx, const LstmLaunch& L, bool vec) {
  const int groups = L.n_units * L.j_tiles;
  const int grid = ((groups + 7) / 8) * 8 * L.n_tiles;
  if (vec)
    lstm_fused_kernel<TN, KS, true><<<grid, 64 * KS, 0, ctx->stream>>>(L);
  else
    lstm_fused_kernel<TN, KS, false><<<grid, 64 * KS, 0, ctx->stream>>>(L);
  ZR_LAUNCH_CHECK("lstm_fused_kernel");
  return ZR_OK;
}

int launch_fused(zr_ctx* ctx, LstmLaunch& L, bool vec) {
  L.j_tiles = (L.H + 31) / 32;
  const int n32 = (L.mb + 31) / 32;
  int tn = ctx->lstm_tn;
  if (tn == 0) {
    // largest column tile that still yields at least one workgroup per CU
    tn = 1;
    const int groups = L.n_units * L.j_tiles;
    if (n32 >= 2 && (long long)groups * ((n32 + 1) / 2) >= 256) tn = 2;
  }
  if (tn > n32) tn = n32 >= 2 ? 2 : 1;
  if (tn == 4 && n32 < 4) tn = 2;
  L.n_tiles = (n32 + tn - 1) / tn;
  int ks = ctx->lstm_ksplit;
  if (ks == 0) {
    const long long wgs = (long long)L.n_units * L.j_tiles * L.n_tiles;
    ks = wgs < 192 ? 8 : 4;
  }
  if (tn == 1) return ks == 8 ? launch_fused_v<1, 8>(ctx, L, vec) : launch_fused_v<1, 4>(ctx, L, vec);
  if (tn == 2) return ks == 8 ? launch_fused_v<2, 8>(ctx, L, vec) : launch_fused_v<2, 4>(ctx, L, vec);
  return launch_fused_v<4, 4>(ctx, L, vec);
}

inline bool aligned16(const void* p) { return ((uintptr_t)p & 15u) == 0; }

}  // namespace

extern "C" {

int zr_lstm_pack_weights(zr_ctx* ctx, const float* const d_M[4], const float* const d_Wh[4],
                         const float* const d_Q[4], const float* const d_b[4], int H, zr_lstm_weights** out) {
  int rc = zr_bind_device(ctx);
  if (rc) return rc;
  ZR_CHECK_ARG(out != nullptr, "zr_lstm_pack_weights: out is null");
  *out = nullptr;
  ZR_CHECK_ARG(H > 0, "zr_lstm_pack_weights: H = %d", H);
  ZR_CHECK_ARG(d_M && d_Wh && d_b, "zr_lstm_pack_weights: null pointer array");
  for (int g = 0; g < 4; ++g) {
    ZR_CHECK_ARG(d_M[g] && d_Wh[g] && d_b[g], "zr_lstm_pack_weights: null matrix for gate %d", g);
    ZR_CHECK_ARG(!d_Q || d_Q[g], "zr_lstm_pack_weights: null Q for gate %d", g);
  }
  const int nseg = d_Q ? 3 : 2;
  const size_t HH = (size_t)H * H;
  zr_lstm_weights* w = new zr_lstm_weights();
  w->H = H;
  w->nseg = nseg;
  w->d_W = nullptr;
  w->d_bias = nullptr;
  if (hipMalloc((void**)&w->d_W, sizeof(float) * HH * 4 * nseg) != hipSuccess ||
      hipMalloc((void**)&w->d_bias, sizeof(float) * 4 * (size_t)H) != hipSuccess) {
    (void)hipGetLastError();
    if (w->d_W) (void)hipFree(w->d_W);
    delete w;
    return zr_set_error(ZR_ENOMEM, "zr_lstm_pack_weights: allocation failed (H = %d, nseg = %d)", H, nseg);
  }
  for (int g = 0; g < 4; ++g) {
    const float* segs[3] = {d_M[g], d_Wh[g], d_Q ? d_Q[g] : nullptr};
    for (int s = 0; s < nseg; ++s) {
      hipError_t e = hipMemcpyAsync(w->d_W + ((size_t)s * 4 + g) * HH, segs[s], sizeof(float) * HH,
                                    hipMemcpyDeviceToDevice, ctx->stream);
      if (e != hipSuccess) {
        (void)hipFree(w->d_W);
        (void)hipFree(w->d_bias);
        delete w;
        return zr_set_error(ZR_EHIP, "zr_lstm_pack_weights: copy failed: %s", hipGetErrorString(e));
      }
    }
    hipError_t e = hipMemcpyAsync(w->d_bias + (size_t)g * H, d_b[g], sizeof(float) * H, hipMemcpyDeviceToDevice,
                                  ctx->stream);
    if (e != hipSuccess) {
      (void)hipFree(w->d_W);
      (void)hipFree(w->d_bias);
      delete w;
      return zr_set_error(ZR_EHIP, "zr_lstm_pack_weights: bias copy failed: %s", hipGetErrorString(e));
    }
  }
  *out = w;
  return ZR_OK;
}

int zr_lstm_weights_destroy(zr_ctx* ctx, zr_lstm_weights* w) {
  if (!w) return ZR_OK;
  int rc = zr_bind_device(ctx);
  if (rc) return rc;
  ZR_HIP(hipStreamSynchronize(ctx->stream));
  if (w->d_W) (void)hipFree(w->d_W);
  if (w->d_bias) (void)hipFree(w->d_bias);
  delete w;
  return ZR_OK;
}

int zr_lstm_step(zr_ctx* ctx, const zr_lstm_weights* w, const float* d_in, const float* d_hprev,
                 const float* d_cprev, const float* d_htild, const int* d_mask01, float clip_threshold, int mb,
                 float* d_h, float* d_c, float* const d_gates[4]) {
  int rc = zr_bind_device(ctx);
  if (rc) return rc;
  ZR_CHECK_ARG(w != nullptr, "zr_lstm_step: weights are null");
  ZR_CHECK_ARG(mb > 0, "zr_lstm_step: mb = %d", mb);
  ZR_CHECK_ARG(d_in && d_hprev && d_cprev && d_mask01 && d_h && d_c, "zr_lstm_step: null pointer");
  ZR_CHECK_ARG(!d_htild || w->nseg == 3, "zr_lstm_step: d_htild given but the weights were packed without Q");
  ZR_CHECK_ARG(d_h != d_hprev && d_h != d_in && d_h != d_htild, "zr_lstm_step: d_h must not alias an input");
  if (d_gates)
    for (int g = 0; g < 4; ++g) ZR_CHECK_ARG(d_gates[g] != nullptr, "zr_lstm_step: d_gates[%d] is null", g);
  const int H = w->H;
  const int nseg = d_htild ? 3 : 2;

  if (!ctx->lstm_fused) {
    // reference-shaped two-phase path: pre-activations to memory (batched over the 4 gates), then the
    // stand-alone fused gate kernel
    void* pre = nullptr;
    rc = zr_ctx_scratch(ctx, 0, sizeof(float) * 4 * (size_t)H * mb, &pre);
    if (rc) return rc;
    ZrGemmDesc d = {};
    d.M = H;
    d.N = mb;
    d.nseg = nseg;
    const float* ins[3] = {d_in, d_hprev, d_htild};
    for (int s = 0; s < nseg; ++s) {
      d.K[s] = H;
      d.A[s] = w->d_W + (size_t)s * 4 * H * H;
      d.lda[s] = H;
      d.B[s] = ins[s];
      d.ldb[s] = H;
    }
    d.C = (float*)pre;
    d.ldc = H;
    d.batch = 4;
    d.strideA = (long long)H * H;
    d.strideC = (long long)H * mb;
    d.epilogue = ZR_EPI_STORE;
    rc = zr_gemm_launch(ctx, d);
    if (rc) return rc;
    const float* b[4] = {w->d_bias, w->d_bias + H, w->d_bias + 2 * (size_t)H, w->d_bias + 3 * (size_t)H};
    return zr_lstm_gates(ctx, (const float*)pre, b, d_cprev, d_mask01, clip_threshold, H, mb, d_h, d_c, d_gates);
  }

  LstmLaunch L = {};
  L.n_units = 1;
  L.H = H;
  L.mb = mb;
  L.clip = clip_threshold;
  LstmUnit& U = L.u[0];
  U.W = w->d_W;
  U.bias = w->d_bias;
  U.in[0] = d_in;
  U.in[1] = d_hprev;
  U.in[2] = d_htild;
  U.gather_ids = nullptr;
  U.cprev = d_cprev;
  U.mask01 = d_mask01;
  U.h = d_h;
  U.c = d_c;
  for (int g = 0; g < 4; ++g) U.gates[g] = d_gates ? d_gates[g] : nullptr;
  U.nseg = nseg;
  U.V = 0;
  const bool vec = (H % 4 == 0) && aligned16(d_in) && aligned16(d_hprev) && (!d_htild || aligned16(d_htild));
  return launch_fused(ctx, L, vec);
}

int zr_lstm_stack_forward(zr_ctx* ctx, int nl, const zr_lstm_weights* const layers[], const float* d_embed, int V,
                          const int* d_ids_nonneg, const int* d_mask01, int T, int mb,
                          const float* const d_h0[], const float* const d_c0[], float clip_threshold,
                          float* const d_h_all[], float* const d_c_all[]) {
  int rc = zr_bind_device(ctx);
  if (rc) return rc;
  ZR_CHECK_ARG(nl > 0 && T > 0 && mb > 0 && V > 0, "zr_lstm_stack_forward: L = %d, T = %d, mb = %d, V = %d", nl, T,
               mb, V);
  ZR_CHECK_ARG(layers && d_embed && d_ids_nonneg && d_mask01 && d_h0 && d_c0 && d_h_all && d_c_all,
               "zr_lstm_stack_forward: null pointer");
  const int H = layers[0] ? layers[0]->H : 0;
  bool vec = (H > 0) && (H % 4 == 0) && aligned16(d_embed);
  for (int l = 0; l < nl; ++l) {
    ZR_CHECK_ARG(layers[l] && layers[l]->H == H, "zr_lstm_stack_forward: layer %d missing or of different size", l);
    ZR_CHECK_ARG(d_h0[l] && d_c0[l] && d_h_all[l] && d_c_all[l], "zr_lstm_stack_forward: null state for layer %d", l);
    vec = vec && aligned16(d_h0[l]) && aligned16(d_h_all[l]);
  }
  const size_t n = (size_t)H * mb;
  // Diagonal wavefront: units (l, t) with l + t = d only depend on diagonal d-1.
  for (int d = 0; d < T + nl - 1; ++d) {
    LstmLaunch L = {};
    L.H = H;
    L.mb = mb;
    L.clip = clip_threshold;
    int nu = 0;
    for (int l = 0; l < nl; ++l) {
      const int t = d - l;
      if (t < 0 || t >= T) continue;
      LstmUnit& U = L.u[nu++];
      U.W = layers[l]->d_W;
      U.bias = layers[l]->d_bias;
      if (l == 0) {
        U.in[0] = d_embed;
        U.gather_ids = d_ids_nonneg + (size_t)t * mb;
        U.V = V;
      } else {
        U.in[0] = d_h_all[l - 1] + (size_t)t * n;
        U.gather_ids = nullptr;
        U.V = 0;
      }
      U.in[1] = (t == 0) ? d_h0[l] : d_h_all[l] + (size_t)(t - 1) * n;
      U.in[2] = nullptr;
      U.cprev = (t == 0) ? d_c0[l] : d_c_all[l] + (size_t)(t - 1) * n;
      U.mask01 = d_mask01 + (size_t)t * mb;
      U.h = d_h_all[l] + (size_t)t * n;
      U.c = d_c_all[l] + (size_t)t * n;
      for (int g = 0; g < 4; ++g) U.gates[g] = nullptr;
      U.nseg = 2;
      if (nu == kMaxUnits) {
        L.n_units = nu;
        rc = launch_fused(ctx, L, vec);
        if (rc) return rc;
        nu = 0;
      }
    }
    if (nu > 0) {
      L.n_units = nu;
      rc = launch_fused(ctx, L, vec);
      if (rc) return rc;
    }
  }
  return ZR_OK;
}

}  // extern "C"
