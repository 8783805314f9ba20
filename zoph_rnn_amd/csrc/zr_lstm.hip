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
  const void* W;            // [nseg][4] packed matrices: fp32 [kp/4][ldw][4] or bf16 [kp/8][ldw][8] each
  const float* bias;        // [4][H]
  const float* in[3];       // segment inputs, H x mb (ld = H)
  const float* inp[3];      // optional copies of the same inputs packed as [H/4][mb][4] (null: use in[])
  const unsigned short* inp_lo[3];  // bf16 weights: inp[] then holds the bf16 "hi" half of the split inputs
                                    // ([H/8][mb][8]) and inp_lo[] the "lo" half
  float* hp;                // optional: h is also written packed as [H/4][mb][4] for the units that consume it
  unsigned short* hsplit_hi;  // optional: h is also written as bf16 terms, k-interleaved by 8 ([H/8][mb][8]), the layout
  unsigned short* hsplit_lo;  // products against bf16 weights read (hsplit_lo null: single term); same rounding as
                              // zr_split_pack_multi_kernel
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
  int bf16;                 // the weights of every unit are bf16 (zr_lstm_weights::bf16)
  int bf16_single;          // bf16 weights: activations enter as one bf16 term instead of two
  int nseg_max;             // largest nseg among the units
  int H, mb;
  int ldw, kp;              // packed weight extents: rows per k-block (H up to 32), K (H up to 8), zero filled
  float* preact;            // non-null: store the four pre-activation sums ([4][H*mb], no bias) instead of the cell
  float clip;
  int j_tiles, n_tiles;
  int buf_ok;               // host: H % 8 == 0 and every operand array is below 4 GiB (buffer-load variants)
  // K split ACROSS workgroups (SPLIT variant of lstm_fused_kernel): blockIdx.y = part of every segment's K range
  int kparts;
  float* partials;   // [tile][part][visit][gate][thread]
  int* counters;     // [tile], zero between launches
};

// Prefetch distance (k-groups) of the register-streaming kernel: a fragment is 4*(4+TN) registers and 4+TN
// 16-byte loads; the accumulators take 64*TN registers of the 512 a wave may use at one wave per SIMD (KS = 4)
// or of the 256 at two (KS = 8).
constexpr int lstm_prefetch_depth(int tn, int ks) {
#ifdef ZR_LSTM_PF
  return ZR_LSTM_PF;
#else
  return ks > 4 ? (tn == 1 ? 5 : 2) : (tn == 1 ? 8 : (tn == 2 ? 6 : (tn == 3 ? 3 : 1)));
#endif
}

// SPLIT: the K range of every segment is also divided over gridDim.y workgroups (a single node cannot fill the chip
// with whole-K tiles).  Each writes its tile of partial sums; the last to arrive at the tile's counter adds the parts
// in part order -- the same order whoever is last, so results do not depend on timing -- and runs the cell epilogue.
// BUF: operands are fetched with buffer loads (zr_mma_segment_u): fp32 weights, 16-byte aligned activations,
// H % 8 == 0 and every operand array below 4 GiB (the host checks).
template <int TN, int KS, bool VEC, bool BF16 = false, bool XPK = false, bool SPLIT = false, bool BUF = false,
          bool ONE_TERM = false>
__global__ void __launch_bounds__(64 * KS) lstm_fused_kernel(LstmLaunch L) {
  // Four waves at up to 64 columns (one workgroup per CU at these register counts anyway) sum their partial tiles in
  // one LDS round, which takes all 16 sub-tiles of every wave at once; the other shapes go gate by gate.
  constexpr bool WIDE = KS == 4 && TN <= 2 && !BF16;
  __shared__ __align__(16) float red[(WIDE ? 4 : 1) * KS * TN * 16 * 64];
  __shared__ int s_last;
  auto visit_slot = [&](int kslice_, int i) {
    if constexpr (WIDE)
      return zr_wide_visit_slot<KS>(kslice_, i);
    else
      return zr_visit_slot<KS>(kslice_, i);
  };
  auto reduce_visit = [&](zr_f32x16(&acc_)[4][TN], int kslice_, int lane_, auto f) {
    if constexpr (WIDE)
      zr_reduce_visit_wide<4, TN, KS>(acc_, red, kslice_, lane_, f);
    else
      zr_reduce_visit<4, TN, KS>(acc_, red, kslice_, lane_, f);
  };
  // Workgroup ids congruent modulo 8 run on the same XCD (round-robin dispatch) and share its L2.  Each XCD gets
  // a contiguous range of (unit, row tile) groups and every column tile of those groups: a weight tile is
  // fetched from memory once however many column tiles read it, and an XCD touches the activations of one or
  // two units only instead of all of them.
  const int id = blockIdx.x;
  const int r8 = id & 7;
  const int q = id >> 3;
  const int nt = q % L.n_tiles;
  const int groups = L.n_units * L.j_tiles;
  const int group = r8 * ((groups + 7) >> 3) + q / L.n_tiles;
  if (q / L.n_tiles >= ((groups + 7) >> 3) || group >= groups) return;
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

  // Epilogue operands are fetched now, ahead of the K loop, so that their memory latency is not paid after it.
  constexpr int NV = zr_visit_count<TN, KS>();
  const float bi = U.bias[jc], bf = U.bias[H + jc], bc = U.bias[2 * H + jc], bo = U.bias[3 * H + jc];
  float cprev_v[NV], mask_v[NV];
#pragma unroll
  for (int i = 0; i < NV; ++i) {
    const int slot = visit_slot(kslice, i);
    const int tn = slot >> 4, r = slot & 15;
    int n = n0 + tn * 32 + 8 * (r >> 2) + 4 * half + (r & 3);
    n = n < L.mb ? n : L.mb - 1;
    cprev_v[i] = L.preact ? 0.0f : U.cprev[(long long)n * H + jc];
    mask_v[i] = (float)U.mask01[n];
  }

  const long long HH = (long long)L.kp * L.ldw;  // elements per packed matrix
  for (int s = 0; s < U.nseg; ++s) {
    if constexpr (BF16) {
      const unsigned short* wbase[4];
      unsigned woff[4];
      const float* xcol[TN];
#pragma unroll
      for (int g = 0; g < 4; ++g) {
        wbase[g] = (const unsigned short*)U.W + ((long long)s * 4 + g) * HH;
        woff[g] = (unsigned)(8 * j + 8 * half * L.ldw);
      }
#pragma unroll
      for (int tn = 0; tn < TN; ++tn) {
        long long c = cols[tn];
        if (s == 0 && U.gather_ids) {
          int idv = U.gather_ids[cols[tn]];
          idv = idv < 0 ? 0 : (idv >= U.V ? U.V - 1 : idv);
          c = idv;
        }
        xcol[tn] = U.in[s] + c * H + 8 * half;
      }
      if constexpr (XPK) {
        const unsigned short* xlo[TN];
#pragma unroll
        for (int tn = 0; tn < TN; ++tn) {
          const long long off = 8LL * (cols[tn] + (long long)half * L.mb);
          xcol[tn] = (const float*)((const unsigned short*)U.inp[s] + off);
          xlo[tn] = U.inp_lo[s] + off;
        }
        // ONE_TERM: single-term mode, activations rounded to bf16 once (no lo array)
        zr_mma_segment_bf16<4, TN, KS, (TN == 1 ? 6 : 4), true, !ONE_TERM>(acc, wbase, woff, (long long)L.ldw, xcol, H,
                                                                            kslice, xlo, L.mb);
      } else {
        zr_mma_segment_bf16<4, TN, KS, (TN == 1 ? 6 : 4), false, !ONE_TERM>(acc, wbase, woff, (long long)L.ldw, xcol, H,
                                                                             kslice);
      }
    } else if constexpr (BUF) {
      // k-groups [g0, g1) of this segment (all of them unless K is also split across workgroups)
      int g0 = 0, g1 = H >> 3;
      if constexpr (SPLIT) {
        const int groups = H >> 3, part = blockIdx.y;
        g0 = (int)((long long)groups * part / L.kparts);
        g1 = (int)((long long)groups * (part + 1) / L.kparts);
      }
      unsigned wsoff[4], xoffb[TN];
#pragma unroll
      for (int g = 0; g < 4; ++g) wsoff[g] = (unsigned)((((long long)s * 4 + g) * HH + (long long)g0 * 8 * L.ldw) * 4);
      const unsigned woffb = 16u * (unsigned)(j + half * L.ldw);
      const bool packed = U.inp[s] != nullptr;
#pragma unroll
      for (int tn = 0; tn < TN; ++tn) {
        unsigned c = (unsigned)cols[tn];
        if (s == 0 && U.gather_ids) {
          int idv = U.gather_ids[cols[tn]];
          c = (unsigned)(idv < 0 ? 0 : (idv >= U.V ? U.V - 1 : idv));
        }
        xoffb[tn] = packed ? 16u * ((unsigned)cols[tn] + (unsigned)(half * L.mb)) : 4u * (c * (unsigned)H + 4u * half);
      }
      const float* xb = packed ? U.inp[s] + (long long)g0 * 8 * L.mb : U.in[s] + g0 * 8;
      zr_mma_segment_ring<4, TN, KS, lstm_prefetch_depth(TN, KS)>(acc, zr_make_rsrc(U.W), wsoff, woffb, 32u * (unsigned)L.ldw,
                                                                  zr_make_rsrc(xb), xoffb,
                                                                  packed ? 32u * (unsigned)L.mb : 32u, (g1 - g0) * 8, kslice);
    } else {
      const float* wbase[4];
      unsigned woff[4];
      const float* xcol[TN];
#pragma unroll
      for (int g = 0; g < 4; ++g) {
        wbase[g] = (const float*)U.W + ((long long)s * 4 + g) * HH;
        woff[g] = (unsigned)(4 * j + 4 * half * L.ldw);  // j < ldw: padded rows are zeros
      }
#pragma unroll
      for (int tn = 0; tn < TN; ++tn) {
        long long c = cols[tn];
        if (s == 0 && U.gather_ids) {
          int idv = U.gather_ids[cols[tn]];
          idv = idv < 0 ? 0 : (idv >= U.V ? U.V - 1 : idv);
          c = idv;
        }
        xcol[tn] = (VEC && U.inp[s]) ? U.inp[s] + 4LL * cols[tn] + 4LL * half * L.mb : U.in[s] + c * H + 4 * half;
      }
      const int xstride = (VEC && U.inp[s]) ? L.mb : 1;
      if constexpr (SPLIT) {
        // this workgroup's share of the segment: k-groups [g0, g1) of H / 8 (H % 8 == 0 on this path)
        const int groups = H >> 3, part = blockIdx.y;
        const int g0 = (int)((long long)groups * part / L.kparts), g1 = (int)((long long)groups * (part + 1) / L.kparts);
#pragma unroll
        for (int g = 0; g < 4; ++g) wbase[g] += (long long)g0 * 8 * L.ldw;
#pragma unroll
        for (int tn = 0; tn < TN; ++tn) xcol[tn] += (long long)g0 * 8 * xstride;
        zr_mma_segment<4, TN, KS, lstm_prefetch_depth(TN, KS), ZR_A_PACK4, VEC>(
            acc, wbase, woff, (long long)L.ldw, xcol, (g1 - g0) * 8, kslice, half, xstride);
      } else {
        zr_mma_segment<4, TN, KS, lstm_prefetch_depth(TN, KS), ZR_A_PACK4, VEC>(
            acc, wbase, woff, (long long)L.ldw, xcol, H, kslice, half, xstride);
      }
    }
  }

  const bool j_ok = j < H;
  auto finish = [&](const float(&z)[4], int tn, int r, int vi) {
    const int n = n0 + tn * 32 + 8 * (r >> 2) + 4 * half + (r & 3);
    if (j_ok && n < L.mb) {
      const long long ix = (long long)n * H + j;
      if (L.preact) {
        const long long gs = (long long)H * L.mb;
        L.preact[ix] = z[0];
        L.preact[gs + ix] = z[1];
        L.preact[2 * gs + ix] = z[2];
        L.preact[3 * gs + ix] = z[3];
        return;
      }
      float gi, gf, gc, go, c, h;
      zr_lstm_cell(z[0] + bi, z[1] + bf, z[2] + bc, z[3] + bo, cprev_v[vi], mask_v[vi], L.clip, gi, gf, gc, go, c, h);
      U.c[ix] = c;
      U.h[ix] = h;
      if (U.hp) U.hp[((long long)(j >> 2) * L.mb + n) * 4 + (j & 3)] = h;
      if (U.hsplit_hi) {
        const __bf16 hb = (__bf16)h;
        const long long o = ((long long)(j >> 3) * L.mb + n) * 8 + (j & 7);
        U.hsplit_hi[o] = __builtin_bit_cast(unsigned short, hb);
        if (U.hsplit_lo) U.hsplit_lo[o] = __builtin_bit_cast(unsigned short, (__bf16)(h - (float)hb));
      }
      if (U.gates[0]) {
        U.gates[0][ix] = gi;
        U.gates[1][ix] = gf;
        U.gates[2][ix] = gc;
        U.gates[3][ix] = go;
      }
    }
  };
  if constexpr (!SPLIT) {
    reduce_visit(acc, kslice, lane, finish);
  } else {
    constexpr int NTHR = 64 * KS;
    const int tile = group * L.n_tiles + nt;
    const int parts = L.kparts, part = blockIdx.y;
    // partial tile of this workgroup: [visit][gate][thread], written and read with device-scope relaxed atomics
    // (cache-bypassing on this multi-die part), published by the counter increment behind the barrier
    float* mine = L.partials + ((long long)tile * parts + part) * (NV * 4 * NTHR) + tid;
    reduce_visit(acc, kslice, lane, [&](const float(&z)[4], int, int, int vi) {
#pragma unroll
      for (int g = 0; g < 4; ++g)
        __hip_atomic_store(mine + (vi * 4 + g) * NTHR, z[g], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    });
    zr_publish_barrier();
    if (tid == 0) {
      const int old = atomicAdd(&L.counters[tile], 1);
      s_last = (old == parts - 1) ? 1 : 0;
    }
    __syncthreads();
    if (!s_last) return;
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "workgroup");
    const float* base = L.partials + (long long)tile * parts * (NV * 4 * NTHR) + tid;
    float sum[NV][4];
    for (int p = 0; p < parts; ++p) {  // part order 0, 1, ... for every finisher
      const float* pp = base + (long long)p * (NV * 4 * NTHR);
      float t[NV][4];
#pragma unroll
      for (int vi = 0; vi < NV; ++vi)
#pragma unroll
        for (int g = 0; g < 4; ++g)
          t[vi][g] = __hip_atomic_load(pp + (vi * 4 + g) * NTHR, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
#pragma unroll
      for (int vi = 0; vi < NV; ++vi)
#pragma unroll
        for (int g = 0; g < 4; ++g) sum[vi][g] = (p == 0) ? t[vi][g] : sum[vi][g] + t[vi][g];
    }
    if (tid == 0) __hip_atomic_store(&L.counters[tile], 0, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);  // next launch
#pragma unroll
    for (int vi = 0; vi < NV; ++vi) {
      const int slot = visit_slot(kslice, vi);
      finish(sum[vi], slot >> 4, slot & 15, vi);
    }
  }
}

// ---------------------------------------------------------------------------------------------------------
// Second kernel: weights staged through LDS and shared by the waves of a workgroup, K split ACROSS workgroups.
//
// Why: with one 128-row x 64-column tile per CU and full K, every CU pulls (128 + 64) * K floats through its L1,
// 384 MB per 4-node launch, and the kernel runs at the L1 fill rate (about 18 GB/s per CU) rather than at the MFMA
// rate.  The traffic per CU is (rows + cols) * K for a fixed rows * cols * K of work, so it falls when a CU owns a
// bigger tile over a shorter K range.  Here a workgroup owns 32 rows x 4 gates x (NWV * 32 * TN) columns -- all
// 128 columns of the benchmark minibatch -- for one K segment (or a part of one): its NWV waves take 32*TN
// columns each, share every weight chunk through LDS (read from L2 once per workgroup, 16-byte coalesced), and
// fetch only their own activation columns.  The S = segments x parts workgroups of a tile write their partial
// tiles to a scratch buffer; the last one to arrive (device-scope counter) adds the partials in split order --
// the same order whoever is last, so results are deterministic -- and runs the gate/cell epilogue in registers.
// ---------------------------------------------------------------------------------------------------------
struct LstmLaunch2 {
  LstmLaunch base;
  int kparts;        // K parts per segment
  int n_chunks;      // ceil(H / 32)
  float* partials;   // [tile][split][wave][4*TN*16][64]
  int* counters;     // [tile], zero between launches
};

template <int TN, int NWV>
__global__ void __launch_bounds__(64 * NWV) lstm_lds_kernel(LstmLaunch2 P) {
  constexpr int KC = 32;                       // k per chunk
  constexpr int NTHR = 64 * NWV;
  constexpr int F4_PER_CHUNK = (KC / 4) * 4 * 32;  // float4 per weight chunk: 8 k-blocks x 4 gates x 32 rows
  constexpr int WLD = (F4_PER_CHUNK + NTHR - 1) / NTHR;  // float4 loads per thread per chunk
  __shared__ zr_f32x4 Ws4[2][F4_PER_CHUNK];
  __shared__ int s_last;
  const LstmLaunch& L = P.base;
  const int id = blockIdx.x;
  const int r8 = id & 7;
  const int q = id >> 3;
  const int splits = L.nseg_max * P.kparts;
  const int sp = q % splits;
  const int n_tiles_total = L.n_units * L.j_tiles * L.n_tiles;
  const int tiles_per_xcd = (n_tiles_total + 7) >> 3;  // contiguous tiles per XCD (ids congruent mod 8 share one)
  const int tile = r8 * tiles_per_xcd + q / splits;
  if (q / splits >= tiles_per_xcd || tile >= n_tiles_total) return;
  const int nt = tile % L.n_tiles;
  const int jt = (tile / L.n_tiles) % L.j_tiles;
  const int unit = tile / (L.n_tiles * L.j_tiles);
  const LstmUnit& U = L.u[unit];
  const int seg = sp / P.kparts;
  const int part = sp % P.kparts;
  const bool seg_live = seg < U.nseg;  // units with fewer segments than the launch maximum contribute zeros

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int jl = lane & 31;
  const int half = lane >> 5;
  const int H = L.H;
  const int j0 = jt * 32;
  const int n0 = nt * (32 * TN * NWV) + wave * (32 * TN);
  const int j = j0 + jl;

  const int c_begin = (int)((long long)P.n_chunks * part / P.kparts);
  const int c_end = (int)((long long)P.n_chunks * (part + 1) / P.kparts);

  // this lane's activation columns (segment `seg`)
  const float* xcol[TN];
#pragma unroll
  for (int tn = 0; tn < TN; ++tn) {
    int c = n0 + tn * 32 + jl;
    c = c < L.mb ? c : L.mb - 1;
    long long col = c;
    const int s_eff = seg_live ? seg : 0;
    if (s_eff == 0 && U.gather_ids) {
      int idv = U.gather_ids[c];
      idv = idv < 0 ? 0 : (idv >= U.V ? U.V - 1 : idv);
      col = idv;
    }
    xcol[tn] = U.in[s_eff] + col * H;
  }
  // this thread's share of a weight chunk: float4 index f -> (k-block, gate, row); a float4 of the packed
  // weights is four consecutive k of one row
  const float* wsrc[WLD];
  bool wok_row[WLD];
  int wkb[WLD];
  const long long HH = (long long)L.kp * L.ldw;
  const int kblocks = L.kp >> 2;
#pragma unroll
  for (int u = 0; u < WLD; ++u) {
    const int f = tid + NTHR * u;
    const int row = f & 31, g = (f >> 5) & 3, kb = f >> 7;
    wok_row[u] = seg_live && (f < F4_PER_CHUNK);  // rows >= H and k >= H of the packed weights are zeros
    wkb[u] = kb;
    wsrc[u] = (const float*)U.W + ((long long)(seg_live ? seg : 0) * 4 + g) * HH + 4 * (j0 + row);
  }

  zr_f32x16 acc[4][TN];
#pragma unroll
  for (int g = 0; g < 4; ++g)
#pragma unroll
    for (int tn = 0; tn < TN; ++tn)
#pragma unroll
      for (int r = 0; r < 16; ++r) acc[g][tn][r] = 0.0f;

  zr_f32x4 wreg[WLD];
  zr_f32x4 xf[2][4][TN];

  // All loads are unconditional with clamped addresses (loads under branches stop the compiler from counting
  // loads in flight and force full waits).  gload only issues loads; out-of-range weights are zeroed by a
  // multiplication in lds_store (weights are finite), so that nothing consumes a loaded value right after its load.
  auto gload = [&](int c, zr_f32x4 (&xdst)[4][TN]) {
    const int cc = c < c_end ? c : c_end - 1;  // dummy chunk (odd chunk count): clamped, zeroed at store time
#pragma unroll
    for (int u = 0; u < WLD; ++u) {
      const int kb = cc * (KC / 4) + wkb[u];
      const int kbc = kb < kblocks ? kb : kblocks - 1;
      wreg[u] = *(const zr_f32x4*)(wsrc[u] + (long long)kbc * (4 * L.ldw));
    }
#pragma unroll
    for (int gq = 0; gq < 4; ++gq) {
      // this lane multiplies k = kx .. kx+3; past the end of the column the matching weights are zero, so
      // any valid address will do
      int kx = cc * KC + 8 * gq + 4 * half;
      kx = (kx + 4 <= H) ? kx : H - 4;
#pragma unroll
      for (int tn = 0; tn < TN; ++tn) xdst[gq][tn] = *(const zr_f32x4*)(xcol[tn] + kx);
    }
  };
  auto lds_store = [&](int buf, int c) {
    const bool chunk_ok = c < c_end;
    const int cc = chunk_ok ? c : c_end - 1;
#pragma unroll
    for (int u = 0; u < WLD; ++u) {
      const int f = tid + NTHR * u;
      const float keep = (chunk_ok && wok_row[u] && (cc * (KC / 4) + wkb[u]) < kblocks) ? 1.0f : 0.0f;
      zr_f32x4 v = wreg[u];
      v.x *= keep;
      v.y *= keep;
      v.z *= keep;
      v.w *= keep;
      if (f < F4_PER_CHUNK) Ws4[buf][f] = v;
    }
  };
  auto compute = [&](int buf, const zr_f32x4 (&xs)[4][TN]) {
    // LDS -> register fragments one k-group ahead of the MFMAs that use them: k-group gq is k-blocks 2*gq and
    // 2*gq + 1, one per half-wave; a lane reads its row's four k of each gate with one 16-byte read
    const zr_f32x4* Ws = &Ws4[buf][0] + half * 4 * 32 + jl;
    float wf[2][4][4];
    auto lds_frag = [&](float (&dst)[4][4], int gq) {
#pragma unroll
      for (int g = 0; g < 4; ++g) {
        const zr_f32x4 v = Ws[(2 * gq * 4 + g) * 32];
        dst[0][g] = v.x;
        dst[1][g] = v.y;
        dst[2][g] = v.z;
        dst[3][g] = v.w;
      }
    };
    lds_frag(wf[0], 0);
#pragma unroll
    for (int gq = 0; gq < 4; ++gq) {
      if (gq + 1 < 4) lds_frag(wf[(gq + 1) & 1], gq + 1);
      // keep the LDS reads ahead of the MFMAs: left alone, the scheduler sinks each read to just before its use
      // (shortest live range) and the matrix pipe idles for an LDS round trip every other instruction
      __builtin_amdgcn_sched_barrier(0);
#pragma unroll
      for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int g = 0; g < 4; ++g)
#pragma unroll
          for (int tn = 0; tn < TN; ++tn)
            acc[g][tn] = __builtin_amdgcn_mfma_f32_32x32x2f32(xs[gq][tn][i], wf[gq & 1][i][g], acc[g][tn], 0, 0, 0);
    }
  };

  if (c_begin < c_end) {
    gload(c_begin, xf[0]);
    lds_store(0, c_begin);
    __syncthreads();
    for (int c = c_begin; c < c_end; c += 2) {
      // even stage: chunk c from buffer 0, prefetch c+1 into buffer 1
      gload(c + 1, xf[1]);
      compute(0, xf[0]);
      lds_store(1, c + 1);
      __syncthreads();
      // odd stage: chunk c+1 (all-zero weights if past the end) from buffer 1, prefetch c+2 into buffer 0
      gload(c + 2, xf[0]);
      compute(1, xf[1]);
      lds_store(0, c + 2);
      __syncthreads();
    }
  }

  const int jc = j < H ? j : H - 1;
  const float bi = U.bias[jc], bf = U.bias[H + jc], bc = U.bias[2 * H + jc], bo = U.bias[3 * H + jc];
  constexpr int SLOTS = 4 * TN * 16;
  if (splits > 1) {
    float* mine = P.partials + (((long long)tile * splits + sp) * NWV + wave) * (SLOTS * 64);
#pragma unroll
    for (int g = 0; g < 4; ++g)
#pragma unroll
      for (int tn = 0; tn < TN; ++tn)
#pragma unroll
        for (int r = 0; r < 16; ++r)
          __hip_atomic_store(mine + ((g * TN + tn) * 16 + r) * 64 + lane, acc[g][tn][r], __ATOMIC_RELAXED,
                             __HIP_MEMORY_SCOPE_AGENT);
    // The partials are written and read with device-scope atomic accesses (write-through / cache-bypassing on
    // this multi-die part), so no L2 write-back + invalidate is needed to publish them -- a full device-scope
    // fence here costs more than the whole K loop.  Every wave waits for its own stores to complete before the
    // barrier; the counter increment after the barrier is a device-scope atomic.
    zr_publish_barrier();
    if (tid == 0) {
      const int old = atomicAdd(&P.counters[tile], 1);
      s_last = (old == splits - 1) ? 1 : 0;
    }
    __syncthreads();
    if (!s_last) return;
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "workgroup");
    const float* base = P.partials + ((long long)tile * splits * NWV + wave) * (SLOTS * 64);
    // split order k = 0, 1, ... for every finisher: the sum does not depend on which workgroup arrived last.
    // All loads of one split are issued before any is consumed.
    for (int k = 0; k < splits; ++k) {
      const float* pk = base + (long long)k * NWV * (SLOTS * 64) + lane;
#pragma unroll
      for (int g = 0; g < 4; ++g)
#pragma unroll
        for (int tn = 0; tn < TN; ++tn) {
          float t[16];
#pragma unroll
          for (int r = 0; r < 16; ++r)
            t[r] = __hip_atomic_load(pk + ((g * TN + tn) * 16 + r) * 64, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
#pragma unroll
          for (int r = 0; r < 16; ++r) acc[g][tn][r] = (k == 0) ? t[r] : acc[g][tn][r] + t[r];
        }
    }
    if (tid == 0) __hip_atomic_store(&P.counters[tile], 0, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);  // next launch
  }
  if (j < H) {
#pragma unroll
    for (int tn = 0; tn < TN; ++tn)
#pragma unroll
      for (int r = 0; r < 16; ++r) {
        const int n = n0 + tn * 32 + 8 * (r >> 2) + 4 * half + (r & 3);
        if (n < L.mb) {
          const long long ix = (long long)n * H + j;
          float gi, gf, gc, go, c, h;
          zr_lstm_cell(acc[0][tn][r] + bi, acc[1][tn][r] + bf, acc[2][tn][r] + bc, acc[3][tn][r] + bo, U.cprev[ix],
                       (float)U.mask01[n], L.clip, gi, gf, gc, go, c, h);
          U.c[ix] = c;
          U.h[ix] = h;
          if (U.hp) U.hp[((long long)(j >> 2) * L.mb + n) * 4 + (j & 3)] = h;
          if (U.gates[0]) {
            U.gates[0][ix] = gi;
            U.gates[1][ix] = gf;
            U.gates[2][ix] = gc;
            U.gates[3][ix] = go;
          }
        }
      }
  }
}

// ---------------------------------------------------------------------------------------------------------
// Whole-sweep kernel: ONE launch runs every (layer, time step) node of a stacked forward pass.
//
// A workgroup owns the same tile -- 32 hidden rows x 32*TN batch columns of one layer -- at every time step and loops
// over t itself.  Node (l, t) needs h of (l-1, t) and of (l, t-1), each produced by the j_tiles workgroups that own
// the same batch columns of that layer: every (layer, column tile) has an arrival counter in device memory that its
// producers bump once per time step, and a consumer waits until the counter reaches (steps needed) * j_tiles.  The
// layers settle into a skewed pipeline: a layer above the first consumes its recurrent input first and the input from
// below second, so it trails the layer below by half a step and that hand-over hides behind half a K loop; a layer
// never waits for the layer above it.
// Compared with one launch per diagonal this removes, per step, the launch, the drain of the slowest tile and the
// refill of the operand pipeline from a cold start; the cell state never leaves registers.
//
// Hand-over through memory: h is written twice, to the caller's array (plain stores, visible at kernel end) and to a
// k-interleaved copy [H/4][mb][4] per (layer, t) that the consumers read.  The chip's eight dies have one L2 each.
// The copy is written with device-scope stores (written through to memory); every wave waits for its stores to
// complete, then a workgroup barrier, then one thread bumps the counter.  A consumer polls the counter with
// device-scope loads and reads the copy with ordinary loads.  Those cannot hit a stale line as long as no line is
// cached before it was written: caches are clean when the kernel starts, every line of a copy is read only after
// the wait for its producers, and with mb % 8 == 0 a 128-byte line (8 columns x 4 rows) has one producer.  For other
// minibatch sizes lines straddle producers, and the consumers invalidate their caches after every wait instead
// (device-scope acquire), which costs about 4 % at the benchmark shape.
//
// Operand fetch: buffer loads (descriptor base + scalar offset advancing with k + fixed 32-bit lane offset), so the K
// loop holds no vector instruction other than the MFMAs; see zr_mma_segment_u.
//
// Progress: the launch must be wholly resident (the host checks grid <= CUs x resident workgroups per CU), then the
// dependency graph is acyclic and every wait ends.  Every wait is bounded all the same: a workgroup that runs out of
// polls marks every counter, which releases all other waiters, raises the status flag and leaves; the others leave
// at their next wait.
// ---------------------------------------------------------------------------------------------------------
constexpr int kSweepGaveUp = 1 << 28;  // bit set in every counter by a workgroup that stopped waiting
constexpr int kSweepCtrStride = 32;    // ints between counters: one 128-byte line each

struct LstmSweep {
  const float* W[kMaxUnits];     // per layer: [2][4] packed fp32 matrices
  const float* bias[kMaxUnits];  // per layer: [4][H]
  const float* h0[kMaxUnits];
  const float* c0[kMaxUnits];
  float* h_all[kMaxUnits];
  float* c_all[kMaxUnits];
  float* gates_all[kMaxUnits];   // null: gates not kept
  const float* embed;
  const int* ids;                // [T][mb], already non-negative
  const int* mask01;             // [T][mb]
  float* hp;                     // [nl][T] k-interleaved copies of h, H*mb floats each
  int* counters;                 // [nl][n_tiles] at kSweepCtrStride, zero at launch
  int* status;                   // set to 1 when a wait was abandoned
  int nl, T, V, H, mb, ldw, kp, j_tiles, n_tiles;
  float clip;
  int spin_limit;
  int fence;   // 1: consumers invalidate their caches after every wait (see lstm_sweep_kernel)
};

// All threads of the workgroup call this.  False: leave the kernel.
__device__ __forceinline__ bool sweep_wait(const LstmSweep& P, int* ctr, int target, int* s_go) {
  if (threadIdx.x == 0) {
    int v = __hip_atomic_load(ctr, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    for (int spins = 0; v < target && spins < P.spin_limit; ++spins) {
      __builtin_amdgcn_s_sleep(8);
      v = __hip_atomic_load(ctr, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    }
    const bool ok = v >= target && !(v & kSweepGaveUp);
    if (!ok) {
      if (!(v & kSweepGaveUp)) {
        const int n = P.nl * P.n_tiles;
        for (int i = 0; i < n; ++i) atomicOr(P.counters + i * kSweepCtrStride, kSweepGaveUp);
      }
      __hip_atomic_store(P.status, 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    }
    *s_go = ok ? 1 : 0;
  }
  __syncthreads();
  const bool go = *s_go != 0;
  if (go && P.fence) __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "agent");
  return go;
}

template <int TN>
__global__ void __launch_bounds__(256) lstm_sweep_kernel(LstmSweep P) {
  constexpr int KS = 4;
  __shared__ __align__(16) float red[KS * 4 * TN * 16 * 64];  // all partial tiles of the workgroup at once
  __shared__ int s_go[2];
  // same die-aware placement as lstm_fused_kernel, with one unit per layer.  (Two workgroups per CU on 32-column tiles
  // -- 512 workgroups for four layers of H = 1000 at 128 columns -- measured 2 % slower than one on 64-column tiles.)
  const int id = blockIdx.x;
  const int r8 = id & 7;
  const int q = id >> 3;
  const int nt = q % P.n_tiles;
  const int groups = P.nl * P.j_tiles;
  const int group = r8 * ((groups + 7) >> 3) + q / P.n_tiles;
  if (q / P.n_tiles >= ((groups + 7) >> 3) || group >= groups) return;
  const int l = group / P.j_tiles;
  const int jt = group % P.j_tiles;

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int kslice = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int H = P.H, mb = P.mb;
  const int j0 = jt * 32;
  const int n0 = nt * 32 * TN;
  const long long n_el = (long long)H * mb;
  constexpr int NV = zr_visit_count<TN, KS>();
  // batch column of visit i of a lane in half-wave `half`, clamped
  auto visit_col = [&](int i, int half) {
    const int slot = zr_wide_visit_slot<KS>(kslice, i);
    const int tn = slot >> 4, r = slot & 15;
    const int n = n0 + tn * 32 + 8 * (r >> 2) + 4 * half + (r & 3);
    return n < mb ? n : mb - 1;
  };
  auto clamp_col = [&](int c) { return c < mb ? c : mb - 1; };
  auto clamp_id = [&](int v) { return v < 0 ? 0 : (v >= P.V ? P.V - 1 : v); };

  const float* bias = P.bias[l];
  float bi, bf, bc, bo;
  float c_state[NV];  // cell state of this thread's outputs, carried from step to step
  int idv[TN];        // layer 0: embedding column of each batch column, fetched one step ahead
  {
    const int jl = lane & 31, half = lane >> 5;
    const int jc = j0 + jl < H ? j0 + jl : H - 1;
    bi = bias[jc], bf = bias[H + jc], bc = bias[2 * H + jc], bo = bias[3 * H + jc];
#pragma unroll
    for (int i = 0; i < NV; ++i) c_state[i] = P.c0[l][(long long)visit_col(i, half) * H + jc];
#pragma unroll
    for (int tn = 0; tn < TN; ++tn) idv[tn] = (l == 0) ? clamp_id(P.ids[clamp_col(n0 + tn * 32 + jl)]) : 0;
  }

  const long long HH = (long long)P.kp * P.ldw;
  const float* Wl = P.W[l];
  int* my_ctr = P.counters + (l * P.n_tiles + nt) * kSweepCtrStride;
  int* below_ctr = P.counters + ((l > 0 ? l - 1 : 0) * P.n_tiles + nt) * kSweepCtrStride;
  float* hp_mine = P.hp + (long long)l * P.T * n_el;
  const float* hp_below = P.hp + (long long)(l > 0 ? l - 1 : 0) * P.T * n_el;
  float* gates = P.gates_all[l];

  for (int t = 0; t < P.T; ++t) {
    // Everything that depends on the lane is derived afresh in each time step from a lane index the compiler cannot
    // see through: hoisted out of the loop, the per-lane addresses of both K loops would have to stay in registers
    // through all of it, and the kernel has none to spare.
    int lane_t = lane;
    asm volatile("" : "+v"(lane_t));
    const int jl = lane_t & 31, half = lane_t >> 5;
    const int j = j0 + jl;
    const bool j_ok = j < H;
    int cols[TN];
#pragma unroll
    for (int tn = 0; tn < TN; ++tn) cols[tn] = clamp_col(n0 + tn * 32 + jl);
    const unsigned woffb = 16u * (unsigned)(j + half * P.ldw);
    int idn[TN];
#pragma unroll
    for (int tn = 0; tn < TN; ++tn) {
      const int tt = t + 1 < P.T ? t + 1 : t;
      idn[tn] = (l == 0) ? clamp_id(P.ids[(long long)tt * mb + cols[tn]]) : 0;
    }

    zr_f32x16 acc[4][TN];
#pragma unroll
    for (int g = 0; g < 4; ++g)
#pragma unroll
      for (int tn = 0; tn < TN; ++tn)
#pragma unroll
        for (int r = 0; r < 16; ++r) acc[g][tn][r] = 0.0f;

    for (int q = 0; q < 2; ++q) {
      // segment 0: input from below (h of (l-1, t), or the embedding columns); segment 1: h of (l, t-1).  Layers above
      // the first take the recurrent segment first: it only needs the layer's own previous step, so a layer can trail
      // the one below it by half a step instead of a whole one (the pipeline of layers fills and drains in half the
      // time) and the wait for the layer below hides behind half a K loop.  The order is fixed per layer, so the
      // summation order, and with it every bit of the result, does not depend on timing.
      const int s = (l > 0) ? 1 - q : q;
      const bool packed = (s == 0) ? (l > 0) : (t > 0);
      // The weights of the first ring stages go out before the wait for the activations: they depend on nothing, so
      // their latency overlaps the poll (and the wait, when there is one): -2.8 % per sweep.  (Sending those of a
      // step's first segment out even earlier, before the previous step's epilogue, keeps 96 more registers live
      // through it and came out 0.3 % slower.)
      unsigned wsoff[4];
#pragma unroll
      for (int g = 0; g < 4; ++g) wsoff[g] = (unsigned)(((long long)s * 4 + g) * HH * 4);
      constexpr int PF = lstm_prefetch_depth(TN, KS);
      ZrFrag<4, TN> ring[PF + 1];
      const __amdgpu_buffer_rsrc_t wrsrc = zr_make_rsrc(Wl);
      zr_preload_w<4, TN, KS, PF>(ring, wrsrc, wsoff, woffb, 32u * (unsigned)P.ldw, H, kslice);
      if (packed) {
        int* ctr = (s == 0) ? below_ctr : my_ctr;
        const int target = ((s == 0) ? t + 1 : t) * P.j_tiles;
        if (!sweep_wait(P, ctr, target, &s_go[s])) return;
      }
      const float* xp = (s == 0) ? hp_below + (long long)t * n_el : hp_mine + (long long)(t > 0 ? t - 1 : 0) * n_el;
      const float* xu = (s == 0) ? P.embed : P.h0[l];
      unsigned xoffb[TN];
#pragma unroll
      for (int tn = 0; tn < TN; ++tn) {
        const unsigned c = (s == 0) ? (unsigned)idv[tn] : (unsigned)cols[tn];
        xoffb[tn] = packed ? 16u * ((unsigned)cols[tn] + (unsigned)(half * mb)) : 4u * (c * (unsigned)H + 4u * half);
      }
      zr_mma_segment_u<4, TN, KS, PF, true>(acc, wrsrc, wsoff, woffb, 32u * (unsigned)P.ldw,
                                            zr_make_rsrc(packed ? xp : xu), xoffb, packed ? 32u * (unsigned)mb : 32u, H,
                                            kslice, ring);
    }

    // the column masks are fetched here, behind the K loops, and arrive while the partial tiles are being summed
    float mask_v[NV];
#pragma unroll
    for (int i = 0; i < NV; ++i) mask_v[i] = (float)P.mask01[(long long)t * mb + visit_col(i, half)];
    float* h_out = P.h_all[l] + (long long)t * n_el;
    float* c_out = P.c_all[l] + (long long)t * n_el;
    float* hp_out = hp_mine + (long long)t * n_el;
    // Only the k-interleaved copy of h, which the waiting workgroups read, goes out before the arrival is published;
    // the outputs nobody waits for (h, c and the gate values kept for training) are held in registers and stored
    // after it, so that their write latency overlaps the next step instead of sitting in front of the publish.
    float h_v[NV], g_v[4][NV];
    zr_reduce_visit_wide<4, TN, KS>(acc, red, kslice, lane, [&](const float(&z)[4], int tn, int r, int vi) {
      const int n = n0 + tn * 32 + 8 * (r >> 2) + 4 * half + (r & 3);
      float c;
      zr_lstm_cell(z[0] + bi, z[1] + bf, z[2] + bc, z[3] + bo, c_state[vi], mask_v[vi], P.clip, g_v[0][vi], g_v[1][vi],
                   g_v[2][vi], g_v[3][vi], c, h_v[vi]);
      c_state[vi] = c;
      if (j_ok && n < mb)
        __hip_atomic_store(hp_out + ((long long)(j >> 2) * mb + n) * 4 + (j & 3), h_v[vi], __ATOMIC_RELAXED,
                           __HIP_MEMORY_SCOPE_AGENT);
    });
    // publish this step: every wave's stores have completed before the barrier, then one arrival per workgroup
    zr_publish_barrier();
    if (tid == 0) atomicAdd(my_ctr, 1);
#pragma unroll
    for (int i = 0; i < NV; ++i) {
      const int slot = zr_wide_visit_slot<KS>(kslice, i);
      const int n = n0 + (slot >> 4) * 32 + 8 * ((slot & 15) >> 2) + 4 * half + (slot & 3);
      if (j_ok && n < mb) {
        const long long ix = (long long)n * H + j;
        c_out[ix] = c_state[i];
        h_out[ix] = h_v[i];
        if (gates) {
          float* gt = gates + (long long)t * 4 * n_el + ix;
#pragma unroll
          for (int g = 0; g < 4; ++g) gt[g * n_el] = g_v[g][i];
        }
      }
    }
#pragma unroll
    for (int tn = 0; tn < TN; ++tn) idv[tn] = idn[tn];
  }
}

// ---------------------------------------------------------------------------------------------------------
// One decoder time step through ALL layers in one launch (the LSTM part of neuralMT_model::forward_prop_target,
// src/model.hpp:2573-2640: layer 0 on the embedding column of the current word, the previous step's attention output
// through Q when feed-input is on, layer l > 0 on h_t of layer l-1).
//
// A time step is a chain: layer l cannot start its M_l . h_t^{l-1} product before layer l-1 has finished, and one
// layer is too little work for the chip, so one launch per layer runs four short launches back to back, each with its
// own launch gap, ramp-up, cross-workgroup sum and tail.  But more than half of the step's products do not depend on
// the step at all: W_h . h_{t-1} of every layer and Q . h~_{t-1} read only the previous step.  Here every
// 32-row x 32*TN-column tile of the state has TWO resident workgroups for the whole step:
//   role 1 streams the products that depend on nothing -- W_h^l . h_{t-1}^l for l = 0, 1, ... (and the upper part of
//          Q's K range) -- never waits, and leaves each layer's partial pre-activation tile in device memory;
//   role 0 computes M_0 . x (x gathered from the embedding) and the lower part of Q's K range, then for each layer:
//          takes role 1's partial tile, adds it to its own sums (own + role 1's: one fixed order, so the result does
//          not depend on timing), runs the gate / cell epilogue, writes h and c, publishes a k-interleaved copy of
//          h for the layer above, and goes on to M_{l+1} . h_t^l as soon as all row tiles of its column tile have
//          arrived (the weights of that product are already in flight while it waits).
// Two workgroups per tile need twice as many resident workgroups as there are 32-column tiles; past that (more than 128
// columns of H = 1000 on 256 compute units) 64-column tiles halve the number of workgroups but leave compute units idle
// (192 columns: 192 workgroups) and double every link of the chain.  Between the two, while the 32-column tiles alone
// still fit, the schedule keeps them and fills the remaining compute units with HELPERS: a role-0 workgroup computes
// the W_h product of the lower layers itself (before M . x, so the wait for the layer below comes last), and each
// helper streams, for several tiles, first the upper part of Q and then the W_h products of the upper layers, layer by
// layer, in the order the chains will come for them (192 columns: 192 chains, 64 helpers of three tiles for layers 2
// and 3 -- 146 us against 168).
// (Four workgroups per tile at two per compute unit -- the chain sharing each compute unit with the backlog of
// independent products -- measured slower: 115 us against 106 at H = 1000, 128 columns, 4 layers; the epilogues and
// hand-overs of the chain take three times as long next to a wave that keeps the matrix pipe busy.)
// Hand-over, progress and bounded waits are those of lstm_sweep_kernel: device-scope stores and counters, a launch that
// must be wholly resident (the host checks), waits that give up after a poll limit, mark every counter and raise the
// status flag.  A finishing workgroup that gives up leaves NaN in the part of h and c it did not finish.  The last
// workgroup to leave returns the counters to zero for the next launch.
// ---------------------------------------------------------------------------------------------------------
struct LstmDecStack {
  const float* W[kMaxUnits];      // per layer: [nseg][4] packed fp32 matrices
  const float* bias[kMaxUnits];   // per layer: [4][H]
  const float* hprev[kMaxUnits];
  const float* cprev[kMaxUnits];
  float* h[kMaxUnits];
  float* c[kMaxUnits];
  const float* in0;               // layer 0 input: the H x V embedding when ids is set, else H x mb columns
  const int* ids;                 // [mb], already non-negative (null: in0 holds the columns themselves)
  const float* htild;             // previous attention output for layer 0's Q segment (null: none)
  const int* mask01;              // [mb]
  float* hp;                      // [nl] k-interleaved copies of h, H*mb floats each
  float* hp_top;                  // optional: the top layer's h k-interleaved, for the caller's next product
  float* partials;                // [nl][tile][visit][gate][thread]: role 1's sums
  int* counters;                  // [nl][tiles] tile flags, then [nl][n_tiles] layer counters at kSweepCtrStride
  int n_counters;                 // ints in `counters` (all of them are marked when a wait is abandoned)
  int* departures;                // workgroups that have left the kernel (zero at launch)
  int* status;
  int nl, V, H, mb, ldw, kp, j_tiles, n_tiles;
  float clip;
  int spin_limit;
  int fence;                      // as in LstmSweep
  int wait_extra;                 // arrivals a layer's wait for the layer below expects beyond the real ones (tests)
  int helpers;                    // 0: every tile has a role-1 workgroup of its own (grid.y = 2); else the number of
                                  // role-1 workgroups behind the chain slots of a one-dimensional grid
  int l_split;                    // role 1 delivers the independent products of layers l_split and up; below that a
                                  // role-0 workgroup computes its own
};

// All threads of the workgroup call this.  False: leave the kernel.
__device__ __forceinline__ bool stack_wait(const LstmDecStack& P, int* ctr, int target, int* s_go) {
  if (threadIdx.x == 0) {
    int v = __hip_atomic_load(ctr, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    for (int spins = 0; v < target && spins < P.spin_limit; ++spins) {
      __builtin_amdgcn_s_sleep(2);
      v = __hip_atomic_load(ctr, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    }
    const bool ok = v >= target && !(v & kSweepGaveUp);
    if (!ok) {
      if (!(v & kSweepGaveUp))
        for (int i = 0; i < P.n_counters; ++i) atomicOr(P.counters + i, kSweepGaveUp);
      __hip_atomic_store(P.status, 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    }
    *s_go = ok ? 1 : 0;
  }
  __syncthreads();
  const bool go = *s_go != 0;
  if (go && P.fence) __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "agent");
  return go;
}

template <int TN>
__global__ void __launch_bounds__(256) lstm_decoder_stack_kernel(LstmDecStack P) {
  constexpr int KS = 4;
  constexpr int PF = lstm_prefetch_depth(TN, KS);
  constexpr int NV = zr_visit_count<TN, KS>();
  __shared__ __align__(16) float red[KS * 4 * TN * 16 * 64];
  __shared__ int s_go[3];
  const int tid = threadIdx.x;

  auto work = [&]() {
    // Chain slots are placed die-aware as in lstm_fused_kernel; a tile's role-1 workgroup lands on the die of its
    // role-0 workgroup (gridDim.x % 8 == 0, helpers % 8 == 0).
    const int slots = P.helpers ? (int)gridDim.x - P.helpers : (int)gridDim.x;
    const int role = P.helpers ? ((int)blockIdx.x >= slots ? 1 : 0) : (int)blockIdx.y;
    const int per_die = (P.j_tiles + 7) >> 3;
    const int lane = tid & 63;
    const int kslice = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int H = P.H, mb = P.mb;
    const long long n_el = (long long)H * mb;
    const long long HH = (long long)P.kp * P.ldw;
    const int kgroups = H >> 3;
    // Q's K range is shared by the two roles: role 0 takes 9/16, so that role 1's sums of layer 0 (which still have
    // to travel) are there when role 0 comes for them
    const int q_split = (kgroups * 9) >> 4;
    const int tiles = P.j_tiles * P.n_tiles;
    int* layer_ctr = P.counters + P.nl * tiles;

    // Jobs.  Role 0: its tile, layer after layer.  Role 1: the independent products of layers l_split and up --
    // without helpers for its own tile (l_split = 0), as a helper for the tiles of chain slots w, w + helpers,
    // w + 2 helpers, ..., layer by layer, in the order the chain will come for them.
    const int first_slot = role == 0 ? (int)blockIdx.x : (P.helpers ? (int)blockIdx.x - slots : (int)blockIdx.x);
    const int slot_step = P.helpers ? P.helpers : slots;
    const int my_slots = role == 0 ? 1 : (slots - first_slot + slot_step - 1) / slot_step;
    const int l_first = role == 0 ? 0 : P.l_split;
    // (a helper's first jobs: the upper part of Q's K range for each of its tiles, when layer 0 has a Q)
    const int q_jobs = (role == 1 && P.helpers && P.htild) ? my_slots : 0;
    const int n_jobs = q_jobs + (P.nl - l_first) * my_slots;
    for (int job = 0; job < n_jobs; ++job) {
      const bool q_only = job < q_jobs;
      const int l = q_only ? 0 : l_first + (job - q_jobs) / my_slots;
      const int id = first_slot + ((q_only ? job : job - q_jobs) % my_slots) * slot_step;
      const int r8 = id & 7;
      const int q8 = id >> 3;
      const int nt = q8 % P.n_tiles;
      const int jt = r8 * per_die + q8 / P.n_tiles;
      if (q8 / P.n_tiles >= per_die || jt >= P.j_tiles) {  // a padding slot
        if (role == 0) return;
        continue;
      }
      const int j0 = jt * 32;
      const int n0 = nt * 32 * TN;
      const int tile = jt * P.n_tiles + nt;
      const bool covered = l >= P.l_split;  // role 1 (or a helper) delivers this layer's independent products

      // per-lane values are derived afresh in every job (see lstm_sweep_kernel)
      int lane_t = lane;
      asm volatile("" : "+v"(lane_t));
      const int jl = lane_t & 31, half = lane_t >> 5;
      const int j = j0 + jl;
      const bool j_ok = j < H;
      const int jc = j_ok ? j : H - 1;
      auto visit_col = [&](int i) {
        const int slot = zr_wide_visit_slot<KS>(kslice, i);
        const int tn = slot >> 4, r = slot & 15;
        const int n = n0 + tn * 32 + 8 * (r >> 2) + 4 * half + (r & 3);
        return n < mb ? n : mb - 1;
      };
      // A finishing workgroup that abandons a wait in layer l0 leaves NaN in its tile of h and c from that layer up
      // (role 1 never waits): whatever of the step's outputs was not finished cannot pass for a result.
      auto abandon = [&](int l0) {
        const float nan = __builtin_nanf("");
        for (int l2 = l0; l2 < P.nl; ++l2)
          for (int e = tid; e < 32 * 32 * TN; e += 256) {
            const int j2 = j0 + (e & 31), n2 = n0 + (e >> 5);
            if (j2 < H && n2 < mb) P.h[l2][(long long)n2 * H + j2] = nan, P.c[l2][(long long)n2 * H + j2] = nan;
          }
      };
      int cols[TN];
#pragma unroll
      for (int tn = 0; tn < TN; ++tn) {
        const int c = n0 + tn * 32 + jl;
        cols[tn] = c < mb ? c : mb - 1;
      }
      const unsigned woffb = 16u * (unsigned)(j + half * P.ldw);

      // epilogue operands of the finishing role go out ahead of the K loops
      float bi = 0.0f, bf = 0.0f, bc = 0.0f, bo = 0.0f, cprev_v[NV], mask_v[NV];
#pragma unroll
      for (int i = 0; i < NV; ++i) cprev_v[i] = 0.0f, mask_v[i] = 0.0f;
      if (role == 0) {
        const float* bias = P.bias[l];
        bi = bias[jc], bf = bias[H + jc], bc = bias[2 * H + jc], bo = bias[3 * H + jc];
#pragma unroll
        for (int i = 0; i < NV; ++i) {
          const int n = visit_col(i);
          cprev_v[i] = P.cprev[l][(long long)n * H + jc];
          mask_v[i] = (float)P.mask01[n];
        }
      }

      zr_f32x16 acc[4][TN];
#pragma unroll
      for (int g = 0; g < 4; ++g)
#pragma unroll
        for (int tn = 0; tn < TN; ++tn)
#pragma unroll
          for (int r = 0; r < 16; ++r) acc[g][tn][r] = 0.0f;

      // The products of this job, the one that may have to wait (M_l . h_t^{l-1}) last:
      //   role 1:                 W_h . h_{t-1}  [+ the upper part of Q's K range in layer 0]  (a helper's Q jobs: Q alone)
      //   role 0, covered layer:  [the lower part of Q]  + M . x
      //   role 0, layer it has to itself:  W_h . h_{t-1}  [+ the lower part of Q]  + M . x
      const bool has_q = l == 0 && P.htild != nullptr;
      const bool own_wh = role == 0 && !covered;
      const int n_wh = role == 1 ? (q_only ? 0 : 1) : (own_wh ? 1 : 0);
      const int nq = n_wh + (has_q ? 1 : 0) + (role == 0 ? 1 : 0);
      for (int q = 0; q < nq; ++q) {
        // s: the matrix (0 = M, 1 = W_h, 2 = Q)
        const int s = q < n_wh ? 1 : ((role == 0 && q == nq - 1) ? 0 : 2);
        int g0 = 0, g1 = kgroups;
        if (s == 2) {
          g0 = role ? q_split : 0;
          g1 = role ? kgroups : q_split;
        }
        const int K = (g1 - g0) * 8;
        const bool packed = s == 0 && l > 0;
        unsigned wsoff[4];
#pragma unroll
        for (int g = 0; g < 4; ++g) wsoff[g] = (unsigned)((((long long)s * 4 + g) * HH + (long long)g0 * 8 * P.ldw) * 4);
        ZrFrag<4, TN> ring[PF + 1];
        const __amdgpu_buffer_rsrc_t wrsrc = zr_make_rsrc(P.W[l]);
        zr_preload_w<4, TN, KS, PF>(ring, wrsrc, wsoff, woffb, 32u * (unsigned)P.ldw, K, kslice);
        if (packed) {
          if (!stack_wait(P, layer_ctr + ((l - 1) * P.n_tiles + nt) * kSweepCtrStride, P.j_tiles + P.wait_extra,
                          &s_go[0])) {
            abandon(l);
            return;
          }
        }
        const float* xb;
        unsigned xoffb[TN];
        if (packed) {
          xb = P.hp + (long long)(l - 1) * n_el;
#pragma unroll
          for (int tn = 0; tn < TN; ++tn) xoffb[tn] = 16u * ((unsigned)cols[tn] + (unsigned)(half * mb));
        } else {
          xb = s == 2 ? P.htild + g0 * 8 : (s == 1 ? P.hprev[l] : P.in0);
          const bool gather = s == 0 && P.ids != nullptr;
#pragma unroll
          for (int tn = 0; tn < TN; ++tn) {
            unsigned c = (unsigned)cols[tn];
            if (gather) {
              const int v = P.ids[cols[tn]];
              c = (unsigned)(v < 0 ? 0 : (v >= P.V ? P.V - 1 : v));
            }
            xoffb[tn] = 4u * (c * (unsigned)H + 4u * half);
          }
        }
        zr_mma_segment_u<4, TN, KS, PF, true>(acc, wrsrc, wsoff, woffb, 32u * (unsigned)P.ldw, zr_make_rsrc(xb), xoffb,
                                              packed ? 32u * (unsigned)mb : 32u, K, kslice, ring);
      }

      float* part = P.partials + ((long long)l * tiles + tile) * (NV * 4 * 256) + tid;
      int* flag = P.counters + l * tiles + tile;
      if (role == 1) {
        zr_reduce_visit_wide<4, TN, KS>(acc, red, kslice, lane, [&](const float(&z)[4], int, int, int vi) {
#pragma unroll
          for (int g = 0; g < 4; ++g)
            __hip_atomic_store(part + (vi * 4 + g) * 256, z[g], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        });
        zr_publish_barrier();
        if (tid == 0) atomicAdd(flag, 1);
        continue;
      }

      // role 0: the other role's sums (normally long there), fetched while this workgroup's partial tiles are summed
      float other[NV][4];
      if (covered || has_q) {
        if (!stack_wait(P, flag, 1, &s_go[1])) {
          abandon(l);
          return;
        }
#pragma unroll
        for (int vi = 0; vi < NV; ++vi)
#pragma unroll
          for (int g = 0; g < 4; ++g)
            other[vi][g] = __hip_atomic_load(part + (vi * 4 + g) * 256, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
      } else {
#pragma unroll
        for (int vi = 0; vi < NV; ++vi)
#pragma unroll
          for (int g = 0; g < 4; ++g) other[vi][g] = 0.0f;
      }
      const bool hand_on = l + 1 < P.nl;
      float* hp_out = P.hp + (long long)l * n_el;
      float h_v[NV], c_v[NV];
      zr_reduce_visit_wide<4, TN, KS>(acc, red, kslice, lane, [&](const float(&z)[4], int tn, int r, int vi) {
        const int n = n0 + tn * 32 + 8 * (r >> 2) + 4 * half + (r & 3);
        float gi, gf, gc, go;
        zr_lstm_cell((z[0] + other[vi][0]) + bi, (z[1] + other[vi][1]) + bf, (z[2] + other[vi][2]) + bc,
                     (z[3] + other[vi][3]) + bo, cprev_v[vi], mask_v[vi], P.clip, gi, gf, gc, go, c_v[vi], h_v[vi]);
        if (hand_on && j_ok && n < mb)
          __hip_atomic_store(hp_out + ((long long)(j >> 2) * mb + n) * 4 + (j & 3), h_v[vi], __ATOMIC_RELAXED,
                             __HIP_MEMORY_SCOPE_AGENT);
      });
      if (hand_on) {
        zr_publish_barrier();
        if (tid == 0) atomicAdd(layer_ctr + (l * P.n_tiles + nt) * kSweepCtrStride, 1);
      }
      float* h_out = P.h[l];
      float* c_out = P.c[l];
      float* hp_top = hand_on ? nullptr : P.hp_top;
#pragma unroll
      for (int i = 0; i < NV; ++i) {
        const int slot = zr_wide_visit_slot<KS>(kslice, i);
        const int n = n0 + (slot >> 4) * 32 + 8 * ((slot & 15) >> 2) + 4 * half + (slot & 3);
        if (j_ok && n < mb) {
          const long long ix = (long long)n * H + j;
          c_out[ix] = c_v[i];
          h_out[ix] = h_v[i];
          if (hp_top) hp_top[((long long)(j >> 2) * mb + n) * 4 + (j & 3)] = h_v[i];
        }
      }
    }
  };
  work();

  // Departure.  The last workgroup out returns the counters to zero for the next launch.
  __syncthreads();
  if (tid == 0) {
    const int total = (int)(gridDim.x * gridDim.y);
    const int before = __hip_atomic_fetch_add(P.departures, 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    s_go[2] = before == total - 1 ? 1 : 0;
  }
  __syncthreads();
  if (!s_go[2]) return;
  for (int i = tid; i < P.n_counters; i += 256) __hip_atomic_store(P.counters + i, 0, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
  if (tid == 0) __hip_atomic_store(P.departures, 0, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}

template <int TN, int KS>
int launch_fused_v(zr_ctx* ctx, const LstmLaunch& L, bool vec) {
  const int groups = L.n_units * L.j_tiles;
  const int grid = ((groups + 7) / 8) * 8 * L.n_tiles;
  if (L.bf16) {
    if constexpr (KS == 4 && TN <= 2) {
      bool xpk = true;  // every segment of every unit has pre-split inputs
      for (int i = 0; i < L.n_units; ++i)
        for (int s2 = 0; s2 < L.u[i].nseg; ++s2) xpk = xpk && L.u[i].inp[s2];  // (inp_lo null: single-term mode)
      if (xpk && L.bf16_single)
        lstm_fused_kernel<TN, KS, true, true, true, false, false, true><<<grid, 64 * KS, 0, ctx->stream>>>(L);
      else if (xpk)
        lstm_fused_kernel<TN, KS, true, true, true><<<grid, 64 * KS, 0, ctx->stream>>>(L);
      else if (L.bf16_single)
        lstm_fused_kernel<TN, KS, true, true, false, false, false, true><<<grid, 64 * KS, 0, ctx->stream>>>(L);
      else
        lstm_fused_kernel<TN, KS, true, true><<<grid, 64 * KS, 0, ctx->stream>>>(L);
      ZR_LAUNCH_CHECK("lstm_fused_kernel (bf16 weights)");
      return ZR_OK;
    } else {
      return zr_set_error(ZR_EINVAL, "bf16 weights: no kernel for column tile %d, K split %d", TN, KS);
    }
  }
  if (vec && L.buf_ok)
    lstm_fused_kernel<TN, KS, true, false, false, false, true><<<grid, 64 * KS, 0, ctx->stream>>>(L);
  else if (vec)
    lstm_fused_kernel<TN, KS, true><<<grid, 64 * KS, 0, ctx->stream>>>(L);
  else
    lstm_fused_kernel<TN, KS, false><<<grid, 64 * KS, 0, ctx->stream>>>(L);
  ZR_LAUNCH_CHECK("lstm_fused_kernel");
  return ZR_OK;
}

// Register-streaming kernel with K also split across `parts` workgroups per tile (SPLIT variant).
template <int TN>
int launch_fused_split(zr_ctx* ctx, LstmLaunch& L, int parts) {
  const int groups = L.n_units * L.j_tiles;
  const long long tiles = (long long)groups * L.n_tiles;
  constexpr int NV = zr_visit_count<TN, 4>();
  void* scratch = nullptr;
  int rc = zr_ctx_scratch(ctx, 0, sizeof(float) * (size_t)tiles * parts * NV * 4 * 256, &scratch);
  if (rc) return rc;
  L.kparts = parts;
  L.partials = (float*)scratch;
  L.counters = ctx->d_counters;
  dim3 grid((unsigned)(((groups + 7) / 8) * 8 * L.n_tiles), (unsigned)parts);
  if (L.buf_ok)
    lstm_fused_kernel<TN, 4, true, false, false, true, true><<<grid, 256, 0, ctx->stream>>>(L);
  else
    lstm_fused_kernel<TN, 4, true, false, false, true><<<grid, 256, 0, ctx->stream>>>(L);
  ZR_LAUNCH_CHECK("lstm_fused_kernel (K split across workgroups)");
  return ZR_OK;
}

template <int TN, int NWV>
int launch_lds_v(zr_ctx* ctx, LstmLaunch& L) {
  LstmLaunch2 P;
  L.n_tiles = (L.mb + 32 * TN * NWV - 1) / (32 * TN * NWV);
  const int tiles = L.n_units * L.j_tiles * L.n_tiles;
  P.n_chunks = (L.H + 31) / 32;
  int kparts = ctx->lstm_kparts;
  if (kparts == 0) {
    // about one workgroup per CU, not more: the finishing workgroup of a tile reads every partial, so its tail
    // grows with the number of splits
    kparts = 256 / (tiles * L.nseg_max);
    if (kparts > 8) kparts = 8;
  }
  if (kparts > P.n_chunks) kparts = P.n_chunks;
  if (kparts < 1) kparts = 1;
  P.kparts = kparts;
  const int splits = L.nseg_max * kparts;
  void* scratch = nullptr;
  const size_t bytes = sizeof(float) * (size_t)tiles * splits * NWV * (4 * TN * 16 * 64);
  int rc = zr_ctx_scratch(ctx, 0, bytes, &scratch);
  if (rc) return rc;
  P.partials = (float*)scratch;
  P.counters = ctx->d_counters;
  P.base = L;
  const int grid = ((tiles + 7) / 8) * 8 * splits;
  lstm_lds_kernel<TN, NWV><<<grid, 64 * NWV, 0, ctx->stream>>>(P);
  ZR_LAUNCH_CHECK("lstm_lds_kernel");
  return ZR_OK;
}

int launch_fused(zr_ctx* ctx, LstmLaunch& L, bool vec) {
  L.j_tiles = (L.H + 31) / 32;
  const int n32 = (L.mb + 31) / 32;
  L.nseg_max = 0;
  for (int i = 0; i < L.n_units; ++i) L.nseg_max = L.u[i].nseg > L.nseg_max ? L.u[i].nseg : L.nseg_max;
  {
    const long long lim = 1LL << 32;
    bool ok = vec && !L.bf16 && (L.H & 7) == 0 && (long long)L.H * L.mb * 4 < lim &&
              4LL * L.nseg_max * L.kp * L.ldw * 4 < lim;
    for (int i = 0; i < L.n_units; ++i) ok = ok && (!L.u[i].gather_ids || (long long)L.u[i].V * L.H * 4 < lim);
    L.buf_ok = ok ? 1 : 0;
  }
  // Kernel choice.  The register-streaming kernel needs no cross-workgroup reduction and wins whenever it can put
  // a workgroup on (nearly) every CU -- a full diagonal of an encoder does.  A single node (a decoder step) gives
  // it only ceil(H/32) * ceil(mb/64) workgroups; there K is split across workgroups too: by the same kernel's SPLIT
  // variant when H % 8 == 0, else by the LDS kernel (which needs a batch wide enough for its 128-column tile).
  if (L.bf16) {
    ZR_CHECK_ARG(vec && L.H % 16 == 0, "bf16 weights need H %% 16 == 0 and 16-byte aligned activations (H = %d)", L.H);
    const long long wg2 = (long long)L.n_units * L.j_tiles * ((n32 + 1) / 2);
    L.n_tiles = (n32 >= 2 && wg2 >= 200) ? (n32 + 1) / 2 : n32;
    return (n32 >= 2 && wg2 >= 200) ? launch_fused_v<2, 4>(ctx, L, vec) : launch_fused_v<1, 4>(ctx, L, vec);
  }
  int kernel = ctx->lstm_kernel;
  if (L.preact) kernel = 1;  // only the register-streaming kernel stores raw pre-activations
  // A launch that cannot put a whole-K tile on most CUs (a decoder node, the first and last diagonals of an encoder)
  // divides K across workgroups as well.
  const long long wgs_whole_k = (long long)L.n_units * L.j_tiles * ((n32 + 1) / 2);
  if (kernel == 0 && vec && (L.H & 7) == 0 && wgs_whole_k < 200) kernel = 3;
  if (kernel == 3 && vec && (L.H & 7) == 0) {
    // 32-column tiles and as few K parts as fill the chip: measured on four decoder nodes of H = 1000 against wider
    // tiles with more parts, 119 us against 138 at 128 columns, 88 against 117 at 64 (a short K range per workgroup
    // never gets its operand pipeline going, and the cross-workgroup sum grows with the parts); when the tiles alone
    // fill the chip no split is made at all (167 against 181 us at 192 columns, 172 against 191 at 256)
    int tn = 1;
    if (ctx->lstm_tn == 2 && n32 >= 2) tn = 2;                   // tuning runs
    if (ctx->lstm_tn == 4 && n32 % 3 == 0) tn = 3;
    L.n_tiles = (n32 + tn - 1) / tn;
    const long long tiles = (long long)L.n_units * L.j_tiles * L.n_tiles;
    int parts = ctx->lstm_kparts;
    if (parts == 0) {
      parts = (int)((256 + tiles / 2) / tiles);
      const int max_parts = (L.H >> 3) / 16;  // at least 16 k-groups per part (4 per wave)
      if (parts > max_parts) parts = max_parts;
      if (parts > 8) parts = 8;
    }
    if (parts >= 2 && tiles <= ZR_MAX_COUNTERS && parts <= (L.H >> 3)) {
      if (tn == 3) return launch_fused_split<3>(ctx, L, parts);
      if (tn == 2) return launch_fused_split<2>(ctx, L, parts);
      return launch_fused_split<1>(ctx, L, parts);
    }
    // no useful split for this shape (e.g. 192 whole-K tiles): one tile per CU on most CUs beats the LDS kernel
    kernel = 1;
  }
  if (kernel == 3) kernel = 0;  // needs 16-byte aligned operands and H % 8 == 0
  if (kernel == 0) kernel = (vec && n32 >= 3 && wgs_whole_k < 200) ? 2 : 1;
  if (kernel == 2 && vec && L.n_units * L.j_tiles * ((n32 + 3) / 4) <= ZR_MAX_COUNTERS) {
    if (n32 > 4 && ctx->lstm_tn == 2) return launch_lds_v<2, 4>(ctx, L);
    return launch_lds_v<1, 4>(ctx, L);
  }
  int tn = ctx->lstm_tn;
  if (tn == 0) {
    // 64-column tiles once they occupy more than half the CUs: 32-column tiles would then need two rounds of
    // workgroups, which costs more than one round of the wider tile
    tn = 1;
    const int groups = L.n_units * L.j_tiles;
    if (n32 >= 2 && (long long)groups * ((n32 + 1) / 2) > 128) tn = 2;
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


// Resident workgroups of lstm_sweep_kernel<TN> the device can hold at once (0: unknown / query failed).
template <int TN>
int sweep_capacity(zr_ctx* ctx) {
  int& cached = ctx->sweep_capacity[TN];
  if (cached == 0) {
    int cus = 0, per_cu = 0;
    if (hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, ctx->device) != hipSuccess ||
        hipOccupancyMaxActiveBlocksPerMultiprocessor(&per_cu, lstm_sweep_kernel<TN>, 256, 0) != hipSuccess) {
      (void)hipGetLastError();
      cached = -1;
    } else {
      ctx->cu_count = cus;
      cached = cus * per_cu > 0 ? cus * per_cu : -1;
    }
  }
  return cached > 0 ? cached : 0;
}

// Runs right behind lstm_sweep_kernel.  A sweep whose workgroups gave up a wait leaves part of h_all / c_all
// unwritten; whatever is queued behind it on the stream would read stale memory.  When the status flag is up this
// kernel overwrites every output of the sweep with NaN, so that nothing downstream can pass for a result; when it
// is down (always, in practice) every workgroup reads one word and leaves.
struct SweepPoison {
  float* out[3 * kMaxUnits];  // h_all, c_all and (where kept) gates_all of every layer
  long long count[3 * kMaxUnits];
  int n_out;
  const int* status;
};

__global__ void __launch_bounds__(256) lstm_sweep_poison_kernel(SweepPoison P) {
  if (__hip_atomic_load(P.status, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) == 0) return;
  const float nan = __builtin_nanf("");
  const long long stride = (long long)gridDim.x * 256;
  for (int a = 0; a < P.n_out; ++a)
    for (long long i = (long long)blockIdx.x * 256 + threadIdx.x; i < P.count[a]; i += stride) P.out[a][i] = nan;
}

template <int TN>
int launch_sweep_v(zr_ctx* ctx, LstmSweep& P, int grid) {
  lstm_sweep_kernel<TN><<<grid, 256, 0, ctx->stream>>>(P);
  ZR_LAUNCH_CHECK("lstm_sweep_kernel");
  SweepPoison Q = {};
  const long long per = (long long)P.T * P.H * P.mb;
  for (int l = 0; l < P.nl; ++l) {
    Q.out[Q.n_out] = P.h_all[l], Q.count[Q.n_out++] = per;
    Q.out[Q.n_out] = P.c_all[l], Q.count[Q.n_out++] = per;
    if (P.gates_all[l]) Q.out[Q.n_out] = P.gates_all[l], Q.count[Q.n_out++] = 4 * per;
  }
  Q.status = P.status;
  lstm_sweep_poison_kernel<<<512, 256, 0, ctx->stream>>>(Q);
  ZR_LAUNCH_CHECK("lstm_sweep_poison_kernel");
  return ZR_OK;
}

// Resident workgroups of lstm_decoder_stack_kernel (either tile width) the device can hold at once (0: unknown /
// query failed).
int stack_step_capacity(zr_ctx* ctx) {
  int& cached = ctx->stack_step_capacity;
  if (cached == 0) {
    int cus = 0, per_cu = 0, per_cu2 = 0;
    if (hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, ctx->device) != hipSuccess ||
        hipOccupancyMaxActiveBlocksPerMultiprocessor(&per_cu, lstm_decoder_stack_kernel<1>, 256, 0) != hipSuccess ||
        hipOccupancyMaxActiveBlocksPerMultiprocessor(&per_cu2, lstm_decoder_stack_kernel<2>, 256, 0) != hipSuccess) {
      (void)hipGetLastError();
      cached = -1;
    } else {
      per_cu = per_cu2 < per_cu ? per_cu2 : per_cu;
      ctx->cu_count = cus;
      cached = cus * per_cu > 0 ? cus * per_cu : -1;
    }
  }
  return cached > 0 ? cached : 0;
}

inline bool aligned16(const void* p) { return ((uintptr_t)p & 15u) == 0; }

}  // namespace

extern "C" {

static int pack_weights(zr_ctx* ctx, const char* who, bool bf16, const float* const d_M[4],
                        const float* const d_Wh[4], const float* const d_Q[4], const float* const d_b[4], int H,
                        zr_lstm_weights** out) {
  int rc = zr_bind_device(ctx);
  if (rc) return rc;
  ZR_CHECK_ARG(out != nullptr, "%s: out is null", who);
  *out = nullptr;
  ZR_CHECK_ARG(H > 0, "%s: H = %d", who, H);
  ZR_CHECK_ARG(!bf16 || H % 16 == 0, "%s: H = %d is not a multiple of 16", who, H);
  ZR_CHECK_ARG(d_M && d_Wh && d_b, "%s: null pointer array", who);
  for (int g = 0; g < 4; ++g) {
    ZR_CHECK_ARG(d_M[g] && d_Wh[g] && d_b[g], "%s: null matrix for gate %d", who, g);
    ZR_CHECK_ARG(!d_Q || d_Q[g], "%s: null Q for gate %d", who, g);
  }
  const int nseg = d_Q ? 3 : 2;
  const int ldw = (H + 31) / 32 * 32;
  const int kp = bf16 ? (H + 15) / 16 * 16 : (H + 7) / 8 * 8;
  const size_t HH = (size_t)kp * ldw;
  const size_t esize = bf16 ? sizeof(unsigned short) : sizeof(float);
  zr_lstm_weights* w = new zr_lstm_weights();
  w->H = H;
  w->bf16 = bf16 ? 1 : 0;
  w->ldw = ldw;
  w->kp = kp;
  w->nseg = nseg;
  w->d_W = nullptr;
  w->d_bias = nullptr;
  if (hipMalloc((void**)&w->d_W, esize * HH * 4 * nseg) != hipSuccess ||
      hipMalloc((void**)&w->d_bias, sizeof(float) * 4 * (size_t)H) != hipSuccess) {
    (void)hipGetLastError();
    if (w->d_W) (void)hipFree(w->d_W);
    delete w;
    return zr_set_error(ZR_ENOMEM, "%s: allocation failed (H = %d, nseg = %d)", who, H, nseg);
  }
  for (int g = 0; g < 4; ++g) {
    const float* segs[3] = {d_M[g], d_Wh[g], d_Q ? d_Q[g] : nullptr};
    for (int s = 0; s < nseg; ++s) {
      const size_t off = ((size_t)s * 4 + g) * HH;
      rc = bf16 ? zr_pack8_bf16_launch(ctx, segs[s], H, H, H, ldw, kp, (unsigned short*)w->d_W + off)
                : zr_pack4_launch(ctx, segs[s], H, H, H, ldw, kp, (float*)w->d_W + off);
      if (rc != ZR_OK) {
        (void)hipFree(w->d_W);
        (void)hipFree(w->d_bias);
        delete w;
        return ZR_EHIP;
      }
    }
    hipError_t e = hipMemcpyAsync(w->d_bias + (size_t)g * H, d_b[g], sizeof(float) * H, hipMemcpyDeviceToDevice,
                                  ctx->stream);
    if (e != hipSuccess) {
      (void)hipFree(w->d_W);
      (void)hipFree(w->d_bias);
      delete w;
      return zr_set_error(ZR_EHIP, "%s: bias copy failed: %s", who, hipGetErrorString(e));
    }
  }
  *out = w;
  return ZR_OK;
}

int zr_lstm_pack_weights(zr_ctx* ctx, const float* const d_M[4], const float* const d_Wh[4],
                         const float* const d_Q[4], const float* const d_b[4], int H, zr_lstm_weights** out) {
  return pack_weights(ctx, "zr_lstm_pack_weights", false, d_M, d_Wh, d_Q, d_b, H, out);
}

int zr_lstm_pack_weights_bf16(zr_ctx* ctx, const float* const d_M[4], const float* const d_Wh[4],
                              const float* const d_Q[4], const float* const d_b[4], int H, zr_lstm_weights** out) {
  return pack_weights(ctx, "zr_lstm_pack_weights_bf16", true, d_M, d_Wh, d_Q, d_b, H, out);
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

static int lstm_step_impl(zr_ctx* ctx, const zr_lstm_weights* w, const float* d_in, const int* d_gather_ids, int V,
                          const float* d_hprev, const float* d_cprev, const float* d_htild, const int* d_mask01,
                          float clip_threshold, int mb, float* d_h, float* d_c, float* const d_gates[4],
                          const unsigned short* const* pre_hi = nullptr, const unsigned short* const* pre_lo = nullptr,
                          unsigned short* out_hi = nullptr, unsigned short* out_lo = nullptr, float* out_hp = nullptr);

int zr_lstm_step(zr_ctx* ctx, const zr_lstm_weights* w, const float* d_in, const float* d_hprev,
                 const float* d_cprev, const float* d_htild, const int* d_mask01, float clip_threshold, int mb,
                 float* d_h, float* d_c, float* const d_gates[4]) {
  return lstm_step_impl(ctx, w, d_in, nullptr, 0, d_hprev, d_cprev, d_htild, d_mask01, clip_threshold, mb, d_h, d_c,
                        d_gates);
}

int zr_lstm_step_embed(zr_ctx* ctx, const zr_lstm_weights* w, const float* d_embed, int V, const int* d_ids_nonneg,
                       const float* d_hprev, const float* d_cprev, const float* d_htild, const int* d_mask01,
                       float clip_threshold, int mb, float* d_h, float* d_c, float* const d_gates[4]) {
  ZR_CHECK_ARG(V > 0 && d_ids_nonneg != nullptr, "zr_lstm_step_embed: V = %d or null token ids", V);
  return lstm_step_impl(ctx, w, d_embed, d_ids_nonneg, V, d_hprev, d_cprev, d_htild, d_mask01, clip_threshold, mb, d_h,
                        d_c, d_gates);
}

// d_gather_ids non-null: d_in is the H x V embedding and column b of the input is d_in[:, d_gather_ids[b]].
// pre_hi / pre_lo (or null; bf16 weights only): segment s's input already split into bf16 terms and k-interleaved by 8
// (pre_lo[s] null in single-term mode); such a segment is neither gathered nor split here.  out_hi / out_lo (or null):
// h is also written in that form, for the product that reads it next.  out_hp (or null; fp32 weights, fused epilogue):
// h is also written k-interleaved ([H/4][mb][4]).
static int lstm_step_impl(zr_ctx* ctx, const zr_lstm_weights* w, const float* d_in, const int* d_gather_ids, int V,
                          const float* d_hprev, const float* d_cprev, const float* d_htild, const int* d_mask01,
                          float clip_threshold, int mb, float* d_h, float* d_c, float* const d_gates[4],
                          const unsigned short* const* pre_hi, const unsigned short* const* pre_lo,
                          unsigned short* out_hi, unsigned short* out_lo, float* out_hp) {
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
  const bool two_terms = ctx->bf16_terms != 1;
  auto presplit = [&](int sg) { return w->bf16 && pre_hi && pre_hi[sg] && (!two_terms || (pre_lo && pre_lo[sg])); };
  if (d_gather_ids && presplit(0)) d_gather_ids = nullptr;  // the split columns are the gathered ones
  if (d_gather_ids && (w->bf16 || !ctx->lstm_fused)) {
    // these paths re-lay-out or re-read their inputs as whole matrices: gather the columns first
    void* x = nullptr;
    rc = zr_ctx_scratch(ctx, 1, sizeof(float) * (size_t)H * mb * (ctx->lstm_fused ? 1 : 5), &x);
    if (rc) return rc;
    float* xg = (float*)x + (ctx->lstm_fused ? 0 : 4 * (size_t)H * mb);  // behind the pre-activation planes
    rc = zr_embed_gather(ctx, d_in, H, V, d_gather_ids, mb, xg);
    if (rc) return rc;
    d_in = xg;
    d_gather_ids = nullptr;
  }

  LstmLaunch L = {};
  L.n_units = 1;
  L.H = H;
  L.mb = mb;
  L.ldw = w->ldw;
  L.kp = w->kp;
  L.bf16 = w->bf16;
  L.bf16_single = ctx->bf16_terms == 1;
  L.clip = clip_threshold;
  LstmUnit& U = L.u[0];
  U.W = w->d_W;
  U.bias = w->d_bias;
  U.in[0] = d_in;
  U.in[1] = d_hprev;
  U.in[2] = d_htild;
  U.gather_ids = d_gather_ids;
  U.cprev = d_cprev;
  U.mask01 = d_mask01;
  U.h = d_h;
  U.c = d_c;
  U.hp = (ctx->lstm_fused && !w->bf16) ? out_hp : nullptr;
  U.hsplit_hi = (ctx->lstm_fused && H % 8 == 0) ? out_hi : nullptr;
  U.hsplit_lo = U.hsplit_hi ? out_lo : nullptr;
  for (int g = 0; g < 4; ++g) U.gates[g] = d_gates ? d_gates[g] : nullptr;
  U.nseg = nseg;
  U.V = d_gather_ids ? V : 0;
  const bool vec = (H % 4 == 0) && aligned16(d_in) && aligned16(d_hprev) && (!d_htild || aligned16(d_htild));
  if (w->bf16 && vec) {
    // split the fp32 inputs into bf16 hi + lo once per node, k-interleaved, instead of in every workgroup's K loop
    void* p = nullptr;
    const size_t e = (size_t)H * mb;
    rc = zr_ctx_scratch(ctx, 0, sizeof(unsigned short) * 2 * e * nseg, &p);
    if (rc) return rc;
    unsigned short* hi = (unsigned short*)p;
    for (int s = 0; s < nseg; ++s) {
      const bool lo = two_terms;
      if (presplit(s)) {
        U.inp[s] = (const float*)pre_hi[s];
        U.inp_lo[s] = lo ? pre_lo[s] : nullptr;
        continue;
      }
      rc = zr_split_pack_x_launch(ctx, U.in[s], H, mb, H, hi, lo ? hi + e : nullptr);
      if (rc) return rc;
      U.inp[s] = (const float*)hi;
      U.inp_lo[s] = lo ? hi + e : nullptr;
      hi += 2 * e;
    }
  }
  if (!ctx->lstm_fused) {
    // reference-shaped two-phase path: the four pre-activation sums go to memory, then the stand-alone fused gate
    // kernel (the reference's element-wise kernels in one pass) adds the biases and runs the cell
    void* pre = nullptr;
    rc = zr_ctx_scratch(ctx, 1, sizeof(float) * 4 * (size_t)H * mb, &pre);
    if (rc) return rc;
    L.preact = (float*)pre;
    rc = launch_fused(ctx, L, vec);
    if (rc) return rc;
    const float* b[4] = {w->d_bias, w->d_bias + H, w->d_bias + 2 * (size_t)H, w->d_bias + 3 * (size_t)H};
    return zr_lstm_gates(ctx, (const float*)pre, b, d_cprev, d_mask01, clip_threshold, H, mb, d_h, d_c, d_gates);
  }
  return launch_fused(ctx, L, vec);
}

int zr_lstm_decoder_step(zr_ctx* ctx, int nl, const zr_lstm_weights* const layers[], const float* d_embed, int V,
                         const int* d_ids_nonneg, const float* const d_hprev[], const float* const d_cprev[],
                         const float* d_htild, const int* d_mask01, float clip_threshold, int mb,
                         float* const d_h[], float* const d_c[]) {
  return zr_lstm_decoder_step_packed(ctx, nl, layers, d_embed, V, d_ids_nonneg, d_hprev, d_cprev, d_htild, d_mask01,
                                     clip_threshold, mb, d_h, d_c, nullptr, nullptr);
}

}  // extern "C"

int zr_lstm_decoder_step_packed(zr_ctx* ctx, int nl, const zr_lstm_weights* const layers[], const float* d_embed, int V,
                                const int* d_ids_nonneg, const float* const d_hprev[], const float* const d_cprev[],
                                const float* d_htild, const int* d_mask01, float clip_threshold, int mb,
                                float* const d_h[], float* const d_c[], float* d_hp_top, int* wrote_hp_top) {
  if (wrote_hp_top) *wrote_hp_top = 0;
  int rc = zr_bind_device(ctx);
  if (rc) return rc;
  ZR_CHECK_ARG(nl > 0 && nl <= kMaxUnits && mb > 0 && V > 0, "zr_lstm_decoder_step: L = %d, mb = %d, V = %d", nl, mb, V);
  ZR_CHECK_ARG(layers && d_embed && d_ids_nonneg && d_hprev && d_cprev && d_mask01 && d_h && d_c,
               "zr_lstm_decoder_step: null pointer");
  const int H = layers[0] ? layers[0]->H : 0;
  bool vec = (H > 0) && (H % 4 == 0) && aligned16(d_embed) && (!d_htild || aligned16(d_htild));
  for (int l = 0; l < nl; ++l) {
    ZR_CHECK_ARG(layers[l] && layers[l]->H == H, "zr_lstm_decoder_step: layer %d missing or of different size", l);
    ZR_CHECK_ARG(layers[l]->bf16 == layers[0]->bf16, "zr_lstm_decoder_step: layers mix fp32 and bf16 weights");
    ZR_CHECK_ARG(d_hprev[l] && d_cprev[l] && d_h[l] && d_c[l], "zr_lstm_decoder_step: null state for layer %d", l);
    ZR_CHECK_ARG(d_h[l] != d_htild, "zr_lstm_decoder_step: d_h[%d] aliases d_htild", l);
    for (int m = 0; m < nl; ++m) {
      ZR_CHECK_ARG(d_h[l] != d_hprev[m] && (l == m || d_h[l] != d_h[m]),
                   "zr_lstm_decoder_step: d_h[%d] aliases another state array", l);
      // the cell state may be updated in place (d_c[l] == d_cprev[l]: each element is read and written by one thread);
      // anything else a workgroup of another tile or layer reads while this one writes may not be d_c[l]
      ZR_CHECK_ARG(d_c[l] != d_hprev[m] && d_c[l] != d_h[m] && (l == m || (d_c[l] != d_c[m] && d_c[l] != d_cprev[m])),
                   "zr_lstm_decoder_step: d_c[%d] aliases another state array", l);
    }
    ZR_CHECK_ARG(d_c[l] != d_htild, "zr_lstm_decoder_step: d_c[%d] aliases d_htild", l);
    vec = vec && aligned16(d_hprev[l]);
  }
  ZR_CHECK_ARG(!d_htild || layers[0]->nseg == 3, "zr_lstm_decoder_step: d_htild given but layer 0 was packed without Q");
  const size_t n = (size_t)H * mb;

  // One launch for the whole step when two workgroups per tile fit on the device together (the same conditions as the
  // single-launch sweep of zr_lstm_stack_forward); otherwise one node after the other.
  if (vec && H % 8 == 0 && H >= 64 && !layers[0]->bf16 && ctx->lstm_fused && ctx->lstm_sweep != 1) {
    const int j_tiles = (H + 31) / 32;
    const int padded = (j_tiles + 7) / 8 * 8;
    const int cap = stack_step_capacity(ctx);
    // 32-column tiles while two workgroups per tile fit on the device together; beyond that, while the 32-column tiles
    // alone still fit, 32-column tiles whose role-1 work of the UPPER layers goes to as many helper workgroups as still
    // fit, several tiles each, while a role-0 workgroup computes the independent products of the lower layers itself
    // (192 columns of H = 1000: 192 chains and 64 helpers of three tiles x two layers fill the 256 compute units);
    // else 64-column tiles in pairs
    const int slots1 = padded * ((mb + 31) / 32);
    int tn = (2LL * slots1 <= cap) ? 1 : 2;
    int helpers = 0, l_split = 0;
    if (tn == 2 && slots1 < cap && ctx->stack_helpers) {
      int hn = cap - slots1 < slots1 ? cap - slots1 : slots1;
      hn &= ~7;
      const int covered = hn > 0 ? (2 * nl * hn) / (slots1 + hn) : 0;
      // (only when the helpers take at least half of the layers: at 224 columns, 32 helpers of seven tiles for the top
      // layer alone, the step measured 206 us against 168 on 64-column tiles; at 160 and 192 columns 136 and 146)
      if (covered >= 1 && 2 * covered >= nl) {
        tn = 1;
        helpers = hn;
        l_split = nl - (covered < nl ? covered : nl);
      }
    }
    const int n_tiles = (mb + 32 * tn - 1) / (32 * tn);
    const long long tiles = (long long)j_tiles * n_tiles;
    const long long wgs = helpers ? (long long)padded * n_tiles + helpers : 2LL * padded * n_tiles;
    const bool fills = wgs * 10 >= 6LL * ctx->cu_count && zr_live_contexts(ctx->device) == 1 &&
                       ctx->stream == ctx->own_stream;
    const long long lim = 1LL << 32;
    const bool offsets_fit = (long long)V * H * 4 < lim && (long long)n * 4 < lim &&
                             12LL * layers[0]->kp * layers[0]->ldw * 4 < lim;
    const long long n_counters = nl * tiles + (long long)nl * n_tiles * kSweepCtrStride;
    if (cap > 0 && wgs <= cap && offsets_fit && n_counters < ZR_MAX_COUNTERS && (fills || ctx->lstm_sweep == 2)) {
      const int NV = tn == 1 ? zr_visit_count<1, 4>() : zr_visit_count<2, 4>();
      LstmDecStack P = {};
      void* p = nullptr;
      const size_t hp_bytes = sizeof(float) * (size_t)nl * n;
      rc = zr_ctx_scratch(ctx, 1, hp_bytes + sizeof(float) * (size_t)nl * tiles * NV * 4 * 256, &p);
      if (rc) return rc;
      P.hp = (float*)p;
      P.partials = (float*)((char*)p + hp_bytes);
      P.counters = ctx->d_counters;
      P.n_counters = (int)n_counters;
      P.departures = ctx->d_counters + (ZR_MAX_COUNTERS - 1);
      for (int l = 0; l < nl; ++l) {
        P.W[l] = (const float*)layers[l]->d_W;
        P.bias[l] = layers[l]->d_bias;
        P.hprev[l] = d_hprev[l];
        P.cprev[l] = d_cprev[l];
        P.h[l] = d_h[l];
        P.c[l] = d_c[l];
      }
      P.in0 = d_embed;
      P.ids = d_ids_nonneg;
      P.hp_top = d_hp_top;
      if (wrote_hp_top && d_hp_top) *wrote_hp_top = 1;
      P.htild = d_htild;
      P.mask01 = d_mask01;
      P.status = ctx->d_flags + 2;
      P.nl = nl;
      P.V = V;
      P.H = H;
      P.mb = mb;
      P.ldw = layers[0]->ldw;
      P.kp = layers[0]->kp;
      P.j_tiles = j_tiles;
      P.n_tiles = n_tiles;
      P.clip = clip_threshold;
      P.spin_limit = ctx->sweep_spin > 0 ? ctx->sweep_spin : (1 << 20);
      P.fence = (mb % 8 == 0) ? 0 : 1;
      P.wait_extra = ctx->step_wait_extra;
      P.helpers = helpers;
      P.l_split = l_split;
      ctx->last_stack_path = ZR_LSTM_STACK_PATH_STEP_SINGLE_LAUNCH;
      const dim3 grid((unsigned)(padded * n_tiles + helpers), helpers ? 1u : 2u);
      if (tn == 1)
        lstm_decoder_stack_kernel<1><<<grid, 256, 0, ctx->stream>>>(P);
      else
        lstm_decoder_stack_kernel<2><<<grid, 256, 0, ctx->stream>>>(P);
      ZR_LAUNCH_CHECK("lstm_decoder_stack_kernel");
      return ZR_OK;
    }
  }
  ctx->last_stack_path = ZR_LSTM_STACK_PATH_STEP_PER_LAYER;
  if (layers[0]->bf16 && vec && ctx->lstm_fused && nl + 2 <= 12) {
    // bf16 weights: every product input enters as bf16 terms, k-interleaved.  Everything the step knows at its start --
    // the embedding columns of the current words, h_{t-1} of every layer, the previous attention output -- is split in
    // ONE launch (as launches of their own these nl + 2 small kernels, and the gather in front of the first, cost more
    // in launch latency than in work); only h_t of the layer below is split between the layers.
    const bool two_terms = ctx->bf16_terms != 1;
    const size_t e = n;  // bf16 elements per array
    void* p = nullptr;
    rc = zr_ctx_scratch(ctx, 1, sizeof(unsigned short) * 2 * e * (size_t)(nl + 3), &p);
    if (rc) return rc;
    unsigned short* hi = (unsigned short*)p;
    unsigned short* lo = hi + e * (size_t)(nl + 3);
    const float* srcs[12];
    int ns = 0;
    srcs[ns++] = d_embed;  // matrix 0: gathered by the word ids
    for (int l = 0; l < nl; ++l) srcs[ns++] = d_hprev[l];
    if (d_htild) srcs[ns++] = d_htild;
    rc = zr_split_pack_multi_launch(ctx, ns, srcs, d_ids_nonneg, V, H, mb, H, hi, two_terms ? lo : nullptr, (long long)e);
    if (rc) return rc;
    // h_t of a layer leaves its launch in both forms: fp32 for the caller and bf16 terms for the layer above (two
    // buffers in turn: a launch reads one while it writes the other) or, from the top layer, for the caller's next
    // product (d_hp_top: hi terms, then H*mb elements further the lo terms)
    // (the second of the two is the embedding columns' slot, free once layer 0 has run)
    unsigned short* below_hi[2] = {hi + e * (size_t)(nl + 2), hi};
    unsigned short* below_lo[2] = {lo + e * (size_t)(nl + 2), lo};
    unsigned short* top_hi = (unsigned short*)d_hp_top;
    unsigned short* top_lo = top_hi ? top_hi + e : nullptr;
    for (int l = 0; l < nl; ++l) {
      const unsigned short* in_hi = l == 0 ? hi : below_hi[(l - 1) & 1];
      const unsigned short* in_lo = l == 0 ? lo : below_lo[(l - 1) & 1];
      const unsigned short* ph[3] = {in_hi, hi + e * (size_t)(1 + l), hi + e * (size_t)(1 + nl)};
      const unsigned short* pl[3] = {in_lo, lo + e * (size_t)(1 + l), lo + e * (size_t)(1 + nl)};
      const bool last = l == nl - 1;
      unsigned short* oh = last ? top_hi : below_hi[l & 1];
      unsigned short* ol = last ? top_lo : below_lo[l & 1];
      rc = lstm_step_impl(ctx, layers[l], l == 0 ? d_embed : d_h[l - 1], l == 0 ? d_ids_nonneg : nullptr, l == 0 ? V : 0,
                          d_hprev[l], d_cprev[l], l == 0 ? d_htild : nullptr, d_mask01, clip_threshold, mb, d_h[l],
                          d_c[l], nullptr, ph, two_terms ? pl : nullptr, oh, two_terms ? ol : nullptr);
      if (rc) return rc;
    }
    if (wrote_hp_top && top_hi) *wrote_hp_top = 1;
    return ZR_OK;
  }
  // (the top layer also leaves its h k-interleaved for the caller's next product, as the single launch does)
  float* top_hp = (!layers[0]->bf16 && ctx->lstm_fused && H % 8 == 0) ? d_hp_top : nullptr;
  for (int l = 0; l < nl; ++l) {
    float* hp_out = l == nl - 1 ? top_hp : nullptr;
    if (l == 0)
      rc = lstm_step_impl(ctx, layers[0], d_embed, d_ids_nonneg, V, d_hprev[0], d_cprev[0], d_htild, d_mask01,
                          clip_threshold, mb, d_h[0], d_c[0], nullptr, nullptr, nullptr, nullptr, nullptr, hp_out);
    else
      rc = lstm_step_impl(ctx, layers[l], d_h[l - 1], nullptr, 0, d_hprev[l], d_cprev[l], nullptr, d_mask01,
                          clip_threshold, mb, d_h[l], d_c[l], nullptr, nullptr, nullptr, nullptr, nullptr, hp_out);
    if (rc) return rc;
  }
  if (wrote_hp_top && top_hp) *wrote_hp_top = 1;
  return ZR_OK;
}

extern "C" {

int zr_lstm_stack_forward(zr_ctx* ctx, int nl, const zr_lstm_weights* const layers[], const float* d_embed, int V,
                          const int* d_ids_nonneg, const int* d_mask01, int T, int mb,
                          const float* const d_h0[], const float* const d_c0[], float clip_threshold,
                          float* const d_h_all[], float* const d_c_all[]) {
  return zr_lstm_stack_forward_train(ctx, nl, layers, d_embed, V, d_ids_nonneg, d_mask01, T, mb, d_h0, d_c0,
                                     clip_threshold, d_h_all, d_c_all, nullptr);
}

int zr_lstm_stack_forward_train(zr_ctx* ctx, int nl, const zr_lstm_weights* const layers[], const float* d_embed,
                                int V, const int* d_ids_nonneg, const int* d_mask01, int T, int mb,
                                const float* const d_h0[], const float* const d_c0[], float clip_threshold,
                                float* const d_h_all[], float* const d_c_all[], float* const d_gates_all[]) {
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
    ZR_CHECK_ARG(layers[l]->bf16 == layers[0]->bf16, "zr_lstm_stack_forward: layers mix fp32 and bf16 weights");
    ZR_CHECK_ARG(d_h0[l] && d_c0[l] && d_h_all[l] && d_c_all[l], "zr_lstm_stack_forward: null state for layer %d", l);
    vec = vec && aligned16(d_h0[l]) && aligned16(d_h_all[l]);
  }
  const size_t n = (size_t)H * mb;
  // One launch for the whole sweep when its workgroups -- one tile of one layer each, kept for all T steps -- fill
  // most of the chip and fit on it together; otherwise one launch per diagonal.
  if (vec && H % 8 == 0 && !layers[0]->bf16 && ctx->lstm_fused && ctx->lstm_sweep != 1 && nl <= kMaxUnits) {
    const int j_tiles = (H + 31) / 32, n32 = (mb + 31) / 32;
    const int groups = nl * j_tiles;
    const int padded = (groups + 7) / 8 * 8;
    int tn = 0;
    if ((long long)padded * n32 <= sweep_capacity<1>(ctx)) tn = 1;
    else if ((long long)padded * ((n32 + 1) / 2) <= sweep_capacity<2>(ctx)) tn = 2;
    const int n_tiles = tn ? (n32 + tn - 1) / tn : 0;
    const long long tiles = (long long)groups * n_tiles;
    // Left to itself the library takes the single launch only when it fills most of the chip and this is the only
    // context on the device: two such launches from two streams could each hold part of the CUs and wait for the
    // rest (their bounded waits would end it, with an error).
    // Nor on a caller-provided stream: the caller's other streams may hold compute units for as long as they like.
    const bool fills = tn && tiles * 10 >= 6LL * ctx->cu_count && zr_live_contexts(ctx->device) == 1 &&
                       ctx->stream == ctx->own_stream;
    // the kernel addresses its operands as descriptor base + 32-bit byte offsets
    const long long lim = 1LL << 32;
    const bool offsets_fit = (long long)V * H * 4 < lim && (long long)n * 4 < lim &&
                             8LL * layers[0]->kp * layers[0]->ldw * 4 < lim;
    if (tn && offsets_fit && (fills || ctx->lstm_sweep == 2) && nl * n_tiles <= 512 &&
        (long long)T * j_tiles < kSweepGaveUp) {
      LstmSweep P = {};
      const size_t ctr_bytes = sizeof(int) * 512 * kSweepCtrStride;
      void* p = nullptr;
      rc = zr_ctx_scratch(ctx, 1, ctr_bytes + sizeof(float) * (size_t)nl * T * n, &p);
      if (rc) return rc;
      P.counters = (int*)p;
      P.hp = (float*)((char*)p + ctr_bytes);
      rc = zr_memset_zero(ctx, P.counters, sizeof(int) * (size_t)nl * n_tiles * kSweepCtrStride);
      if (rc) return rc;
      for (int l = 0; l < nl; ++l) {
        P.W[l] = (const float*)layers[l]->d_W;
        P.bias[l] = layers[l]->d_bias;
        P.h0[l] = d_h0[l];
        P.c0[l] = d_c0[l];
        P.h_all[l] = d_h_all[l];
        P.c_all[l] = d_c_all[l];
        P.gates_all[l] = d_gates_all ? d_gates_all[l] : nullptr;
      }
      P.embed = d_embed;
      P.ids = d_ids_nonneg;
      P.mask01 = d_mask01;
      P.status = ctx->d_flags + 2;
      P.nl = nl;
      P.T = T;
      P.V = V;
      P.H = H;
      P.mb = mb;
      P.ldw = layers[0]->ldw;
      P.kp = layers[0]->kp;
      P.j_tiles = j_tiles;
      P.n_tiles = n_tiles;
      P.clip = clip_threshold;
      P.spin_limit = ctx->sweep_spin > 0 ? ctx->sweep_spin : (1 << 20);
      // Without the invalidation a consumer relies on never having cached a line before its producer wrote it: true
      // when no 128-byte line of the k-interleaved copies is shared between two producers, i.e. mb % 8 == 0.
      P.fence = (mb % 8 == 0) ? 0 : 1;
      ctx->last_stack_path = ZR_LSTM_STACK_PATH_SWEEP;
      return tn == 1 ? launch_sweep_v<1>(ctx, P, padded * n_tiles) : launch_sweep_v<2>(ctx, P, padded * n_tiles);
    }
  }
  // Every h is also written in a k-interleaved layout ([H/4][mb][4]) into a small ping-pong buffer per layer: its
  // two consumers on the next diagonal, (l+1, t) and (l, t+1), then fetch activations with contiguous 16-byte
  // loads.  The buffer written on diagonal d is read on d+1 only and overwritten on d+2.
  ctx->last_stack_path = ZR_LSTM_STACK_PATH_DIAGONALS;
  float* hp_buf = nullptr;
  if (vec && H % 8 == 0 && !layers[0]->bf16) {
    void* p = nullptr;
    rc = zr_ctx_scratch(ctx, 1, sizeof(float) * 2 * (size_t)nl * n, &p);
    if (rc) return rc;
    hp_buf = (float*)p;
  }
  auto hp_of = [&](int l, int d) { return hp_buf + ((size_t)(d & 1) * nl + l) * n; };
  // Diagonal wavefront: units (l, t) with l + t = d only depend on diagonal d-1.
  for (int d = 0; d < T + nl - 1; ++d) {
    LstmLaunch L = {};
    L.H = H;
    L.mb = mb;
    L.ldw = layers[0]->ldw;
    L.kp = layers[0]->kp;
    L.bf16 = layers[0]->bf16;
    L.bf16_single = ctx->bf16_terms == 1;
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
      U.inp[0] = (hp_buf && l > 0) ? hp_of(l - 1, d - 1) : nullptr;
      U.inp[1] = (hp_buf && t > 0) ? hp_of(l, d - 1) : nullptr;
      U.inp[2] = nullptr;
      U.hp = hp_buf ? hp_of(l, d) : nullptr;
      U.cprev = (t == 0) ? d_c0[l] : d_c_all[l] + (size_t)(t - 1) * n;
      U.mask01 = d_mask01 + (size_t)t * mb;
      U.h = d_h_all[l] + (size_t)t * n;
      U.c = d_c_all[l] + (size_t)t * n;
      for (int g = 0; g < 4; ++g)
        U.gates[g] = (d_gates_all && d_gates_all[l]) ? d_gates_all[l] + ((size_t)t * 4 + g) * n : nullptr;
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
