// fp32 MFMA contraction core for gfx950 (64-lane waves, v_mfma_f32_32x32x2_f32).
//
// Shape of the work: every GEMM on this path is  C(M x N) = W(M x K) * X(K x N)  with a large weight matrix W
// streamed once, and a small activation matrix X (N = minibatch <= a few hundred columns).  Both are
// column-major, so W is contiguous along M and X is contiguous along K.
//
// Operand mapping.  The instruction computes D(32x32) += a(32x2) * b(2x32); lane l supplies a[l%32][l/32]
// and b[l/32][l%32], and holds D[8*(r/4) + 4*(l/32) + r%4][l%32] in accumulator register r.  We put the
// ACTIVATIONS on the a side (D row = batch column n) and the WEIGHTS on the b side (D column = output row m):
// then lane%32 indexes m, so the 32 lanes of a half-wave read 32 consecutive floats of a weight column
// (one 128-byte line) and write 32 consecutive floats of an output column -- every weight load and every
// output store is a full-line access, straight from/to registers, with no LDS transpose.
//
// K order.  Within a group of 8 consecutive k, lanes 0-31 take k0..k0+3 and lanes 32-63 take k0+4..k0+7, one k
// per MFMA: the i-th MFMA of the group multiplies k0+i (half 0) and k0+4+i (half 1).  Any pairing of k values
// is valid as long as both operands use the same one; this one lets each lane fetch its four activation
// values of a group with a single 16-byte load along K.
//
// Latency.  The weights come from HBM / the memory-side cache, a microsecond or more away, while one k-group of
// MFMAs lasts a fraction of that.  Operands are therefore fetched PF groups ahead into a ring of register
// fragments (software pipeline); weight addresses are a wave-uniform base plus a fixed per-lane offset so the
// address arithmetic stays on the scalar unit.
//
// Split K.  KS waves of a workgroup may share one output tile and take the k-groups round-robin; their
// partial tiles are summed through LDS in a fixed order (deterministic) before the epilogue runs.
#ifndef ZR_MFMA_CORE_H
#define ZR_MFMA_CORE_H

#include "zr_internal.h"

// Prefetch distance in k-groups for a TM x TN sub-tile wave: as deep as the register budget of the fragment
// ring allows (a fragment is 4*(TM+TN) registers).
constexpr int zr_prefetch_depth(int tm, int tn) {
#ifdef ZR_PF_OVERRIDE
  return ZR_PF_OVERRIDE;
#else
  return 4 * (tm + tn) <= 20 ? 3 : (4 * (tm + tn) <= 24 ? 2 : 1);
#endif
}

// How the weight operand is laid out in memory (element (row, k) of sub-tile tm):
//   ZR_A_NN     column-major:  wbase[row + k*lda]                 one 4-byte load per k
//   ZR_A_TRANS  row-major:     wbase[k + row*lda]                 one 16-byte load per 4 k (VEC)
//   ZR_A_PACK4  k-interleaved: wbase[((k/4)*lda + row)*4 + k%4]   one 16-byte load per 4 k, and the 32 lanes of a
//               half-wave read 512 contiguous bytes; K is padded to a multiple of 8 with zeros.  A wave can keep at
//               most 63 vector-memory instructions in flight, so 16-byte loads let it keep four times the bytes of
//               ZR_A_NN on the wire -- what hiding memory latency with one wave per SIMD needs.
enum { ZR_A_NN = 0, ZR_A_TRANS = 1, ZR_A_PACK4 = 2 };

template <int TM, int TN>
struct ZrFrag {
  float x[TN][4];  // activations: x[tn][i] = X[k_i][n(tn, lane%32)]
  float w[TM][4];  // weights:     w[tm][i] = W[m(tm, lane%32)][k_i]
};

// One K segment.
//   wbase[tm]: wave-uniform pointer to the weight matrix of sub-tile tm
//   woff[tm]:  this lane's fixed element offset into it:
//                ZR_A_NN:     row + 4*half*lda
//                ZR_A_TRANS:  row*lda + 4*half
//                ZR_A_PACK4:  row*4 + 4*half*lda
//   xcol[tn]:  this lane's activation column, already advanced by 4*half
//   xstride:   element step of xcol per k: 1 for a plain column (X[k][n] at column base + k); mb for activations
//              packed like ZR_A_PACK4 ([k/4][n][4], element step per k-block of 4 is 4*mb, so per k it is mb):
//              then the 32 lanes of a half-wave read 512 contiguous bytes instead of 16 bytes from each of 32
//              lines.  Packed activations require VEC and K % 8 == 0.
// Rows / columns are pre-clamped by the caller so that out-of-range lanes read valid memory.
// kslice must be wave-uniform.
template <int TM, int TN, int KS, int PF, int AMODE, bool VEC>
__device__ __forceinline__ void zr_mma_segment(zr_f32x16 (&acc)[TM][TN], const float* const (&wbase)[TM],
                                               const unsigned (&woff)[TM], long long lda,
                                               const float* const (&xcol)[TN], int K, int kslice, int half,
                                               int xstride = 1) {
  const int nfull = K >> 3;
  constexpr int NS = PF + 1;

  auto load_full = [&](ZrFrag<TM, TN>& f, int g) {
    const int kg = g * 8;  // wave-uniform
#pragma unroll
    for (int tn = 0; tn < TN; ++tn) {
      if (VEC) {
        const zr_f32x4 v = *(const zr_f32x4*)(xcol[tn] + (long long)kg * xstride);
        f.x[tn][0] = v.x;
        f.x[tn][1] = v.y;
        f.x[tn][2] = v.z;
        f.x[tn][3] = v.w;
      } else {
#pragma unroll
        for (int i = 0; i < 4; ++i) f.x[tn][i] = xcol[tn][kg + i];
      }
    }
#pragma unroll
    for (int tm = 0; tm < TM; ++tm) {
      if (AMODE == ZR_A_PACK4) {
        const float* p = wbase[tm] + (long long)kg * lda;  // uniform
        const zr_f32x4 v = *(const zr_f32x4*)(p + woff[tm]);
        f.w[tm][0] = v.x;
        f.w[tm][1] = v.y;
        f.w[tm][2] = v.z;
        f.w[tm][3] = v.w;
      } else if (AMODE == ZR_A_TRANS) {
        const float* p = wbase[tm] + kg;  // uniform
        if (VEC) {
          const zr_f32x4 v = *(const zr_f32x4*)(p + woff[tm]);
          f.w[tm][0] = v.x;
          f.w[tm][1] = v.y;
          f.w[tm][2] = v.z;
          f.w[tm][3] = v.w;
        } else {
#pragma unroll
          for (int i = 0; i < 4; ++i) f.w[tm][i] = p[woff[tm] + i];
        }
      } else {
#pragma unroll
        for (int i = 0; i < 4; ++i) {
          const float* p = wbase[tm] + (long long)(kg + i) * lda;  // uniform
          f.w[tm][i] = p[woff[tm]];
        }
      }
    }
  };

  auto mma = [&](const ZrFrag<TM, TN>& f) {
#pragma unroll
    for (int i = 0; i < 4; ++i)
#pragma unroll
      for (int tm = 0; tm < TM; ++tm)
#pragma unroll
        for (int tn = 0; tn < TN; ++tn)
          acc[tm][tn] = __builtin_amdgcn_mfma_f32_32x32x2f32(f.x[tn][i], f.w[tm][i], acc[tm][tn], 0, 0, 0);
  };

  // The steady-state loop is free of branches: every stage issues the loads of the group PF stages ahead
  // (group indices past the end are clamped to the last group: a few redundant loads of valid memory) and then
  // multiplies the fragment loaded PF stages ago.  Keeping loads unconditional matters: with loads under
  // branches the compiler cannot count how many younger loads are in flight and waits for all of them.
  if (kslice < nfull) {
    const int last = nfull - 1;
    const int n_mine = (nfull - kslice + KS - 1) / KS;  // groups owned by this wave: kslice, kslice+KS, ...
    ZrFrag<TM, TN> f[NS];
#pragma unroll
    for (int s = 0; s < PF; ++s) {
      const int gl = kslice + s * KS;
      load_full(f[s], gl < last ? gl : last);
    }
    int it = 0;
    for (; it + NS <= n_mine; it += NS) {
#pragma unroll
      for (int s = 0; s < NS; ++s) {
        const int gl = kslice + (it + s + PF) * KS;
        load_full(f[(s + PF) % NS], gl < last ? gl : last);
        mma(f[s]);
      }
    }
    // at most PF groups remain, all of them already loaded
#pragma unroll
    for (int s = 0; s < PF; ++s)
      if (it + s < n_mine) mma(f[s]);
  }
  // tail group (K not a multiple of 8): zero-filled, owned by the slice whose turn it is
  if ((K & 7) != 0 && (nfull % KS) == kslice) {
    const int kg = nfull * 8;
    ZrFrag<TM, TN> t;
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const int k = kg + 4 * half + i;
      const bool ok = k < K;
      // xcol/woff already include this lane's 4*half: index relative to them
      const int rel = ok ? kg + i : (K - 1) - 4 * half;
#pragma unroll
      for (int tn = 0; tn < TN; ++tn) {
        const float v = xcol[tn][rel];
        t.x[tn][i] = ok ? v : 0.0f;
      }
#pragma unroll
      for (int tm = 0; tm < TM; ++tm) {
        // ZR_A_PACK4: the padded tail block exists in memory, this lane's four values sit side by side
        const float v = AMODE == ZR_A_PACK4   ? wbase[tm][(long long)kg * lda + woff[tm] + i]
                        : AMODE == ZR_A_TRANS ? wbase[tm][(long long)woff[tm] + rel]
                                              : wbase[tm][(long long)woff[tm] + (long long)rel * lda];
        t.w[tm][i] = ok ? v : 0.0f;
      }
    }
    mma(t);
  }
}

// Variant of zr_mma_segment for k-interleaved weights and 16-byte activation loads that fetches through buffer
// descriptors: an address is descriptor base (scalar registers) + a scalar byte offset that advances with k + a 32-bit
// per-lane byte offset that stays fixed through the segment, so a load needs no vector address arithmetic at all
// (64-bit vector adds would compete with the MFMAs for the vector issue slot).  The stages of the ring are fenced
// off from each other for the instruction scheduler -- left alone it gathers the loads of a whole ring revolution
// at its end, which drains the ring once per revolution -- and, inside a stage, the loads are spread evenly among
// the MFMAs.
//   wrsrc:    descriptor over the TM weight sub-tiles' matrices; wsoff[tm] = byte offset of sub-tile tm's matrix
//   woffb:    this lane's byte offset into every weight sub-tile: 4 * (4*row + 4*half*lda)
//   xrsrc:    descriptor over the activations
//   xoffb[tn]: this lane's byte offset of its column, 4*half included
//   wstep / xstep: bytes per k-group of 8 (weights: 32*lda; activations: 32 for a plain column, 32*mb k-interleaved)
// Every offset sum must stay below 4 GiB (the host checks the extents).
typedef unsigned zr_u32x4v __attribute__((ext_vector_type(4)));
// Cache policy operand of the weight fetches (the buffer-load builtin's last argument): 0 = default, ZR_AUX_STREAM =
// the non-temporal hint.  A matrix that is read once per step and is a large part of the memory-side cache (the output
// layer's: 200 MB of its 256 MB at 50 000 x 1000) otherwise pushes out everything the rest of the step re-reads -- the
// LSTM and attention matrices, the source states -- and every step fetches all of it from memory again.
constexpr int ZR_AUX_STREAM = 2;
__device__ __forceinline__ __amdgpu_buffer_rsrc_t zr_make_rsrc(const void* base) {
  // raw buffer, no bounds limit to speak of, 32-bit data format (descriptor word 3 for this GPU family)
  return __builtin_amdgcn_make_buffer_rsrc(const_cast<void*>(base), 0, 0xFFFFFFFF, 0x00020000);
}

// The weight halves of the first PF ring stages of a segment, issued ahead of time (zr_mma_segment_u with WPRE then
// fetches only the activation halves in its prologue): weights depend on nothing, so a caller that must wait for its
// activations can have them in flight during the wait.
template <int TM, int TN, int KS, int PF, int WAUX = 0>
__device__ __forceinline__ void zr_preload_w(ZrFrag<TM, TN> (&f)[PF + 1], __amdgpu_buffer_rsrc_t wrsrc,
                                             const unsigned (&wsoff)[TM], unsigned woffb, unsigned wstep, int K,
                                             int kslice) {
  const int last = (K >> 3) - 1;
#pragma unroll
  for (int s = 0; s < PF; ++s) {
    int gl = kslice + s * KS;
    gl = gl < last ? gl : last;
#pragma unroll
    for (int tm = 0; tm < TM; ++tm) {
      const zr_u32x4v v =
          __builtin_amdgcn_raw_buffer_load_b128(wrsrc, (int)woffb, (int)(wsoff[tm] + (unsigned)gl * wstep), WAUX);
      f[s].w[tm][0] = __uint_as_float(v.x);
      f[s].w[tm][1] = __uint_as_float(v.y);
      f[s].w[tm][2] = __uint_as_float(v.z);
      f[s].w[tm][3] = __uint_as_float(v.w);
    }
  }
}

template <int TM, int TN, int KS, int PF, bool WPRE = false, int WAUX = 0>
__device__ __forceinline__ void zr_mma_segment_u(zr_f32x16 (&acc)[TM][TN], __amdgpu_buffer_rsrc_t wrsrc,
                                                 const unsigned (&wsoff)[TM], unsigned woffb, unsigned wstep,
                                                 __amdgpu_buffer_rsrc_t xrsrc, const unsigned (&xoffb)[TN],
                                                 unsigned xstep, int K, int kslice, ZrFrag<TM, TN> (&f)[PF + 1]) {
  const int nfull = K >> 3;  // K % 8 == 0
  constexpr int NS = PF + 1;
  auto load_x = [&](ZrFrag<TM, TN>& f, int g) {
    const unsigned ug = (unsigned)g;  // wave-uniform
#pragma unroll
    for (int tn = 0; tn < TN; ++tn) {
      const zr_u32x4v v = __builtin_amdgcn_raw_buffer_load_b128(xrsrc, (int)xoffb[tn], (int)(ug * xstep), 0);
      f.x[tn][0] = __uint_as_float(v.x);
      f.x[tn][1] = __uint_as_float(v.y);
      f.x[tn][2] = __uint_as_float(v.z);
      f.x[tn][3] = __uint_as_float(v.w);
    }
  };
  auto load_full = [&](ZrFrag<TM, TN>& f, int g) {
    const unsigned ug = (unsigned)g;  // wave-uniform
    load_x(f, g);
#pragma unroll
    for (int tm = 0; tm < TM; ++tm) {
      const zr_u32x4v v = __builtin_amdgcn_raw_buffer_load_b128(wrsrc, (int)woffb, (int)(wsoff[tm] + ug * wstep), WAUX);
      f.w[tm][0] = __uint_as_float(v.x);
      f.w[tm][1] = __uint_as_float(v.y);
      f.w[tm][2] = __uint_as_float(v.z);
      f.w[tm][3] = __uint_as_float(v.w);
    }
  };
  auto mma = [&](const ZrFrag<TM, TN>& f) {
#pragma unroll
    for (int i = 0; i < 4; ++i)
#pragma unroll
      for (int tm = 0; tm < TM; ++tm)
#pragma unroll
        for (int tn = 0; tn < TN; ++tn)
          acc[tm][tn] = __builtin_amdgcn_mfma_f32_32x32x2f32(f.x[tn][i], f.w[tm][i], acc[tm][tn], 0, 0, 0);
  };
  if (kslice < nfull) {
    const int last = nfull - 1;
    const int n_mine = (nfull - kslice + KS - 1) / KS;
#pragma unroll
    for (int s = 0; s < PF; ++s) {
      const int gl = kslice + s * KS;
      if (WPRE)
        load_x(f[s], gl < last ? gl : last);
      else
        load_full(f[s], gl < last ? gl : last);
    }
    int it = 0;
    for (; it + NS <= n_mine; it += NS) {
#pragma unroll
      for (int s = 0; s < NS; ++s) {
        const int gl = kslice + (it + s + PF) * KS;
        load_full(f[(s + PF) % NS], gl < last ? gl : last);
        mma(f[s]);
        {
          // one load, then its share of the stage's MFMAs: a load issued while the matrix pipe works costs nothing,
          // a run of loads leaves the pipe idle for as long as their issue takes
          constexpr int NL = TM + TN, NM = 4 * TM * TN, PER = NM / NL;
#pragma unroll
          for (int q = 0; q < NL; ++q) {
            __builtin_amdgcn_sched_group_barrier(0x008, PER, 0);  // MFMA
            __builtin_amdgcn_sched_group_barrier(0x020, 1, 0);    // vector memory read
          }
          __builtin_amdgcn_sched_group_barrier(0x008, NM - NL * PER, 0);
        }
        __builtin_amdgcn_sched_barrier(0);
      }
    }
#pragma unroll
    for (int s = 0; s < PF; ++s)
      if (it + s < n_mine) mma(f[s]);
  }
}

// The same with a ring of its own (no weights fetched ahead).
template <int TM, int TN, int KS, int PF, int WAUX = 0>
__device__ __forceinline__ void zr_mma_segment_ring(zr_f32x16 (&acc)[TM][TN], __amdgpu_buffer_rsrc_t wrsrc,
                                                 const unsigned (&wsoff)[TM], unsigned woffb, unsigned wstep,
                                                 __amdgpu_buffer_rsrc_t xrsrc, const unsigned (&xoffb)[TN],
                                                 unsigned xstep, int K, int kslice) {
  ZrFrag<TM, TN> f[PF + 1];
  zr_mma_segment_u<TM, TN, KS, PF, false, WAUX>(acc, wrsrc, wsoff, woffb, wstep, xrsrc, xoffb, xstep, K, kslice, f);
}

// Workgroup barrier that also publishes: when it returns, every store any thread of the workgroup issued before it
// has completed (device-scope write-through stores have reached memory), so one thread may then announce the
// workgroup's data to other workgroups with a device-scope atomic.  A workgroup-scope release fence alone only keeps
// the compiler from sinking the stores; it does not make a wave wait for the acknowledgements of stores in flight,
// hence the explicit vmcnt(0) (s_waitcnt operand: vmcnt = 0, expcnt and lgkmcnt at their maxima = no wait).
__device__ __forceinline__ void zr_publish_barrier() {
  __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup");
  __builtin_amdgcn_s_waitcnt(0x0F70);
  __syncthreads();
}

// 16-byte store that is written through to memory (device scope), what __hip_atomic_store(..., __HIP_MEMORY_SCOPE_AGENT)
// is for one float: for data another workgroup reads behind a counter.
// The instruction is followed by one idle cycle: a store of more than 8 bytes reads its data registers one cycle after
// it issues, and the compiler, which inserts that cycle behind its own stores, does not look inside an asm statement
// (without it the first register was seen overwritten by the next instruction).
__device__ __forceinline__ void zr_store16_device(void* p, zr_f32x4 v) {
  asm volatile("global_store_dwordx4 %0, %1, off sc1\n\ts_nop 0" ::"v"(p), "v"(v) : "memory");
}

// Number of visits zr_reduce_visit makes per thread, and the accumulator slot (tn*16 + r) of visit i: callers use
// them to fetch epilogue operands (previous cell state, biases) before the K loop instead of after it.
template <int TN, int KS>
constexpr int zr_visit_count() { return KS == 1 ? TN * 16 : TN * 16 / KS; }
template <int KS>
__device__ __forceinline__ int zr_visit_slot(int kslice, int i) { return KS == 1 ? i : kslice + KS * i; }

// Sums the KS partial tiles of a workgroup and calls f(vals[TM], tn, r, i) once per (tn, r, lane) owned by the
// calling thread, where vals[tm] is the finished accumulator register r of sub-tile (tm, tn) for this lane and i
// is the visit index (slot tn*16 + r == zr_visit_slot<KS>(kslice, i)).
// Every lane of a wave calls f with the same (tn, r) at the same time (wave-uniform control flow), and a
// thread keeps its lane index, so the caller's mapping  m <- lane%32,  n <- 8*(r/4) + 4*(lane/32) + r%4  holds.
// `red` is LDS of KS * TN*16 * 64 floats (unused when KS == 1).  All threads of the workgroup must call this.
template <int TM, int TN, int KS, class F>
__device__ __forceinline__ void zr_reduce_visit(zr_f32x16 (&acc)[TM][TN], float* red, int kslice, int lane, F f) {
  if (KS == 1) {
#pragma unroll
    for (int tn = 0; tn < TN; ++tn)
#pragma unroll
      for (int r = 0; r < 16; ++r) {
        float vals[TM];
#pragma unroll
        for (int tm = 0; tm < TM; ++tm) vals[tm] = acc[tm][tn][r];
        f(vals, tn, r, tn * 16 + r);
      }
  } else {
    constexpr int SLOTS = TN * 16;           // accumulator registers per sub-tile row of the tile
    constexpr int PT = SLOTS / KS;           // slots finished by each wave
    static_assert(SLOTS % KS == 0, "KS must divide TN*16");
    float pre[TM][PT];
#pragma unroll
    for (int tm = 0; tm < TM; ++tm) {
      __syncthreads();  // previous round's reads are done
#pragma unroll
      for (int tn = 0; tn < TN; ++tn)
#pragma unroll
        for (int r = 0; r < 16; ++r) red[((size_t)kslice * SLOTS + tn * 16 + r) * 64 + lane] = acc[tm][tn][r];
      __syncthreads();
#pragma unroll
      for (int i = 0; i < PT; ++i) {
        const int slot = kslice + KS * i;
        float s = 0.0f;
#pragma unroll
        for (int w = 0; w < KS; ++w) s += red[((size_t)w * SLOTS + slot) * 64 + lane];
        pre[tm][i] = s;
      }
    }
#pragma unroll
    for (int i = 0; i < PT; ++i) {
      const int slot = kslice + KS * i;
      float vals[TM];
#pragma unroll
      for (int tm = 0; tm < TM; ++tm) vals[tm] = pre[tm][i];
      f(vals, slot / 16, slot % 16, i);
    }
  }
}

// The same reduction in ONE round, for kernels that own a whole CU's LDS: every wave writes all TM*TN of its partial
// tiles (16-byte stores, four consecutive accumulator registers of a lane each), one barrier, and every wave sums
// the KS copies of the groups of four it finishes (16-byte loads; the sum runs over the waves in the same order as
// in zr_reduce_visit, so both give the same bits).  Against TM rounds of write-barrier-read this saves 2*TM - 2
// barriers with their exposed LDS latency and three quarters of the LDS instructions.  `red` holds
// KS * TM * TN*16 * 64 floats, 16-byte aligned (128 KB for TM=4, TN=2, KS=4).  Visit i of wave `kslice` is
// accumulator slot zr_wide_visit_slot<KS>(kslice, i); otherwise the contract is zr_reduce_visit's.
template <int KS>
__device__ __forceinline__ int zr_wide_visit_slot(int kslice, int i) { return (kslice + KS * (i >> 2)) * 4 + (i & 3); }

template <int TM, int TN, int KS, class F>
__device__ __forceinline__ void zr_reduce_visit_wide(zr_f32x16 (&acc)[TM][TN], float* red, int kslice, int lane, F f) {
  constexpr int G4 = TN * 4;   // groups of four accumulator registers per sub-tile row of the tile
  constexpr int PG = G4 / KS;  // groups finished by each wave
  static_assert(KS > 1 && G4 % KS == 0, "KS must divide TN*4");
  zr_f32x4* red4 = (zr_f32x4*)red;
  __syncthreads();  // the previous use of `red` is over
#pragma unroll
  for (int tm = 0; tm < TM; ++tm)
#pragma unroll
    for (int g4 = 0; g4 < G4; ++g4) {
      zr_f32x4 v;
#pragma unroll
      for (int c = 0; c < 4; ++c) v[c] = acc[tm][g4 >> 2][(g4 & 3) * 4 + c];
      red4[((kslice * TM + tm) * G4 + g4) * 64 + lane] = v;
    }
  __syncthreads();
  zr_f32x4 pre[TM][PG];
#pragma unroll
  for (int i4 = 0; i4 < PG; ++i4)
#pragma unroll
    for (int tm = 0; tm < TM; ++tm) {
      zr_f32x4 sum = {0.0f, 0.0f, 0.0f, 0.0f};
#pragma unroll
      for (int w = 0; w < KS; ++w) sum += red4[((w * TM + tm) * G4 + kslice + KS * i4) * 64 + lane];
      pre[tm][i4] = sum;
    }
#pragma unroll
  for (int i = 0; i < PG * 4; ++i) {
    const int slot = zr_wide_visit_slot<KS>(kslice, i);
    float vals[TM];
#pragma unroll
    for (int tm = 0; tm < TM; ++tm) vals[tm] = pre[tm][i >> 2][i & 3];
    f(vals, slot >> 4, slot & 15, i);
  }
}

// ---------------------------------------------------------------------------------------------------------
// (max, sum of exp(v - max)) over the 32 lanes of each half-wave, for G independent values per lane at once.
// In the MFMA output layout a half-wave holds the 32 rows of one output column, so this is the softmax partial
// of a 32-row block.  The G butterflies are interleaved (a lone butterfly is a chain of ten dependent cross-lane
// moves, each with the latency of an LDS round trip); the steps inside a 16-lane row are DPP moves on the
// vector ALU, only the last one crosses rows.  Must be called by all 64 lanes.  Lanes with ok == false
// contribute nothing; if no lane of a half is ok the result is (-inf, 0).
// ---------------------------------------------------------------------------------------------------------
template <int CTRL>
__device__ __forceinline__ float zr_dpp_move(float x) {
  return __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(x), CTRL, 0xF, 0xF, false));
}

template <int G>
__device__ __forceinline__ void zr_half_wave_softmax_stats(const float (&v)[G], const bool (&ok)[G], float (&mx)[G],
                                                           float (&se)[G]) {
  // lane pairings: quad_perm(1,0,3,2), quad_perm(2,3,0,1), row_half_mirror, row_mirror, then lanes 16 apart
#pragma unroll
  for (int g = 0; g < G; ++g) mx[g] = ok[g] ? v[g] : -INFINITY;
#pragma unroll
  for (int g = 0; g < G; ++g) mx[g] = fmaxf(mx[g], zr_dpp_move<0xB1>(mx[g]));
#pragma unroll
  for (int g = 0; g < G; ++g) mx[g] = fmaxf(mx[g], zr_dpp_move<0x4E>(mx[g]));
#pragma unroll
  for (int g = 0; g < G; ++g) mx[g] = fmaxf(mx[g], zr_dpp_move<0x141>(mx[g]));
#pragma unroll
  for (int g = 0; g < G; ++g) mx[g] = fmaxf(mx[g], zr_dpp_move<0x140>(mx[g]));
#pragma unroll
  for (int g = 0; g < G; ++g) mx[g] = fmaxf(mx[g], __shfl_xor(mx[g], 16, 64));
  // hardware base-2 exponential (one ulp) of (v - max) * log2(e): relative error below 1e-7 * |v - max|, far inside
  // what the sums of these terms are used for
#pragma unroll
  for (int g = 0; g < G; ++g) se[g] = ok[g] ? __builtin_amdgcn_exp2f((v[g] - mx[g]) * 1.4426950408889634f) : 0.0f;
#pragma unroll
  for (int g = 0; g < G; ++g) se[g] += zr_dpp_move<0xB1>(se[g]);
#pragma unroll
  for (int g = 0; g < G; ++g) se[g] += zr_dpp_move<0x4E>(se[g]);
#pragma unroll
  for (int g = 0; g < G; ++g) se[g] += zr_dpp_move<0x141>(se[g]);
#pragma unroll
  for (int g = 0; g < G; ++g) se[g] += zr_dpp_move<0x140>(se[g]);
#pragma unroll
  for (int g = 0; g < G; ++g) se[g] += __shfl_xor(se[g], 16, 64);
}

// ---------------------------------------------------------------------------------------------------------
// bf16-weight variant of the contraction core (v_mfma_f32_32x32x16_bf16, 16 k per instruction).
//
// Weights are stored as bf16, k-interleaved in blocks of 8: element (row, k) at ((k/8)*lda + row)*8 + k%8 (lda =
// rows rounded up to 32, K a multiple of 16, pads zero), so a lane's operand for one instruction -- 8 consecutive k
// of its row -- is one 16-byte load and a half-wave reads 512 contiguous bytes.  Half-wave 0 takes k0..k0+7,
// half-wave 1 k0+8..k0+15.
// Activations stay fp32 in memory.  Each value is split in registers into two bf16 terms, x = hi + lo with
// hi = bf16(x) and lo = bf16(x - hi), and both are multiplied with the same weight operand: the products are exact
// in fp32, accumulation is fp32, and the only error beyond an fp32 contraction is the 2^-17 relative residue of
// the split.  Two bf16 instructions replace eight fp32 ones.
//   woff[tm]:  8*row + 8*half*lda   (bf16 elements)
//   xcol[tn]:  this lane's activation column advanced by 8*half
// XPK: the activations were split and packed beforehand (zr_split_pack_multi_kernel): two bf16 arrays hi and lo, each
// k-interleaved like the weights ([K/8][N][8]); xcol[tn] / xlo[tn] then point at this lane's first block
// (base + 8*(col + half*N)), xstride = N, and the loop body has no conversion arithmetic and only contiguous loads.
// ---------------------------------------------------------------------------------------------------------
// ZR_A_PACK8_BF16_1T: the same weight layout in single-term mode (activations rounded to bf16 once, no lo array)
enum { ZR_A_PACK8_BF16 = 3, ZR_A_PACK8_BF16_1T = 4 };
constexpr bool zr_is_bf16_mode(int amode) { return amode == ZR_A_PACK8_BF16 || amode == ZR_A_PACK8_BF16_1T; }
typedef __bf16 zr_bf16x8 __attribute__((ext_vector_type(8)));
typedef __bf16 zr_bf16x2 __attribute__((ext_vector_type(2)));
typedef unsigned zr_u32x4 __attribute__((ext_vector_type(4)));

// (x0, x1) -> packed bf16 pairs hi and lo with x = hi + lo up to 2^-17 |x|
__device__ __forceinline__ void zr_split_bf16_pair(float x0, float x1, unsigned& hi, unsigned& lo) {
  zr_bf16x2 h;
  h[0] = (__bf16)x0;
  h[1] = (__bf16)x1;
  const unsigned hu = __builtin_bit_cast(unsigned, h);
  const float h0 = __uint_as_float(hu << 16), h1 = __uint_as_float(hu & 0xFFFF0000u);
  zr_bf16x2 l;
  l[0] = (__bf16)(x0 - h0);
  l[1] = (__bf16)(x1 - h1);
  hi = hu;
  lo = __builtin_bit_cast(unsigned, l);
}

template <int TM, int TN>
struct ZrFragBf16 {
  zr_f32x4 x[TN][2];  // 8 consecutive k of this lane's column as fp32, or (XPK) [0] = hi and [1] = lo bf16 octets
  zr_u32x4 w[TM];     // 8 consecutive k of this lane's row, bf16
};

// LO = false (with XPK): single-term mode -- only the hi halves are fetched and multiplied: every activation is
// rounded to bf16 once (relative error 2^-9), half the matrix instructions and half the activation operand traffic.
template <int TM, int TN, int KS, int PF, bool XPK = false, bool LO = true>
__device__ __forceinline__ void zr_mma_segment_bf16(zr_f32x16 (&acc)[TM][TN], const unsigned short* const (&wbase)[TM],
                                                    const unsigned (&woff)[TM], long long lda,
                                                    const float* const (&xcol)[TN], int K, int kslice,
                                                    const unsigned short* const* xlo = nullptr, int xstride = 0) {
  const int nfull = K >> 4;  // K % 16 == 0 (checked by the host code)
  constexpr int NS = PF + 1;

  auto load_full = [&](ZrFragBf16<TM, TN>& f, int g) {
    const int kg = g * 16;  // wave-uniform
#pragma unroll
    for (int tn = 0; tn < TN; ++tn) {
      if (XPK) {
        const long long off = (long long)kg * xstride;  // bf16 elements; uniform
        f.x[tn][0] = *(const zr_f32x4*)((const unsigned short*)xcol[tn] + off);
        if (LO) f.x[tn][1] = *(const zr_f32x4*)(xlo[tn] + off);
      } else {
        f.x[tn][0] = *(const zr_f32x4*)(xcol[tn] + kg);
        f.x[tn][1] = *(const zr_f32x4*)(xcol[tn] + kg + 4);
      }
    }
#pragma unroll
    for (int tm = 0; tm < TM; ++tm) {
      const unsigned short* p = wbase[tm] + (long long)kg * lda;  // uniform
      f.w[tm] = *(const zr_u32x4*)(p + woff[tm]);
    }
  };

  auto mma = [&](const ZrFragBf16<TM, TN>& f) {
    zr_bf16x8 w[TM];
#pragma unroll
    for (int tm = 0; tm < TM; ++tm) w[tm] = __builtin_bit_cast(zr_bf16x8, f.w[tm]);
#pragma unroll
    for (int tn = 0; tn < TN; ++tn) {
      if (XPK) {
        const zr_bf16x8 ph = __builtin_bit_cast(zr_bf16x8, f.x[tn][0]), pl = __builtin_bit_cast(zr_bf16x8, f.x[tn][1]);
#pragma unroll
        for (int tm = 0; tm < TM; ++tm)
          acc[tm][tn] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(ph, w[tm], acc[tm][tn], 0, 0, 0);
        if (LO) {
#pragma unroll
          for (int tm = 0; tm < TM; ++tm)
            acc[tm][tn] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(pl, w[tm], acc[tm][tn], 0, 0, 0);
        }
        continue;
      }
      unsigned h0, h1, h2, h3, l0, l1, l2, l3;
      zr_split_bf16_pair(f.x[tn][0].x, f.x[tn][0].y, h0, l0);
      zr_split_bf16_pair(f.x[tn][0].z, f.x[tn][0].w, h1, l1);
      zr_split_bf16_pair(f.x[tn][1].x, f.x[tn][1].y, h2, l2);
      zr_split_bf16_pair(f.x[tn][1].z, f.x[tn][1].w, h3, l3);
      const zr_u32x4 hi = {h0, h1, h2, h3}, lo = {l0, l1, l2, l3};
      const zr_bf16x8 xh = __builtin_bit_cast(zr_bf16x8, hi), xl = __builtin_bit_cast(zr_bf16x8, lo);
#pragma unroll
      for (int tm = 0; tm < TM; ++tm)
        acc[tm][tn] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(xh, w[tm], acc[tm][tn], 0, 0, 0);
      if (LO) {
#pragma unroll
        for (int tm = 0; tm < TM; ++tm)
          acc[tm][tn] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(xl, w[tm], acc[tm][tn], 0, 0, 0);
      }
    }
  };

  // same branch-free software pipeline as zr_mma_segment
  if (kslice < nfull) {
    const int last = nfull - 1;
    const int n_mine = (nfull - kslice + KS - 1) / KS;
    ZrFragBf16<TM, TN> f[NS];
#pragma unroll
    for (int s = 0; s < PF; ++s) {
      const int gl = kslice + s * KS;
      load_full(f[s], gl < last ? gl : last);
    }
    int it = 0;
    for (; it + NS <= n_mine; it += NS) {
#pragma unroll
      for (int s = 0; s < NS; ++s) {
        const int gl = kslice + (it + s + PF) * KS;
        load_full(f[(s + PF) % NS], gl < last ? gl : last);
        mma(f[s]);
      }
    }
#pragma unroll
    for (int s = 0; s < PF; ++s)
      if (it + s < n_mine) mma(f[s]);
  }
}

#endif
