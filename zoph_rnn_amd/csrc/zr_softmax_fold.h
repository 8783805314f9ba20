// Folding of the output layer's per-32-row-block (max, sum exp(x - max)) pairs into one pair per column: shared by
// softmax_colstats_kernel (zr_softmax.hip) and the beam's selection on blocks (zr_beam.hip), so that both arrive at the
// same bits (outputdist_overflow_prevention_kernel, src/custom_kernels.h:503-577, takes one max and one sum per column;
// here they are assembled from the blocks in one fixed order).
#pragma once
#include <hip/hip_runtime.h>
#include <math.h>

__device__ __forceinline__ void zr_softmax_fold(float& m, float& sm, float pm, float ps) {
  const float mn = fmaxf(m, pm);
  sm = (m == mn ? sm : sm * expf(m - mn)) + (pm == mn ? ps : ps * expf(pm - mn));
  m = mn;
}

// All 256 threads of a workgroup call this with the column's pairs ([nblocks][2] floats, contiguous).  Every thread
// folds its pairs into one running pair -- eight loads at a time, all in flight together -- then the threads' pairs are
// folded across the wave and the four waves, always in the same order.  On return thread 0 holds the column's (max, sum)
// in (mx, sum); block_max, if given, receives the largest block maximum this thread saw (-inf if none).
// s_m, s_s: four floats of shared memory each.
__device__ __forceinline__ void zr_softmax_fold_column(const float* __restrict__ pairs, int nblocks, float* s_m, float* s_s,
                                                       float& mx, float& sum, float* block_max) {
  typedef float zr_f32x2 __attribute__((ext_vector_type(2)));
  const int tid = threadIdx.x;
  const int lane = tid & 63, wave = tid >> 6;
  const zr_f32x2* pp = (const zr_f32x2*)pairs;
  mx = -INFINITY;
  sum = 0.0f;
  float bmax = -INFINITY;
  for (int b0 = 0; b0 < nblocks; b0 += 2048) {
    zr_f32x2 pr[8];
#pragma unroll
    for (int u = 0; u < 8; ++u) {
      const int b = b0 + tid + 256 * u;
      pr[u] = zr_f32x2{-INFINITY, 0.0f};
      if (b < nblocks) pr[u] = pp[b];
    }
#pragma unroll
    for (int u = 0; u < 8; ++u) {
      zr_softmax_fold(mx, sum, pr[u].x, pr[u].y);
      bmax = fmaxf(bmax, pr[u].x);  // (NaN never wins a maximum)
    }
  }
  if (block_max) *block_max = bmax;
#pragma unroll
  for (int off = 32; off > 0; off >>= 1) {
    const float om = __shfl_xor(mx, off, 64), os = __shfl_xor(sum, off, 64);
    // both partners add in the same order, so every lane ends with the same bits
    float a_m = (lane & off) ? om : mx, a_s = (lane & off) ? os : sum;
    const float b_m = (lane & off) ? mx : om, b_s = (lane & off) ? sum : os;
    zr_softmax_fold(a_m, a_s, b_m, b_s);
    mx = a_m;
    sum = a_s;
  }
  if (lane == 0) {
    s_m[wave] = mx;
    s_s[wave] = sum;
  }
  __syncthreads();
  if (tid == 0) {
    mx = s_m[0];
    sum = s_s[0];
#pragma unroll
    for (int w = 1; w < 4; ++w) zr_softmax_fold(mx, sum, s_m[w], s_s[w]);
  }
}
