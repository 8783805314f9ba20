// Device-side scalar maths shared by the fused LSTM epilogue and the stand-alone gate kernel.
#ifndef ZR_MATH_H
#define ZR_MATH_H

#include <hip/hip_runtime.h>

// forward_sigmoid_kernel, float overload (reference: src/custom_kernels.h:58-65): 1 / (1 + e^-v).  The reference's
// feed-input variant (:92-99) evaluates the same expression in double and rounds to float.  Here it runs on the
// hardware base-2 exponential and reciprocal (each within one ulp), three instructions instead of a library expf
// and a full-precision division: a tile's epilogue evaluates five transcendentals per output element while the
// matrix pipe waits.  The result is within a few ulp of the reference's, far inside the 1e-4 contract; the
// saturated ends are exact (v >= 17: 1, v <= -89: 0).
__device__ __forceinline__ float zr_sigmoid(float v) {
  return __builtin_amdgcn_rcpf(1.0f + __builtin_amdgcn_exp2f(-1.4426950408889634f * v));
}

// forward_tanh_kernel (src/custom_kernels.h:106-135) and the tanhf of forward_h_t_kernel (:162-168) the same way:
// (1 - e^-2|v|) / (1 + e^-2|v|) with the sign restored, and the odd series through v^7 below 0.1, where the
// quotient form would cancel (series remainder < 3e-11 |v| there).
__device__ __forceinline__ float zr_tanh(float v) {
  const float a = fabsf(v);
  const float t = __builtin_amdgcn_exp2f(-2.8853900817779268f * a);
  const float big = (1.0f - t) * __builtin_amdgcn_rcpf(1.0f + t);
  const float a2 = a * a;
  const float small = a * (1.0f + a2 * (-0.33333334f + a2 * (0.13333334f + a2 * -0.053968254f)));
  return copysignf(a < 0.1f ? small : big, v);
}

// One LSTM cell update from the four biased pre-activations (reference: forward_c_t_kernel :141-147,
// clip_mat_kernel :2222-2231, forward_h_t_kernel :162-168, zero_c_t_and_h_t :184-192).
// clip <= 0 disables clipping; mask is 0.0f or 1.0f.
__device__ __forceinline__ void zr_lstm_cell(float zi, float zf, float zc, float zo, float c_prev, float mask,
                                             float clip, float& gi, float& gf, float& gc, float& go, float& c,
                                             float& h) {
  gi = zr_sigmoid(zi);
  gf = zr_sigmoid(zf);
  gc = zr_tanh(zc);
  go = zr_sigmoid(zo);
  float cv = gf * c_prev + gi * gc;
  if (clip > 0.0f) cv = fminf(fmaxf(cv, -clip), clip);
  float hv = go * zr_tanh(cv);
  c = cv * mask;
  h = hv * mask;
}

#endif
