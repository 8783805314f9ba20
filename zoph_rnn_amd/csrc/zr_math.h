// Device-side scalar maths shared by the fused LSTM epilogue and the stand-alone gate kernel.
#ifndef ZR_MATH_H
#define ZR_MATH_H

#include <hip/hip_runtime.h>

// forward_sigmoid_kernel, float overload (reference: src/custom_kernels.h:58-65).  The reference's feed-input
// variant (:92-99) evaluates the same expression in double and rounds to float; the two differ by at most
// one float ulp, far inside the 1e-4 contract, so one fp32 form serves both.
__device__ __forceinline__ float zr_sigmoid(float v) { return 1.0f / (1.0f + expf(-v)); }

// One LSTM cell update from the four biased pre-activations (reference: forward_c_t_kernel :141-147,
// clip_mat_kernel :2222-2231, forward_h_t_kernel :162-168, zero_c_t_and_h_t :184-192).
// clip <= 0 disables clipping; mask is 0.0f or 1.0f.
__device__ __forceinline__ void zr_lstm_cell(float zi, float zf, float zc, float zo, float c_prev, float mask,
                                             float clip, float& gi, float& gf, float& gc, float& go, float& c,
                                             float& h) {
  gi = zr_sigmoid(zi);
  gf = zr_sigmoid(zf);
  gc = tanhf(zc);
  go = zr_sigmoid(zo);
  float cv = gf * c_prev + gi * gc;
  if (clip > 0.0f) cv = fminf(fmaxf(cv, -clip), clip);
  float hv = go * tanhf(cv);
  c = cv * mask;
  h = hv * mask;
}

#endif
