// What the forward and the backward pass of KDA share: the operator's options as the kernels see them and the scalar
// functions of the gate.
#pragma once

namespace gdn {

struct KdaFlags {
  int l2norm, use_gate, has_lower_bound, beta_sigmoid, beta_x2, g_f32, beta_f32;
  float lower_bound;
};

__device__ __forceinline__ float kda_sigmoid(float x) { return 1.f / (1.f + __expf(-x)); }
// log(1 + e^x) = max(x, 0) + log(1 + e^{-|x|}) with the hardware exponential and logarithm: absolute error of the
// order of 1e-7 everywhere (the argument of the logarithm lies in (1, 2])
__device__ __forceinline__ float kda_softplus(float x) { return fmaxf(x, 0.f) + __logf(1.f + __expf(-fabsf(x))); }

// VEC consecutive fp32 values of an LDS row
template <int VEC> __device__ __forceinline__ void ld_f32(const float* p, float* f) {
#pragma unroll
  for (int e = 0; e < VEC; e += 4) {
    const f32x4 x = *reinterpret_cast<const f32x4*>(p + e);
    f[e] = x[0]; f[e + 1] = x[1]; f[e + 2] = x[2]; f[e + 3] = x[3];
  }
}

}  // namespace gdn
