// What the forward and the backward pass of KDA share: the operator's options as the kernels see them and the scalar
// functions of the gate.
#pragma once

namespace gdn {

struct KdaFlags {
  int l2norm, use_gate, has_lower_bound, beta_sigmoid, beta_x2, g_f32, beta_f32;
  float lower_bound;
};

// A compile-time integer as a function argument: lets one generic lambda be stamped out once per mode.
template <int V> struct IntConst { static constexpr int value = V; };

// The hardware reciprocal and base-2 logarithm, one instruction each (1 ulp), in place of the IEEE division and the
// range-checked logarithm: a gate costs a few instructions per element, and the kernels evaluate one per token and
// key channel.
__device__ __forceinline__ float kda_sigmoid(float x) { return __builtin_amdgcn_rcpf(1.f + __expf(-x)); }
// log(1 + e^x) = max(x, 0) + log(1 + e^{-|x|}): the argument of the logarithm lies in (1, 2], absolute error of the
// order of 1e-7 everywhere
__device__ __forceinline__ float kda_softplus(float x) {
  return fmaxf(x, 0.f) + 0.69314718f * __builtin_amdgcn_logf(1.f + __expf(-fabsf(x)));
}
// softplus and its derivative, the sigmoid, from one exponential
__device__ __forceinline__ void kda_softplus_sigmoid(float x, float& sp, float& sg) {
  const float t = __expf(-fabsf(x)), r = __builtin_amdgcn_rcpf(1.f + t);
  sp = fmaxf(x, 0.f) + 0.69314718f * __builtin_amdgcn_logf(1.f + t);
  sg = x >= 0.f ? r : t * r;
}

// The cumulative log decay G enters the kernels only through e^{G}, e^{G_i - G_j}.  The 16-bit kernels keep it in units
// of log 2 (G log2 e, applied once where the gate leaves its values), so that each of the many exponentials is the
// hardware's base-2 instruction alone, without the multiplication in front of it.  The fp32 kernels (the parity path)
// keep natural units: a difference of pre-scaled values carries the rounding of both, which grows with |G| instead of
// with the difference.
template <typename T> struct KdaDecay {
  static constexpr bool kBase2 = sizeof(T) == 2;
  static constexpr float kUnit = kBase2 ? 1.4426950408889634f : 1.f;   // G as stored = G * kUnit
  static __device__ __forceinline__ float exp(float x) {
    if constexpr (kBase2) return __builtin_amdgcn_exp2f(x);
    else return __expf(x);
  }
};

// The gate: the log decay of one token and channel from the gate input x, in the units G is kept in (au = e^{A_log} kUnit,
// lbu = lower_bound kUnit, a = e^{A_log}).  MODE 0: x is the log decay itself; 1: -e^{A_log} softplus(x + bias);
// 2: lower_bound sigmoid(e^{A_log} (x + bias)).  The forward and the backward kernels both form G through this function
// and kda_cumsum_part below, in the same order of operations, so both hold the same bits.
template <typename T, int MODE> __device__ __forceinline__ float kda_gate(float x, float bias, float a, float au, float lbu) {
  if (MODE == 0) return x * KdaDecay<T>::kUnit;
  if (MODE == 1) return -au * kda_softplus(x + bias);
  return lbu * kda_sigmoid(a * (x + bias));
}

// Cumulative sum down the 64 tokens of G [64][LDG] (LDS), first step: thread (part, d) of PARTS x DK threads sums its
// 64 / PARTS rows of channel d in place and leaves their total in tot[part][d].  After a barrier row i of part p holds
// its cumulative sum once kda_cumsum_before(tot, p, d) is added.
template <int DK, int LDG, int PARTS> __device__ __forceinline__ void kda_cumsum_part(float* Gs, float* tot, int t) {
  constexpr int RPP = 64 / PARTS;
  const int d = t % DK, part = t / DK;
  float run = 0.f;
#pragma unroll
  for (int r = 0; r < RPP; ++r) {
    run += Gs[(part * RPP + r) * LDG + d];
    Gs[(part * RPP + r) * LDG + d] = run;
  }
  tot[part * DK + d] = run;
}
template <int DK, int PARTS> __device__ __forceinline__ float kda_cumsum_before(const float* tot, int part, int d) {
  float off = 0.f;
#pragma unroll
  for (int p = 0; p < PARTS - 1; ++p) off += p < part ? tot[p * DK + d] : 0.f;
  return off;
}

// VEC consecutive fp32 values of an LDS row
template <int VEC> __device__ __forceinline__ void ld_f32(const float* p, float* f) {
#pragma unroll
  for (int e = 0; e < VEC; e += 4) {
    const f32x4 x = *reinterpret_cast<const f32x4*>(p + e);
    f[e] = x[0]; f[e + 1] = x[1]; f[e + 2] = x[2]; f[e + 3] = x[3];
  }
}

}  // namespace gdn
