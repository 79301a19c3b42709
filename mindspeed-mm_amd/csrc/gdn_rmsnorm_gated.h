// Arithmetic of the gated RMSNorm (Qwen3_5RMSNormGated.forward, mindspeed_mm/fsdp/models/qwen3_5/modeling_qwen3_5.py:330-349)
// on one 16-byte piece of a row, shared by the stand-alone kernels and by the output kernel of the chunked rule when
// it applies the norm in its epilogue: both must round at the same places and add in the same order to agree bit
// for bit.
//     xn = x * rsqrt(mean(x^2) + eps)        (fp32, then cast to the input dtype)
//     y  = (weight * xn) * silu(gate)        (gate in fp32; result cast to the input dtype)
// ACT = 1 is the norm of the KDA layer (KimiK_3_MoeRMSNormGated.forward,
// mindspeed_mm/fsdp/models/kimi_k3/modeling_kimi_linear.py:83-96): the gate passes through a sigmoid that is cast to
// the input dtype before the product,
//     y  = (weight * xn) * cast(sigmoid(gate))
#pragma once
#include "gdn_common.h"

namespace gdn {

__device__ __forceinline__ float sigmoid_(float p) { return 1.f / (1.f + __expf(-p)); }

// round to T and back: the reference casts to the input dtype between the steps
template <typename T> __device__ __forceinline__ float round_to(float x) { return Elem<T>::to_f(Elem<T>::from_f(x)); }

template <typename T, typename TW> __device__ __forceinline__ void load_weight(float* w, const TW* p) {
  constexpr int V = Elem<T>::kVec;
  if constexpr (sizeof(TW) == sizeof(T)) {
    const Vec16<TW> v = ld16(p);
#pragma unroll
    for (int e = 0; e < V; ++e) w[e] = v.get(e);
  } else {
#pragma unroll
    for (int e = 0; e < V; ++e) w[e] = Elem<TW>::to_f(p[e]);
  }
}

// sum of the squares of a piece's elements, added in element order
template <typename T> __device__ __forceinline__ float piece_sumsq(const Vec16<T>& xv) {
  float ss = 0.f;
#pragma unroll
  for (int e = 0; e < Elem<T>::kVec; ++e) { const float f = xv.get(e); ss += f * f; }
  return ss;
}

// TW = T: weight in the input dtype, weight * xn is rounded to T as in the reference; TW = float: kept in fp32
template <typename T, typename TW, int ACT = 0>
__device__ __forceinline__ Vec16<T> rmsnorm_gated_piece(const Vec16<T>& xv, const Vec16<T>& gv, const float* w, float rstd) {
  Vec16<T> out = zero16<T>();
#pragma unroll
  for (int e = 0; e < Elem<T>::kVec; ++e) {
    const float xn = round_to<T>(xv.get(e) * rstd);
    const float t = sizeof(TW) == sizeof(T) ? round_to<T>(w[e] * xn) : w[e] * xn;
    const float gf = gv.get(e);
    out.set(e, ACT == 0 ? t * (gf * sigmoid_(gf)) : t * round_to<T>(sigmoid_(gf)));
  }
  return out;
}

}  // namespace gdn
