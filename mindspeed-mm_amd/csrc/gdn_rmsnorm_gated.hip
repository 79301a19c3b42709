// Gated RMSNorm: the step right after the gated delta rule in the reference layer
// (Qwen3_5RMSNormGated.forward, mindspeed_mm/fsdp/models/qwen3_5/modeling_qwen3_5.py:330-349, called at :897-900 on
// rows of head_v_dim elements):
//     xn = x * rsqrt(mean(x^2) + eps)        (fp32, then cast to the input dtype)
//     y  = (weight * xn) * silu(gate)        (gate in fp32; result cast to the input dtype)
// Row-wise and bandwidth-bound: forward reads x, gate and writes y; backward reads x, gate, dy and writes dx, dgate.
// A row of N elements is held by N/VEC neighbouring lanes (16 bytes each); row sums use data-parallel-primitive moves.
// With gate_activation = 1 the gate passes through a sigmoid instead (the KDA layer's norm, KimiK_3_MoeRMSNormGated,
// mindspeed_mm/fsdp/models/kimi_k3/modeling_kimi_linear.py:75-96): s = cast(sigmoid(gate)).
// Backward, with t = weight * xn, s = silu(gate) or sigmoid(gate), xh = x * rstd in fp32:
//     dgate = dy t s'(gate)     dt = dy s     dweight = sum_rows dt xn     dxn = dt weight
//     dx = rstd (dxn - xh mean(dxn xh))
// dweight is accumulated per thread over the rows it visits, reduced inside the workgroup through LDS and written as one
// partial row per workgroup; rmsnorm_gated_dw_reduce_kernel adds the partials in a fixed order (bitwise reproducible).
#include "gdn_common.h"
#include "gdn_profile.h"
#include "gdn_rmsnorm_gated.h"

namespace gdn {

template <int LPR> __device__ __forceinline__ float row_lanes_sum(float v) {
  if constexpr (LPR <= 32) {
    return lane_group_sum<LPR>(v);
  } else {
    v = lane_group_sum<32>(v);
    return v + __shfl_xor(v, 32);
  }
}

// TW = T: weight in the input dtype, weight * xn is rounded to T as in the reference; TW = float: kept in fp32
template <typename T, typename TW, int LPR, int ACT>
__global__ __launch_bounds__(kThreads) void rmsnorm_gated_fwd_kernel(const T* __restrict__ x, const T* __restrict__ gate,
                                                                     const TW* __restrict__ weight, T* __restrict__ y,
                                                                     float* __restrict__ rstd_out, int64_t rows,
                                                                     float eps) {
  constexpr int V = Elem<T>::kVec, N = LPR * V, RPB = kThreads / LPR;
  const int c = threadIdx.x % LPR;
  float w[V];
  load_weight<T, TW>(w, weight + c * V);
  for (int64_t row = (int64_t)blockIdx.x * RPB + threadIdx.x / LPR; row < (rows + RPB - 1) / RPB * RPB;
       row += (int64_t)gridDim.x * RPB) {
    const bool ok = row < rows;      // uniform trip count: every lane takes part in the row sums
    const Vec16<T> xv = ok ? ld16(x + row * N + c * V) : zero16<T>();
    const Vec16<T> gv = ok ? ld16(gate + row * N + c * V) : zero16<T>();
    const float ss = row_lanes_sum<LPR>(piece_sumsq<T>(xv));
    const float rstd = rsqrtf(ss * (1.f / N) + eps);
    const Vec16<T> out = rmsnorm_gated_piece<T, TW, ACT>(xv, gv, w, rstd);
    if (ok) {
      __builtin_nontemporal_store(out.raw, reinterpret_cast<u32x4*>(y + row * N + c * V));
      if (c == 0) rstd_out[row] = rstd;
    }
  }
}

template <typename T, typename TW, int LPR, int ACT>
__global__ __launch_bounds__(kThreads) void rmsnorm_gated_bwd_kernel(
    const T* __restrict__ x, const T* __restrict__ gate, const TW* __restrict__ weight,
    const float* __restrict__ rstd_in, const T* __restrict__ dy, T* __restrict__ dx, T* __restrict__ dgate,
    float* __restrict__ part, int64_t rows) {
  constexpr int V = Elem<T>::kVec, N = LPR * V, RPB = kThreads / LPR;
  __shared__ float red[kThreads * V];
  const int c = threadIdx.x % LPR, rg = threadIdx.x / LPR;
  float w[V], dwa[V];
  load_weight<T, TW>(w, weight + c * V);
#pragma unroll
  for (int e = 0; e < V; ++e) dwa[e] = 0.f;
  for (int64_t row = (int64_t)blockIdx.x * RPB + rg; row < (rows + RPB - 1) / RPB * RPB;
       row += (int64_t)gridDim.x * RPB) {
    const bool ok = row < rows;
    const Vec16<T> xv = ok ? ld16(x + row * N + c * V) : zero16<T>();
    const Vec16<T> gv = ok ? ld16(gate + row * N + c * V) : zero16<T>();
    const Vec16<T> dv = ok ? ld16(dy + row * N + c * V) : zero16<T>();
    const float rstd = ok ? rstd_in[row] : 0.f;
    float dxn[V], xh[V], dot = 0.f;
    Vec16<T> dgo = zero16<T>(), dxo = zero16<T>();
#pragma unroll
    for (int e = 0; e < V; ++e) {
      xh[e] = xv.get(e) * rstd;
      const float xn = round_to<T>(xh[e]);
      const float t = sizeof(TW) == sizeof(T) ? round_to<T>(w[e] * xn) : w[e] * xn;
      const float gf = gv.get(e), sg = sigmoid_(gf), d = dv.get(e);
      dgo.set(e, ACT == 0 ? d * t * sg * (1.f + gf * (1.f - sg)) : d * t * sg * (1.f - sg));
      const float dt = ACT == 0 ? d * gf * sg : d * round_to<T>(sg);
      dwa[e] += dt * xn;
      dxn[e] = dt * w[e];
      dot += dxn[e] * xh[e];
    }
    dot = row_lanes_sum<LPR>(dot) * (1.f / N);
#pragma unroll
    for (int e = 0; e < V; ++e) dxo.set(e, rstd * (dxn[e] - xh[e] * dot));
    if (ok) {
      __builtin_nontemporal_store(dxo.raw, reinterpret_cast<u32x4*>(dx + row * N + c * V));
      __builtin_nontemporal_store(dgo.raw, reinterpret_cast<u32x4*>(dgate + row * N + c * V));
    }
  }
  // workgroup partial of dweight: add the RPB row groups in a fixed order
#pragma unroll
  for (int e = 0; e < V; ++e) red[threadIdx.x * V + e] = dwa[e];
  __syncthreads();
  for (int i = threadIdx.x; i < N; i += kThreads) {
    const int cc = i / V, e = i % V;
    float s = 0.f;
    for (int r = 0; r < RPB; ++r) s += red[(r * LPR + cc) * V + e];
    part[(int64_t)blockIdx.x * N + i] = s;
  }
}

// one workgroup per column: strided partial sums per thread, then a fixed-order tree through LDS
__global__ __launch_bounds__(kThreads) void rmsnorm_gated_dw_reduce_kernel(const float* __restrict__ part,
                                                                           float* __restrict__ dw, int nparts, int N) {
  __shared__ float red[kThreads];
  const int i = blockIdx.x;
  float s = 0.f;
  for (int p = threadIdx.x; p < nparts; p += kThreads) s += part[(int64_t)p * N + i];
  red[threadIdx.x] = s;
  __syncthreads();
  for (int m = kThreads / 2; m > 0; m >>= 1) {
    if ((int)threadIdx.x < m) red[threadIdx.x] += red[threadIdx.x + m];
    __syncthreads();
  }
  if (threadIdx.x == 0) dw[i] = red[0];
}

static int rmsnorm_blocks(int64_t rows, int rpb) {
  const int64_t need = (rows + rpb - 1) / rpb;
  return (int)(need < 2048 ? (need > 0 ? need : 1) : 2048);   // a few workgroups per CU, grid-stride over the rows
}

template <typename T, typename TW, int LPR>
static int rmsnorm_fwd_launch(const void* x, const void* gate, const void* weight, void* y, float* rstd, int64_t rows,
                              float eps, int act, hipStream_t st) {
  const dim3 grid(rmsnorm_blocks(rows, kThreads / LPR));
  if (act == 0)
    GDN_LAUNCH(kKernRmsNormFwd, st, (rmsnorm_gated_fwd_kernel<T, TW, LPR, 0>), grid, dim3(kThreads), 0, st, (const T*)x,
               (const T*)gate, (const TW*)weight, (T*)y, rstd, rows, eps);
  else
    GDN_LAUNCH(kKernRmsNormFwd, st, (rmsnorm_gated_fwd_kernel<T, TW, LPR, 1>), grid, dim3(kThreads), 0, st, (const T*)x,
               (const T*)gate, (const TW*)weight, (T*)y, rstd, rows, eps);
  return (int)hipGetLastError();
}

template <typename T, typename TW, int LPR>
static int rmsnorm_bwd_launch(const void* x, const void* gate, const void* weight, const float* rstd, const void* dy,
                              void* dx, void* dgate, float* dw, float* part, int64_t rows, int act, hipStream_t st) {
  constexpr int N = LPR * Elem<T>::kVec;
  const int nb = rmsnorm_blocks(rows, kThreads / LPR);
  if (act == 0)
    GDN_LAUNCH(kKernRmsNormBwd, st, (rmsnorm_gated_bwd_kernel<T, TW, LPR, 0>), dim3(nb), dim3(kThreads), 0, st, (const T*)x,
               (const T*)gate, (const TW*)weight, rstd, (const T*)dy, (T*)dx, (T*)dgate, part, rows);
  else
    GDN_LAUNCH(kKernRmsNormBwd, st, (rmsnorm_gated_bwd_kernel<T, TW, LPR, 1>), dim3(nb), dim3(kThreads), 0, st, (const T*)x,
               (const T*)gate, (const TW*)weight, rstd, (const T*)dy, (T*)dx, (T*)dgate, part, rows);
  GDN_LAUNCH(kKernRmsNormReduce, st, rmsnorm_gated_dw_reduce_kernel, dim3(N), dim3(kThreads), 0, st,
             (const float*)part, dw, nb, N);
  return (int)hipGetLastError();
}

// lanes per row for a row of N elements of `elem` bytes, or 0 if the size is not supported
static int rmsnorm_lpr(int N, int elem) {
  const int vec = 16 / elem;
  if (N <= 0 || N % vec != 0) return 0;
  const int lpr = N / vec;
  return (lpr == 4 || lpr == 8 || lpr == 16 || lpr == 32 || lpr == 64) ? lpr : 0;
}

}  // namespace gdn

#define GDN_RMS_DISPATCH(CALL)                                                          \
  switch (lpr) {                                                                        \
    case 4: return CALL(4);                                                             \
    case 8: return CALL(8);                                                             \
    case 16: return CALL(16);                                                           \
    case 32: return CALL(32);                                                           \
    default: return CALL(64);                                                           \
  }

extern "C" int gdn_rmsnorm_gated_fwd(const void* x, const void* gate, const void* weight, void* y, float* rstd,
                                     int64_t rows, int N, float eps, int dtype, int weight_dtype, int gate_activation,
                                     void* stream) {
  using namespace gdn;
  if (!x || !gate || !weight || !y || !rstd) return -1;
  if (rows < 0) return -2;
  if (dtype != 0 && dtype != 1) return -4;
  if (weight_dtype != 0 && weight_dtype != dtype) return -4;
  if (gate_activation != 0 && gate_activation != 1) return -4;
  const int lpr = rmsnorm_lpr(N, dtype == 0 ? 4 : 2);
  if (lpr == 0) return -3;
  if (rows == 0) return 0;
  hipStream_t st = (hipStream_t)stream;
  if (dtype == 0) {
#define CALL(L_) rmsnorm_fwd_launch<float, float, L_>(x, gate, weight, y, rstd, rows, eps, gate_activation, st)
    GDN_RMS_DISPATCH(CALL)
#undef CALL
  } else if (weight_dtype == 1) {
#define CALL(L_) rmsnorm_fwd_launch<bf16_t, bf16_t, L_>(x, gate, weight, y, rstd, rows, eps, gate_activation, st)
    GDN_RMS_DISPATCH(CALL)
#undef CALL
  } else {
#define CALL(L_) rmsnorm_fwd_launch<bf16_t, float, L_>(x, gate, weight, y, rstd, rows, eps, gate_activation, st)
    GDN_RMS_DISPATCH(CALL)
#undef CALL
  }
}

extern "C" int64_t gdn_rmsnorm_gated_bwd_workspace_bytes(int64_t rows, int N) {
  (void)rows;
  return (int64_t)2048 * (N > 0 ? N : 1) * (int64_t)sizeof(float);
}

extern "C" int gdn_rmsnorm_gated_bwd(const void* x, const void* gate, const void* weight, const float* rstd,
                                     const void* dy, void* dx, void* dgate, float* dweight, void* workspace,
                                     int64_t workspace_bytes, int64_t rows, int N, int dtype, int weight_dtype,
                                     int gate_activation, void* stream) {
  using namespace gdn;
  if (!x || !gate || !weight || !rstd || !dy || !dx || !dgate || !dweight || !workspace) return -1;
  if (rows < 0) return -2;
  if (dtype != 0 && dtype != 1) return -4;
  if (weight_dtype != 0 && weight_dtype != dtype) return -4;
  if (gate_activation != 0 && gate_activation != 1) return -4;
  const int lpr = rmsnorm_lpr(N, dtype == 0 ? 4 : 2);
  if (lpr == 0) return -3;
  if (workspace_bytes < gdn_rmsnorm_gated_bwd_workspace_bytes(rows, N)) return -5;
  hipStream_t st = (hipStream_t)stream;
  float* part = static_cast<float*>(workspace);
  if (rows == 0) {   // dweight = 0: the reduction over zero partials
    GDN_LAUNCH(kKernRmsNormReduce, st, rmsnorm_gated_dw_reduce_kernel, dim3(N), dim3(kThreads), 0, st,
               (const float*)part, dweight, 0, N);
    return (int)hipGetLastError();
  }
  if (dtype == 0) {
#define CALL(L_) rmsnorm_bwd_launch<float, float, L_>(x, gate, weight, rstd, dy, dx, dgate, dweight, part, rows, gate_activation, st)
    GDN_RMS_DISPATCH(CALL)
#undef CALL
  } else if (weight_dtype == 1) {
#define CALL(L_) rmsnorm_bwd_launch<bf16_t, bf16_t, L_>(x, gate, weight, rstd, dy, dx, dgate, dweight, part, rows, gate_activation, st)
    GDN_RMS_DISPATCH(CALL)
#undef CALL
  } else {
#define CALL(L_) rmsnorm_bwd_launch<bf16_t, float, L_>(x, gate, weight, rstd, dy, dx, dgate, dweight, part, rows, gate_activation, st)
    GDN_RMS_DISPATCH(CALL)
#undef CALL
  }
}
