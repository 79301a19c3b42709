// Gates of the gated delta rule from the layer's projections, one pass instead of a chain of elementwise launches:
//     beta = sigmoid(b)                                        (in b's dtype)
//     g    = -exp(A_log) * softplus(a + dt_bias)               (fp32; a, A_log, dt_bias promoted to fp32 first)
// with a, b [tokens, Hv] and A_log, dt_bias [Hv], as in Qwen3_5GatedDeltaNet.forward
// (mindspeed_mm/fsdp/models/qwen3_5/modeling_qwen3_5.py:833-841).  softplus is torch's: x for x > 20, log1p(exp(x)) else.
// Backward, given dg (fp32) and dbeta (b's dtype):
//     db = dbeta * beta (1 - beta)        da = dg * (-exp(A_log)) * sigmoid(a + dt_bias)
//     ddt_bias[h] = sum_t da[t,h] (before rounding)            dA_log[h] = sum_t dg[t,h] * g[t,h]
// The sums over tokens are formed in a fixed order (per-thread, per-workgroup, then one workgroup per head), so the
// result does not depend on scheduling.
#include "gdn_common.h"
#include "gdn_profile.h"

#include <mutex>

namespace gdn {

// Partial sums of gdn_gate_bwd_noalloc: [workgroups <= 1024][2][Hv <= kGateNoAllocMaxHv] fp32, 1 MiB per device, held
// until the process ends.  Every slot a launch reads has been written by the same launch, so nothing needs clearing.
constexpr int kGateNoAllocMaxHv = 128;
constexpr int kGateMaxBlocks = 1024;
static __device__ __align__(256) float gate_scratch[kGateMaxBlocks * 2 * kGateNoAllocMaxHv];

template <typename T> __device__ __forceinline__ float gate_ld(const T* p, int64_t i) { return Elem<T>::to_f(p[i]); }
__device__ __forceinline__ float gate_sigmoid(float x) { return 1.f / (1.f + expf(-x)); }
__device__ __forceinline__ float gate_softplus(float x) { return x > 20.f ? x : log1pf(expf(x)); }

template <typename T, typename TP>
__global__ __launch_bounds__(kThreads) void gate_fwd_kernel(const T* __restrict__ a, const T* __restrict__ b,
                                                            const TP* __restrict__ A_log, const TP* __restrict__ dt_bias,
                                                            float* __restrict__ g, T* __restrict__ beta, int64_t n, int Hv) {
  for (int64_t i = (int64_t)blockIdx.x * kThreads + threadIdx.x; i < n; i += (int64_t)gridDim.x * kThreads) {
    const int h = (int)(i % Hv);
    beta[i] = Elem<T>::from_f(gate_sigmoid(gate_ld(b, i)));
    g[i] = -expf(gate_ld(A_log, h)) * gate_softplus(gate_ld(a, i) + gate_ld(dt_bias, h));
  }
}

// A workgroup covers kThreads / Hv tokens per pass, thread t always the head t % Hv; part [blocks][2][Hv].
template <typename T, typename TP>
__global__ __launch_bounds__(kThreads) void gate_bwd_kernel(const T* __restrict__ a, const T* __restrict__ b,
                                                            const TP* __restrict__ A_log, const TP* __restrict__ dt_bias,
                                                            const float* __restrict__ dg, const T* __restrict__ dbeta,
                                                            T* __restrict__ da, T* __restrict__ db,
                                                            float* __restrict__ part, int64_t tokens, int Hv) {
  __shared__ float red[2 * kThreads];
  const int rows = kThreads / Hv, tid = threadIdx.x, h = tid % Hv, r = tid / Hv;
  float s_bias = 0.f, s_alog = 0.f;
  if (r < rows) {
    const float na = -expf(gate_ld(A_log, h)), bias = gate_ld(dt_bias, h);
    for (int64_t t = (int64_t)blockIdx.x * rows + r; t < tokens; t += (int64_t)gridDim.x * rows) {
      const int64_t i = t * Hv + h;
      const float s = gate_sigmoid(gate_ld(b, i));
      db[i] = Elem<T>::from_f(gate_ld(dbeta, i) * s * (1.f - s));
      const float x = gate_ld(a, i) + bias, d = dg[i];
      const float dx = d * na * (x > 20.f ? 1.f : gate_sigmoid(x));
      da[i] = Elem<T>::from_f(dx);
      s_bias += dx;
      s_alog += d * na * gate_softplus(x);
    }
  }
  red[tid] = s_bias;
  red[kThreads + tid] = s_alog;
  __syncthreads();
  if (tid < Hv) {
    float sb = 0.f, sa = 0.f;
    for (int q = 0; q < rows; ++q) { sb += red[q * Hv + tid]; sa += red[kThreads + q * Hv + tid]; }
    part[((int64_t)blockIdx.x * 2 + 0) * Hv + tid] = sb;
    part[((int64_t)blockIdx.x * 2 + 1) * Hv + tid] = sa;
  }
}

// one workgroup per (head, which): strided partial sums per thread, then a fixed-order tree through LDS
__global__ __launch_bounds__(kThreads) void gate_reduce_kernel(const float* __restrict__ part, float* __restrict__ ddt_bias,
                                                               float* __restrict__ dA_log, int nparts, int Hv) {
  __shared__ float red[kThreads];
  const int h = blockIdx.x, which = blockIdx.y;
  float s = 0.f;
  for (int p = threadIdx.x; p < nparts; p += kThreads) s += part[((int64_t)p * 2 + which) * Hv + h];
  red[threadIdx.x] = s;
  __syncthreads();
  for (int m = kThreads / 2; m > 0; m >>= 1) {
    if ((int)threadIdx.x < m) red[threadIdx.x] += red[threadIdx.x + m];
    __syncthreads();
  }
  if (threadIdx.x == 0) (which == 0 ? ddt_bias : dA_log)[h] = red[0];
}

static int gate_bwd_blocks(int64_t tokens, int Hv) {
  const int rows = kThreads / Hv;
  const int64_t need = (tokens + rows - 1) / rows;
  return (int)(need < kGateMaxBlocks ? (need > 0 ? need : 1) : kGateMaxBlocks);
}

template <typename T, typename TP>
static int gate_fwd_launch(const void* a, const void* b, const void* A_log, const void* dt_bias, float* g, void* beta,
                           int64_t tokens, int Hv, hipStream_t st) {
  const int64_t n = tokens * Hv, need = (n + kThreads - 1) / kThreads;
  GDN_LAUNCH(kKernGateFwd, st, (gate_fwd_kernel<T, TP>), dim3((int)(need < 4096 ? need : 4096)), dim3(kThreads), 0, st,
             (const T*)a, (const T*)b, (const TP*)A_log, (const TP*)dt_bias, g, (T*)beta, n, Hv);
  return (int)hipGetLastError();
}

template <typename T, typename TP>
static int gate_bwd_launch(const void* a, const void* b, const void* A_log, const void* dt_bias, const float* dg,
                           const void* dbeta, void* da, void* db, float* dA_log, float* ddt_bias, float* part,
                           int64_t tokens, int Hv, hipStream_t st) {
  const int nb = gate_bwd_blocks(tokens, Hv);
  GDN_LAUNCH(kKernGateBwd, st, (gate_bwd_kernel<T, TP>), dim3(nb), dim3(kThreads), 0, st, (const T*)a, (const T*)b,
             (const TP*)A_log, (const TP*)dt_bias, dg, (const T*)dbeta, (T*)da, (T*)db, part, tokens, Hv);
  GDN_LAUNCH(kKernGateReduce, st, gate_reduce_kernel, dim3(Hv, 2), dim3(kThreads), 0, st, (const float*)part, ddt_bias,
             dA_log, nb, Hv);
  return (int)hipGetLastError();
}

static int gate_check(int64_t tokens, int Hv, int dtype, int param_dtype) {
  if (tokens < 0 || Hv <= 0) return -2;
  if (Hv > kThreads) return -3;
  if (dtype != 0 && dtype != 1) return -4;
  if (param_dtype != 0 && param_dtype != dtype) return -4;
  return 0;
}

}  // namespace gdn

extern "C" int gdn_gate_fwd(const void* a, const void* b, const void* A_log, const void* dt_bias, float* g, void* beta,
                            int64_t tokens, int Hv, int dtype, int param_dtype, void* stream) {
  using namespace gdn;
  if (!a || !b || !A_log || !dt_bias || !g || !beta) return -1;
  if (int e = gate_check(tokens, Hv, dtype, param_dtype)) return e;
  if (tokens == 0) return 0;
  hipStream_t st = (hipStream_t)stream;
  if (dtype == 0) return gate_fwd_launch<float, float>(a, b, A_log, dt_bias, g, beta, tokens, Hv, st);
  if (param_dtype == 1) return gate_fwd_launch<bf16_t, bf16_t>(a, b, A_log, dt_bias, g, beta, tokens, Hv, st);
  return gate_fwd_launch<bf16_t, float>(a, b, A_log, dt_bias, g, beta, tokens, Hv, st);
}

extern "C" int64_t gdn_gate_bwd_workspace_bytes(int64_t tokens, int Hv) {
  if (tokens < 0 || Hv <= 0 || Hv > gdn::kThreads) return 0;
  return (int64_t)gdn::gate_bwd_blocks(tokens, Hv) * 2 * Hv * 4;
}

extern "C" int gdn_gate_bwd(const void* a, const void* b, const void* A_log, const void* dt_bias, const float* dg,
                            const void* dbeta, void* da, void* db, float* dA_log, float* ddt_bias, void* workspace,
                            int64_t workspace_bytes, int64_t tokens, int Hv, int dtype, int param_dtype, void* stream) {
  using namespace gdn;
  if (!a || !b || !A_log || !dt_bias || !dg || !dbeta || !da || !db || !dA_log || !ddt_bias || !workspace) return -1;
  if (int e = gate_check(tokens, Hv, dtype, param_dtype)) return e;
  if (workspace_bytes < gdn_gate_bwd_workspace_bytes(tokens, Hv)) return -5;
  hipStream_t st = (hipStream_t)stream;
  float* part = static_cast<float*>(workspace);
  if (dtype == 0)
    return gate_bwd_launch<float, float>(a, b, A_log, dt_bias, dg, dbeta, da, db, dA_log, ddt_bias, part, tokens, Hv, st);
  if (param_dtype == 1)
    return gate_bwd_launch<bf16_t, bf16_t>(a, b, A_log, dt_bias, dg, dbeta, da, db, dA_log, ddt_bias, part, tokens, Hv, st);
  return gate_bwd_launch<bf16_t, float>(a, b, A_log, dt_bias, dg, dbeta, da, db, dA_log, ddt_bias, part, tokens, Hv, st);
}

namespace gdn {
// Device address of gate_scratch on the current device.  In host code the array's name is only a handle: the address
// a kernel may use comes from hipGetSymbolAddress, once per device (each device holds its own copy).
static int gate_scratch_ptr(float** out) {
  constexpr int kMaxDevices = 64;
  static std::mutex mu;
  static float* ptrs[kMaxDevices] = {};
  int dev = 0;
  if (hipError_t e = hipGetDevice(&dev)) return (int)e;
  if (dev < 0 || dev >= kMaxDevices) return -2;
  std::lock_guard<std::mutex> lk(mu);
  if (ptrs[dev] == nullptr) {
    void* p = nullptr;
    if (hipError_t e = hipGetSymbolAddress(&p, HIP_SYMBOL(gate_scratch))) return (int)e;
    if (p == nullptr) return -1;
    ptrs[dev] = static_cast<float*>(p);
  }
  *out = ptrs[dev];
  return 0;
}
}  // namespace gdn

extern "C" int gdn_gate_bwd_noalloc(const void* a, const void* b, const void* A_log, const void* dt_bias,
                                    const float* dg, const void* dbeta, void* da, void* db, float* dA_log,
                                    float* ddt_bias, int64_t tokens, int Hv, int dtype, int param_dtype, void* stream) {
  using namespace gdn;
  if (!a || !b || !A_log || !dt_bias || !dg || !dbeta || !da || !db || !dA_log || !ddt_bias) return -1;
  if (int e = gate_check(tokens, Hv, dtype, param_dtype)) return e;
  if (Hv > kGateNoAllocMaxHv) return -3;   // the partial sums would not fit the library's own buffer
  float* part = nullptr;
  if (int e = gate_scratch_ptr(&part)) return e;
  hipStream_t st = (hipStream_t)stream;
  if (dtype == 0)
    return gate_bwd_launch<float, float>(a, b, A_log, dt_bias, dg, dbeta, da, db, dA_log, ddt_bias, part, tokens, Hv, st);
  if (param_dtype == 1)
    return gate_bwd_launch<bf16_t, bf16_t>(a, b, A_log, dt_bias, dg, dbeta, da, db, dA_log, ddt_bias, part, tokens, Hv, st);
  return gate_bwd_launch<bf16_t, float>(a, b, A_log, dt_bias, dg, dbeta, da, db, dA_log, ddt_bias, part, tokens, Hv, st);
}
