// Fused recurrent gated delta rule (decode).  Per (sequence b, value head h) and token t:
//     S <- e^{g} S;  delta = beta (v - S^T k);  S <- S + k delta^T;  o = scale S^T q
// (reference math: mindspeed_mm/fsdp/models/qwen3_5/modeling_qwen3_5.py:478-517).
//
// The kernel is bound by streaming the fp32 state [K,V] (64 KB at K=V=128) through HBM once in, once
// out.  One workgroup of 256 threads owns a [K, BV] column slab of one state; the slab lives in
// registers for all T tokens of the call.  With S_old the state before the token,
//     S^T k = e^g (S_old^T k),   S^T q = e^g (S_old^T q) + (k.q) delta
// so both contractions are taken in ONE pass over the registers, then the rank-1 update is applied.
// No MFMA: 6 flop per 8 bytes of state traffic, far below the matrix-core ridge.
//
// q, k, v are read with a token stride, so they can be the column ranges of the convolution's [tokens, D] output, and
// the gates can be formed here from the layer's projections (g = -exp(A_log) softplus(a + dt_bias), beta = sigmoid(b)
// rounded to b's dtype as the layer's `b.sigmoid()` is; modeling_qwen3_5.py:833-841) instead of being passed in: a
// decode step of the layer is then the convolution update followed by this kernel, with no copies in between.
#include "gdn_common.h"
#include "gdn_profile.h"

namespace gdn {

struct RecurrentGates {   // either g, beta (fp32 [tokens,Hv]) or the projections a, b [tokens,Hv] and A_log, dt_bias [Hv]
  const float* g;
  const float* beta;
  const void* a;
  const void* b;
  const void* A_log;
  const void* dt_bias;
};

template <typename T, typename TP, int DK, int BV>
__global__ __launch_bounds__(256) void recurrent_kernel(
    const T* __restrict__ q, const T* __restrict__ k, const T* __restrict__ v, int64_t sq, int64_t sk, int64_t sv,
    RecurrentGates gates, const float* state_in, float* state_out, T* __restrict__ o, const int64_t* __restrict__ cu,
    int B, int T_len, int Hqk, int Hv, int V, float scale, int use_l2norm) {
  constexpr int CG = BV / 4;            // column groups (4 fp32 = 16 bytes each)
  constexpr int NRG = kThreads / CG;    // row groups
  constexpr int RPT = DK / NRG;         // state rows held by a thread
  constexpr int RGW = 64 / CG;          // row groups inside one wave
  static_assert(DK % NRG == 0 && RPT >= 1, "tile shape");
  __shared__ float ks[DK], qs[DK], red[4][CG][8], red3[4][3];

  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int cg = tid % CG, rg = tid / CG;
  const int b = blockIdx.x / Hv, h = blockIdx.x % Hv, hq = h / (Hv / Hqk);
  const int v0 = blockIdx.y * BV + cg * 4;
  const int64_t sbase = ((int64_t)(b * Hv + h) * DK) * V + v0;

  float S[RPT][4];
#pragma unroll
  for (int i = 0; i < RPT; ++i) {
    const int row = rg + NRG * i;
    if (state_in != nullptr) {
      const f32x4 x = *reinterpret_cast<const f32x4*>(state_in + sbase + (int64_t)row * V);
      S[i][0] = x[0]; S[i][1] = x[1]; S[i][2] = x[2]; S[i][3] = x[3];
    } else {
      S[i][0] = S[i][1] = S[i][2] = S[i][3] = 0.f;
    }
  }

  // packed input (cu given): "sequence" b owns the tokens cu[b] .. cu[b+1] of the one batch row
  const int64_t tok0 = cu != nullptr ? cu[b] : (int64_t)b * T_len;
  const int ntok = cu != nullptr ? (int)(cu[b + 1] - cu[b]) : T_len;
  for (int t = 0; t < ntok; ++t) {
    const int64_t tok = tok0 + t;
    // ---- q, k of this token: optional l2 norm, q pre-scaled ----
    float kv_ = 0.f, qv_ = 0.f;
    if (tid < DK) {
      kv_ = Elem<T>::to_f(k[tok * sk + hq * DK + tid]);
      qv_ = Elem<T>::to_f(q[tok * sq + hq * DK + tid]);
    }
    const float sk = wave_sum(kv_ * kv_), sq = wave_sum(qv_ * qv_), skq = wave_sum(kv_ * qv_);
    if (lane == 0) { red3[wave][0] = sk; red3[wave][1] = sq; red3[wave][2] = skq; }
    __syncthreads();
    const float tk = red3[0][0] + red3[1][0] + red3[2][0] + red3[3][0];
    const float tq = red3[0][1] + red3[1][1] + red3[2][1] + red3[3][1];
    float kq = red3[0][2] + red3[1][2] + red3[2][2] + red3[3][2];
    float rk = 1.f, rq = scale;
    if (use_l2norm) { rk = rsqrtf(tk + 1e-6f); rq = scale * rsqrtf(tq + 1e-6f); }
    kq *= rk * rq;
    if (tid < DK) { ks[tid] = kv_ * rk; qs[tid] = qv_ * rq; }
    __syncthreads();

    // ---- one pass over the slab: S_old^T k and S_old^T q ----
    float pk[4] = {0.f, 0.f, 0.f, 0.f}, pq[4] = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int i = 0; i < RPT; ++i) {
      const float kk = ks[rg + NRG * i], qq = qs[rg + NRG * i];
#pragma unroll
      for (int c = 0; c < 4; ++c) { pk[c] += S[i][c] * kk; pq[c] += S[i][c] * qq; }
    }
#pragma unroll
    for (int m = CG; m < 64; m <<= 1) {
#pragma unroll
      for (int c = 0; c < 4; ++c) { pk[c] += __shfl_xor(pk[c], m); pq[c] += __shfl_xor(pq[c], m); }
    }
    if (lane < CG) {
#pragma unroll
      for (int c = 0; c < 4; ++c) { red[wave][cg][c] = pk[c]; red[wave][cg][4 + c] = pq[c]; }
    }
    __syncthreads();

    float eg, bt;
    if (gates.a == nullptr) {
      eg = __expf(gates.g[tok * Hv + h]);
      bt = gates.beta[tok * Hv + h];
    } else {
      const float x = Elem<T>::to_f(static_cast<const T*>(gates.a)[tok * Hv + h]) +
                      Elem<TP>::to_f(static_cast<const TP*>(gates.dt_bias)[h]);
      const float sp = x > 20.f ? x : log1pf(expf(x));
      eg = __expf(-expf(Elem<TP>::to_f(static_cast<const TP*>(gates.A_log)[h])) * sp);   // as __expf(g) of a passed-in g
      const float sg = 1.f / (1.f + expf(-Elem<T>::to_f(static_cast<const T*>(gates.b)[tok * Hv + h])));
      bt = Elem<T>::to_f(Elem<T>::from_f(sg));
    }
    float delta[4], ov[4];
    Vec16<T> vv;
    if constexpr (sizeof(T) == 4) {
      vv = ld16(v + tok * sv + h * V + v0);
    } else {
      const u32x2 w = *reinterpret_cast<const u32x2*>(v + tok * sv + h * V + v0);
      vv.raw = u32x4{w[0], w[1], 0u, 0u};
    }
#pragma unroll
    for (int c = 0; c < 4; ++c) {
      const float skv = red[0][cg][c] + red[1][cg][c] + red[2][cg][c] + red[3][cg][c];
      const float sqv = red[0][cg][4 + c] + red[1][cg][4 + c] + red[2][cg][4 + c] + red[3][cg][4 + c];
      delta[c] = bt * (vv.get(c) - eg * skv);
      ov[c] = eg * sqv + kq * delta[c];
    }
    // ---- rank-1 update in registers ----
#pragma unroll
    for (int i = 0; i < RPT; ++i) {
      const float kk = ks[rg + NRG * i];
#pragma unroll
      for (int c = 0; c < 4; ++c) S[i][c] = eg * S[i][c] + kk * delta[c];
    }
    if (rg == 0) {
      T* op = o + (tok * Hv + h) * V + v0;
      if constexpr (sizeof(T) == 4) {
        *reinterpret_cast<f32x4*>(op) = f32x4{ov[0], ov[1], ov[2], ov[3]};
      } else {
        Vec16<T> ow = zero16<T>();
#pragma unroll
        for (int c = 0; c < 4; ++c) ow.set(c, ov[c]);
        *reinterpret_cast<u32x2*>(op) = u32x2{ow.raw[0], ow.raw[1]};
      }
    }
    // red/ks/qs are rewritten only after the next token's first barrier
  }

  if (state_out != nullptr) {
#pragma unroll
    for (int i = 0; i < RPT; ++i) {
      const int row = rg + NRG * i;
      // streaming store: the slab is not read again by this kernel, and keeping it out of the L2 on its way to
      // memory leaves the cache to the loads (measured: 219 -> 163 us per batch-256 step)
      __builtin_nontemporal_store(f32x4{S[i][0], S[i][1], S[i][2], S[i][3]},
                                  reinterpret_cast<f32x4*>(state_out + sbase + (int64_t)row * V));
    }
  }
  (void)RGW; (void)B;
}

template <typename T, typename TP>
static int launch_recurrent(const void* q, const void* k, const void* v, int64_t sq, int64_t sk, int64_t sv,
                            const RecurrentGates& gates, const float* state_in, float* state_out, void* o, int B,
                            int T_len, int Hqk, int Hv, int K, int V, float scale, int use_l2norm, hipStream_t stream,
                            const int64_t* cu = nullptr) {
#define GDN_REC(DK_, BV_)                                                                                          \
  GDN_LAUNCH(kKernRecurrent, stream, (recurrent_kernel<T, TP, DK_, BV_>), dim3(B * Hv, V / BV_), dim3(kThreads), 0, \
             stream, (const T*)q, (const T*)k, (const T*)v, sq, sk, sv, gates, state_in, state_out, (T*)o, cu, B,     \
             T_len, Hqk, Hv, V, scale, use_l2norm)
  const bool wide = (V % 128 == 0);
  if (K == 64 && wide) GDN_REC(64, 128);
  else if (K == 64) GDN_REC(64, 64);
  else if (K == 128 && wide) GDN_REC(128, 128);
  else if (K == 128) GDN_REC(128, 64);
  else if (K == 256 && wide) GDN_REC(256, 128);
  else if (K == 256) GDN_REC(256, 64);
  else return -3;
#undef GDN_REC
  return (int)hipGetLastError();
}

static int recurrent_check(int B, int T, int Hqk, int Hv, int V) {
  if (B <= 0 || T < 0 || Hqk <= 0 || Hv <= 0 || Hv % Hqk != 0) return -2;
  if (V % 64 != 0 || V <= 0) return -3;
  return 0;
}

}  // namespace gdn

extern "C" int gdn_recurrent_fwd(const void* q, const void* k, const void* v, const float* g, const float* beta,
                                 const float* state_in, float* state_out, void* o, int B, int T, int Hqk, int Hv,
                                 int K, int V, float scale, int use_qk_l2norm, int dtype, void* stream) {
  using namespace gdn;
  if (!q || !k || !v || !g || !beta || !o) return -1;
  if (int e = recurrent_check(B, T, Hqk, Hv, V)) return e;
  if (T == 0 && state_out == nullptr) return 0;
  hipStream_t s = (hipStream_t)stream;
  const RecurrentGates gates{g, beta, nullptr, nullptr, nullptr, nullptr};
  const int64_t nq = (int64_t)Hqk * K, nv = (int64_t)Hv * V;
  if (dtype == 0)
    return launch_recurrent<float, float>(q, k, v, nq, nq, nv, gates, state_in, state_out, o, B, T, Hqk, Hv, K, V, scale,
                                          use_qk_l2norm, s);
  if (dtype == 1)
    return launch_recurrent<bf16_t, float>(q, k, v, nq, nq, nv, gates, state_in, state_out, o, B, T, Hqk, Hv, K, V, scale,
                                           use_qk_l2norm, s);
  return -4;
}

extern "C" int gdn_recurrent_fwd_packed(const void* q, const void* k, const void* v, const float* g, const float* beta,
                                        const float* state_in, float* state_out, void* o, const int64_t* cu_seqlens,
                                        int N, int T, int Hqk, int Hv, int K, int V, float scale, int use_qk_l2norm,
                                        int dtype, void* stream) {
  using namespace gdn;
  if (!q || !k || !v || !g || !beta || !o || !cu_seqlens) return -1;
  if (int e = recurrent_check(N, T, Hqk, Hv, V)) return e;
  hipStream_t s = (hipStream_t)stream;
  const RecurrentGates gates{g, beta, nullptr, nullptr, nullptr, nullptr};
  const int64_t nq = (int64_t)Hqk * K, nv = (int64_t)Hv * V;
  if (dtype == 0)
    return launch_recurrent<float, float>(q, k, v, nq, nq, nv, gates, state_in, state_out, o, N, T, Hqk, Hv, K, V, scale,
                                          use_qk_l2norm, s, cu_seqlens);
  if (dtype == 1)
    return launch_recurrent<bf16_t, float>(q, k, v, nq, nq, nv, gates, state_in, state_out, o, N, T, Hqk, Hv, K, V, scale,
                                           use_qk_l2norm, s, cu_seqlens);
  return -4;
}

extern "C" int gdn_recurrent_fwd_qkv(const void* qkv, int64_t token_stride, const void* a, const void* b,
                                     const void* A_log, const void* dt_bias, const float* state_in, float* state_out,
                                     void* o, int B, int T, int Hqk, int Hv, int K, int V, float scale,
                                     int use_qk_l2norm, int dtype, int param_dtype, void* stream) {
  using namespace gdn;
  if (!qkv || !a || !b || !A_log || !dt_bias || !o) return -1;
  if (int e = recurrent_check(B, T, Hqk, Hv, V)) return e;
  if (dtype != 0 && dtype != 1) return -4;
  if (param_dtype != 0 && param_dtype != dtype) return -4;
  const int64_t nq = (int64_t)Hqk * K, nv = (int64_t)Hv * V, vec = dtype == 0 ? 4 : 8, es = dtype == 0 ? 4 : 2;
  if (token_stride < 2 * nq + nv || token_stride % vec != 0 || ((uintptr_t)qkv & 15) != 0) return -6;
  if (T == 0 && state_out == nullptr) return 0;
  hipStream_t s = (hipStream_t)stream;
  const RecurrentGates gates{nullptr, nullptr, a, b, A_log, dt_bias};
  const char* base = static_cast<const char*>(qkv);
  const void *q = base, *k = base + nq * es, *v = base + 2 * nq * es;
  if (dtype == 0)
    return launch_recurrent<float, float>(q, k, v, token_stride, token_stride, token_stride, gates, state_in, state_out,
                                          o, B, T, Hqk, Hv, K, V, scale, use_qk_l2norm, s);
  if (param_dtype == 1)
    return launch_recurrent<bf16_t, bf16_t>(q, k, v, token_stride, token_stride, token_stride, gates, state_in,
                                            state_out, o, B, T, Hqk, Hv, K, V, scale, use_qk_l2norm, s);
  return launch_recurrent<bf16_t, float>(q, k, v, token_stride, token_stride, token_stride, gates, state_in, state_out,
                                         o, B, T, Hqk, Hv, K, V, scale, use_qk_l2norm, s);
}
