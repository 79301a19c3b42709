// Causal short depthwise conv1d (+SiLU) over token-major activations x[B,T,D], weight[W,D]:
//     y[t,d] = act( sum_{w<W} xpad[t-(W-1)+w, d] * weight[w,d] + bias[d] ) (+ residual[t,d])
// where xpad reads the sequence's initial_state[n,d,W+tau] for tau = position - sequence start < 0
// (zero when there is none) and never crosses a cu_seqlens boundary.
// Reference semantics: mindspeed_mm/fsdp/ops/gdn/triton/convolution.py:41-181 (fwd), :193-514 (bwd),
// :723-759 (final state); tests/ut_fsdp/models/qwen3_5/test_causal_conv1d/reference_impl.py:18-102;
// decode update mindspeed_mm/fsdp/models/qwen3_5/modeling_qwen3_5.py:373-389.
//
// All kernels are HBM bound (2*W flop per element).  A thread owns 16 bytes of channels (8 bf16 /
// 4 fp32) and walks a tile of consecutive tokens with the last W inputs in registers, so x is read
// once; the backward pass recomputes the pre-activation in registers instead of re-reading y.
#include "gdn_common.h"
#include "gdn_profile.h"

namespace gdn {

constexpr int kConvThreads = 128;

struct SeqCursor {  // which sequence a flattened token index belongs to
  const int64_t* cu; int N; int T; int n; int64_t bos, eos;
  __device__ __forceinline__ void init(const int64_t* cu_, int N_, int T_, int64_t t) {
    cu = cu_; N = N_; T = T_;
    if (cu == nullptr) { n = (int)(t / T); bos = (int64_t)n * T; eos = bos + T; return; }
    int lo = 0, hi = N - 1;
    while (lo < hi) { const int mid = (lo + hi + 1) >> 1; if (cu[mid] <= t) lo = mid; else hi = mid - 1; }
    n = lo; bos = cu[n]; eos = cu[n + 1];
    while (t >= eos && n + 1 < N) { ++n; bos = eos; eos = cu[n + 1]; }  // skip empty sequences
  }
  __device__ __forceinline__ bool advance_to(int64_t t) {  // returns true if a new sequence was entered
    bool moved = false;
    while (t >= eos && n + 1 < N) {
      ++n; bos = eos; eos = (cu == nullptr) ? bos + T : cu[n + 1]; moved = true;
    }
    return moved;
  }
};

template <typename T, int V> struct ChanVec { float x[V]; };

template <typename T> __device__ __forceinline__ void unpack_chan(float* dst, const Vec16<T>& v) {
#pragma unroll
  for (int e = 0; e < Elem<T>::kVec; ++e) dst[e] = v.get(e);
}
template <typename T> __device__ __forceinline__ void load_chan(float* dst, const T* p) { unpack_chan(dst, ld16(p)); }
// tokens whose rows are requested together before any of them is used: a thread walks its channels token by token,
// and without this only one 16-byte load per thread would be in flight
constexpr int kConvAhead = 4;
template <typename T> __device__ __forceinline__ void store_chan(T* p, const float* src) {
  Vec16<T> v = zero16<T>();
#pragma unroll
  for (int e = 0; e < Elem<T>::kVec; ++e) v.set(e, src[e]);
  // streaming store: outputs are not read again by these kernels, the L2 stays with the sliding input window
  __builtin_nontemporal_store(v.raw, reinterpret_cast<u32x4*>(p));
}

// input at flattened position tau for the sequence described by cur (tau may precede the sequence)
template <typename T>
__device__ __forceinline__ void load_hist(float* dst, const T* x, const T* init, int64_t tau, const SeqCursor& cur,
                                          int D, int W, int d0) {
  constexpr int V = Elem<T>::kVec;
  if (tau >= cur.bos) { load_chan(dst, x + tau * D + d0); return; }
  const int j = W + (int)(tau - cur.bos);
  if (init != nullptr && j >= 1) {
#pragma unroll
    for (int e = 0; e < V; ++e) dst[e] = Elem<T>::to_f(init[((int64_t)cur.n * D + d0 + e) * W + j]);
  } else {
#pragma unroll
    for (int e = 0; e < V; ++e) dst[e] = 0.f;
  }
}

// v_rcp_f32 (1 ulp) instead of an IEEE division: ten instructions fewer per element
__device__ __forceinline__ float sigmoidf_(float p) { return __builtin_amdgcn_rcpf(1.f + __expf(-p)); }

template <typename T, int W>
__global__ __launch_bounds__(kConvThreads) GDN_WAVES_PER_SIMD(W <= 4 ? 4 : 2) void conv1d_fwd_kernel(
    const T* __restrict__ x, const T* __restrict__ weight, const T* __restrict__ bias, const T* __restrict__ residual,
    const T* __restrict__ init, const int64_t* __restrict__ cu, T* __restrict__ y, int64_t total, int T_len, int N,
    int D, int tile, int silu) {
  constexpr int V = Elem<T>::kVec;
  // one linear grid, channel blocks fastest: the number of token tiles is not bounded by the y dimension's 65535
  const int nbd = (D / V + kConvThreads - 1) / kConvThreads, bx = blockIdx.x % nbd;
  const int64_t by = blockIdx.x / nbd;
  const int d0 = (bx * kConvThreads + threadIdx.x) * V;
  if (d0 >= D) return;
  const int64_t t0 = by * tile;
  const int64_t t1 = t0 + tile < total ? t0 + tile : total;
  float wgt[W][V], bs[V], win[W][V];
#pragma unroll
  for (int w = 0; w < W; ++w) load_chan(wgt[w], weight + (int64_t)w * D + d0);
#pragma unroll
  for (int e = 0; e < V; ++e) bs[e] = 0.f;
  if (bias != nullptr) load_chan(bs, bias + d0);
  SeqCursor cur;
  cur.init(cu, N, T_len, t0);
#pragma unroll
  for (int w = 0; w < W - 1; ++w) load_hist(win[w], x, init, t0 - (W - 1) + w, cur, D, W, d0);
  for (int64_t tb = t0; tb < t1; tb += kConvAhead) {
    Vec16<T> xr[kConvAhead];
#pragma unroll
    for (int u = 0; u < kConvAhead; ++u)
      if (tb + u < t1) xr[u] = ld16(x + (tb + u) * D + d0);
#pragma unroll
    for (int u = 0; u < kConvAhead; ++u) {
      const int64_t t = tb + u;
      if (t >= t1) break;
      if (cur.advance_to(t)) {
#pragma unroll
        for (int w = 0; w < W - 1; ++w) load_hist(win[w], x, init, t - (W - 1) + w, cur, D, W, d0);
      }
      unpack_chan(win[W - 1], xr[u]);
      float out[V];
#pragma unroll
      for (int e = 0; e < V; ++e) {
        float a = bs[e];
#pragma unroll
        for (int w = 0; w < W; ++w) a += win[w][e] * wgt[w][e];
        out[e] = silu ? a * sigmoidf_(a) : a;
      }
      if (residual != nullptr) {
        float r[V];
        load_chan(r, residual + t * D + d0);
#pragma unroll
        for (int e = 0; e < V; ++e) out[e] += r[e];
      }
      store_chan(y + t * D + d0, out);
#pragma unroll
      for (int w = 0; w < W - 1; ++w)
#pragma unroll
        for (int e = 0; e < V; ++e) win[w][e] = win[w + 1][e];
    }
  }
}

// final_state[n,d,w] = x[T_n - W + w] (falls back to the initial state / zero for T_n < W)
template <typename T>
__global__ void conv1d_final_state_kernel(const T* __restrict__ x, const T* __restrict__ init,
                                          const int64_t* __restrict__ cu, T* __restrict__ fs, int T_len, int N, int D,
                                          int W) {
  const int64_t idx = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (idx >= (int64_t)N * D) return;
  const int n = (int)(idx / D), d = (int)(idx % D);
  const int64_t bos = cu ? cu[n] : (int64_t)n * T_len;
  const int len = cu ? (int)(cu[n + 1] - bos) : T_len;
  for (int w = 0; w < W; ++w) {
    const int src = len - W + w;
    T val = Elem<T>::from_f(0.f);
    if (src >= 0) val = x[(bos + src) * D + d];
    else if (init != nullptr) val = init[((int64_t)n * D + d) * W + (src + W)];
    fs[((int64_t)n * D + d) * W + w] = val;
  }
}

// Backward.  With p the pre-activation and dyp = dy * act'(p):
//   dx[s]   = sum_u dyp[s+u] * weight[W-1-u]   (s+u inside the sequence of s)  (+ dht at the last W tokens)
//   dw[w]   = sum_t dyp[t] * xpad[t-(W-1)+w],   db = sum_t dyp[t]
// Each thread writes its tile's partial dw/db to part[tile][W+1][D]; conv1d_reduce_kernel sums them.
template <typename T, int W>
__global__ __launch_bounds__(kConvThreads) void conv1d_bwd_kernel(
    const T* __restrict__ x, const T* __restrict__ dy, const T* __restrict__ weight, const T* __restrict__ bias,
    const T* __restrict__ init, const T* __restrict__ dht, const int64_t* __restrict__ cu, T* __restrict__ dx,
    float* __restrict__ part, int64_t total, int T_len, int N, int D, int tile, int silu) {
  constexpr int V = Elem<T>::kVec;
  // one linear grid, channel blocks fastest: the number of token tiles is not bounded by the y dimension's 65535
  const int nbd = (D / V + kConvThreads - 1) / kConvThreads, bx = blockIdx.x % nbd;
  const int64_t by = blockIdx.x / nbd;
  const int d0 = (bx * kConvThreads + threadIdx.x) * V;
  if (d0 >= D) return;
  const int64_t t0 = by * tile;
  const int64_t t1 = t0 + tile < total ? t0 + tile : total;
  const int64_t tend = t1 + (W - 1) < total ? t1 + (W - 1) : total;  // halo: dyp of later tokens feeds dx
  float wgt[W][V], bs[V], win[W][V], dyw[W][V], dwa[W][V], dba[V];
#pragma unroll
  for (int w = 0; w < W; ++w) {
    load_chan(wgt[w], weight + (int64_t)w * D + d0);
#pragma unroll
    for (int e = 0; e < V; ++e) { dwa[w][e] = 0.f; dyw[w][e] = 0.f; }
  }
#pragma unroll
  for (int e = 0; e < V; ++e) { bs[e] = 0.f; dba[e] = 0.f; }
  if (bias != nullptr) load_chan(bs, bias + d0);
  SeqCursor cur, lag;   // cur follows t (leading), lag follows s = t-(W-1) (the dx being emitted)
  cur.init(cu, N, T_len, t0);
  lag.init(cu, N, T_len, t0);
#pragma unroll
  for (int w = 0; w < W - 1; ++w) load_hist(win[w], x, init, t0 - (W - 1) + w, cur, D, W, d0);
  // t runs W-1 steps past the last dyp so that the final dx of the tile are flushed.  W tokens per trip: the windows
  // win (x[t-(W-1)+j]) and dyw (dyp[s+u], s = t-(W-1)) are rings whose logical index j sits in slot (uu + j) % W at
  // the uu-th token of a trip, so sliding a window moves no register.
  // The rows of a trip are requested one trip ahead (two register sets, the loop runs two trips per turn), the same
  // loads on every path: rows past the end repeat the last one and are never used.
  auto request = [&](Vec16<T> (&xr)[W], Vec16<T> (&gr)[W], int64_t tb) {
#pragma unroll
    for (int u = 0; u < W; ++u) {
      const int64_t row = tb + u < total ? tb + u : total - 1;
      xr[u] = ld16(x + row * D + d0);
      gr[u] = ld16(dy + row * D + d0);
    }
  };
  auto trip = [&](int64_t tb, const Vec16<T> (&xr)[W], const Vec16<T> (&gr)[W]) {
#pragma unroll
    for (int uu = 0; uu < W; ++uu) {
      const int64_t t = tb + uu;
      if (t >= t1 + (W - 1)) return;
      constexpr int kNewest = W - 1;
      float* newest_x = win[(uu + kNewest) % W];
      float* newest_g = dyw[(uu + kNewest) % W];
      if (t < tend) {
        if (cur.advance_to(t)) {
#pragma unroll
          for (int w = 0; w < W - 1; ++w) load_hist(win[(uu + w) % W], x, init, t - (W - 1) + w, cur, D, W, d0);
        }
        unpack_chan(newest_x, xr[uu]);
        float g[V];
        unpack_chan(g, gr[uu]);
#pragma unroll
        for (int e = 0; e < V; ++e) {
          if (silu) {
            float p = bs[e];
#pragma unroll
            for (int w = 0; w < W; ++w) p += win[(uu + w) % W][e] * wgt[w][e];
            const float sg = sigmoidf_(p);
            g[e] *= sg * (1.f + p * (1.f - sg));
          }
          newest_g[e] = g[e];
        }
        if (t < t1) {
#pragma unroll
          for (int e = 0; e < V; ++e) {
            dba[e] += g[e];
#pragma unroll
            for (int w = 0; w < W; ++w) dwa[w][e] += g[e] * win[(uu + w) % W][e];
          }
        }
      } else {
#pragma unroll
        for (int e = 0; e < V; ++e) newest_g[e] = 0.f;
      }
      const int64_t s_ = t - (W - 1);
      if (s_ >= t0 && s_ < t1) {
        lag.advance_to(s_);
        float out[V];
#pragma unroll
        for (int e = 0; e < V; ++e) out[e] = 0.f;
#pragma unroll
        for (int u = 0; u < W; ++u) {
          if (s_ + u < lag.eos) {
#pragma unroll
            for (int e = 0; e < V; ++e) out[e] += dyw[(uu + u) % W][e] * wgt[W - 1 - u][e];
          }
        }
        if (dht != nullptr) {
          const int64_t wq = s_ - (lag.eos - W);   // final_state[n,d,wq] = x[s]
          if (wq >= 0) {
#pragma unroll
            for (int e = 0; e < V; ++e) out[e] += Elem<T>::to_f(dht[((int64_t)lag.n * D + d0 + e) * W + wq]);
          }
        }
        store_chan(dx + s_ * D + d0, out);
      }
    }
  };
  Vec16<T> xa[W], ga[W], xb[W], gb[W];
  request(xa, ga, t0);
  for (int64_t tb = t0; tb < t1 + (W - 1); tb += 2 * W) {
    request(xb, gb, tb + W);
    trip(tb, xa, ga);
    if (tb + W >= t1 + (W - 1)) break;
    request(xa, ga, tb + 2 * W);
    trip(tb + W, xb, gb);
  }
  float* pp = part + by * (W + 1) * D;
#pragma unroll
  for (int w = 0; w < W; ++w)
#pragma unroll
    for (int e = 0; e < V; ++e) pp[(int64_t)w * D + d0 + e] = dwa[w][e];
#pragma unroll
  for (int e = 0; e < V; ++e) pp[(int64_t)W * D + d0 + e] = dba[e];
}

__global__ void conv1d_reduce_kernel(const float* __restrict__ part, float* __restrict__ dw, float* __restrict__ db,
                                     int ntiles, int W, int D) {
  const int64_t idx = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (idx >= (int64_t)(W + 1) * D) return;
  float s = 0.f;
  for (int i = 0; i < ntiles; ++i) s += part[(int64_t)i * (W + 1) * D + idx];
  if (idx < (int64_t)W * D) dw[idx] = s;
  else if (db != nullptr) db[idx - (int64_t)W * D] = s;
}

// dh0[n,d,j] = sum_{i<=j-1, i<len} dyp[bos+i] * weight[j-1-i]  (j>=1)   (+ dht[n,d,j-len] when len < W)
template <typename T>
__global__ void conv1d_dh0_kernel(const T* __restrict__ x, const T* __restrict__ dy, const T* __restrict__ weight,
                                  const T* __restrict__ bias, const T* __restrict__ init, const T* __restrict__ dht,
                                  const int64_t* __restrict__ cu, T* __restrict__ dh0, int T_len, int N, int D, int W,
                                  int silu) {
  const int64_t idx = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (idx >= (int64_t)N * D) return;
  const int n = (int)(idx / D), d = (int)(idx % D);
  const int64_t bos = cu ? cu[n] : (int64_t)n * T_len;
  const int len = cu ? (int)(cu[n + 1] - bos) : T_len;
  float acc[8];
  for (int j = 0; j < W; ++j) acc[j] = 0.f;
  for (int i = 0; i < W - 1 && i < len; ++i) {
    float g = Elem<T>::to_f(dy[(bos + i) * D + d]);
    if (silu) {
      float p = bias ? Elem<T>::to_f(bias[d]) : 0.f;
      for (int w = 0; w < W; ++w) {
        const int tau = i - (W - 1) + w;
        float xv = 0.f;
        if (tau >= 0) xv = Elem<T>::to_f(x[(bos + tau) * D + d]);
        else if (init != nullptr && W + tau >= 1) xv = Elem<T>::to_f(init[((int64_t)n * D + d) * W + W + tau]);
        p += xv * Elem<T>::to_f(weight[(int64_t)w * D + d]);
      }
      const float sg = sigmoidf_(p);
      g *= sg * (1.f + p * (1.f - sg));
    }
    for (int j = i + 1; j < W; ++j) acc[j] += g * Elem<T>::to_f(weight[(int64_t)(j - 1 - i) * D + d]);
  }
  if (dht != nullptr)
    for (int w = 0; len + w < W; ++w) acc[len + w] += Elem<T>::to_f(dht[((int64_t)n * D + d) * W + w]);
  for (int j = 0; j < W; ++j) dh0[((int64_t)n * D + d) * W + j] = Elem<T>::from_f(acc[j]);
}

// Decode update: hidden[B,T,D], conv_state[B,D,S] rolled in place, weight[D,W].
template <typename T>
__global__ void conv1d_update_kernel(const T* __restrict__ hidden, T* __restrict__ state, const T* __restrict__ weight,
                                     const T* __restrict__ bias, T* __restrict__ out, int B, int T_len, int D, int W,
                                     int S, int silu) {
  const int64_t idx = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (idx >= (int64_t)B * D) return;
  const int b = (int)(idx / D), d = (int)(idx % D);
  float st[17], wg[8];   // st[0..S-1] = state, st[S] = the incoming token; needs S >= W-1
  for (int j = 0; j < S; ++j) st[j] = Elem<T>::to_f(state[((int64_t)b * D + d) * S + j]);
  for (int w = 0; w < W; ++w) wg[w] = Elem<T>::to_f(weight[(int64_t)d * W + w]);
  const float bs = bias ? Elem<T>::to_f(bias[d]) : 0.f;
  for (int t = 0; t < T_len; ++t) {
    st[S] = Elem<T>::to_f(hidden[((int64_t)b * T_len + t) * D + d]);
    float a = bs;
    for (int w = 0; w < W; ++w) a += st[S + 1 - W + w] * wg[w];
    out[((int64_t)b * T_len + t) * D + d] = Elem<T>::from_f(silu ? a * sigmoidf_(a) : a);
    for (int j = 0; j < S; ++j) st[j] = st[j + 1];   // roll: the state always ends with the newest input
  }
  for (int j = 0; j < S; ++j) state[((int64_t)b * D + d) * S + j] = Elem<T>::from_f(st[j]);
}

// The same for the usual state length S == W with a row of W elements 8 or 16 bytes long: the state row and the
// weight row of a channel are one vector load each, the window lives in registers with constant indices.
template <typename T, int W>
__global__ __launch_bounds__(256) void conv1d_update_rows_kernel(const T* __restrict__ hidden, T* __restrict__ state,
                                                                 const T* __restrict__ weight, const T* __restrict__ bias,
                                                                 T* __restrict__ out, int B, int T_len, int D, int silu) {
  constexpr int kBytes = W * (int)sizeof(T);
  static_assert(kBytes == 8 || kBytes == 16, "a row is one 8- or 16-byte vector");
  typedef uint32_t RowVec __attribute__((ext_vector_type(kBytes / 4)));
  union Row { RowVec v; T e[W]; };
  const int64_t idx = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (idx >= (int64_t)B * D) return;
  const int b = (int)(idx / D), d = (int)(idx % D);
  Row r, wr;
  r.v = *reinterpret_cast<const RowVec*>(state + idx * W);
  wr.v = *reinterpret_cast<const RowVec*>(weight + (int64_t)d * W);
  float st[W + 1], wg[W];
#pragma unroll
  for (int j = 0; j < W; ++j) { st[j] = Elem<T>::to_f(r.e[j]); wg[j] = Elem<T>::to_f(wr.e[j]); }
  const float bs = bias ? Elem<T>::to_f(bias[d]) : 0.f;
  for (int t = 0; t < T_len; ++t) {
    st[W] = Elem<T>::to_f(hidden[((int64_t)b * T_len + t) * D + d]);
    float a = bs;
#pragma unroll
    for (int w = 0; w < W; ++w) a += st[1 + w] * wg[w];
    out[((int64_t)b * T_len + t) * D + d] = Elem<T>::from_f(silu ? a * sigmoidf_(a) : a);
#pragma unroll
    for (int j = 0; j < W; ++j) st[j] = st[j + 1];
  }
#pragma unroll
  for (int j = 0; j < W; ++j) r.e[j] = Elem<T>::from_f(st[j]);
  *reinterpret_cast<RowVec*>(state + idx * W) = r.v;
}

template <typename T> struct ConvLaunch {
  static int fwd(const void* x, const void* weight, const void* bias, const void* residual, const void* init,
                 const int64_t* cu, void* y, void* fs, int B, int T_len, int N, int D, int W, int silu,
                 hipStream_t st) {
    constexpr int V = Elem<T>::kVec;
    const int64_t total = (int64_t)B * T_len;
    const int tile = 64;
    const int64_t nblocks = (int64_t)((D / V + kConvThreads - 1) / kConvThreads) * ((total + tile - 1) / tile);
    if (nblocks > 0x7fffffffLL) return -3;
    dim3 grid((unsigned)nblocks);
    if (total > 0) {
      switch (W) {
#define GDN_CASE(W_)                                                                                              \
  case W_:                                                                                                        \
    GDN_LAUNCH(kKernConvFwd, st, (conv1d_fwd_kernel<T, W_>), grid, dim3(kConvThreads), 0, st, (const T*)x,   \
                       (const T*)weight, (const T*)bias, (const T*)residual, (const T*)init, cu, (T*)y, total,    \
                       T_len, N, D, tile, silu);                                                                  \
    break;
        GDN_CASE(1) GDN_CASE(2) GDN_CASE(3) GDN_CASE(4) GDN_CASE(5) GDN_CASE(6) GDN_CASE(7) GDN_CASE(8)
#undef GDN_CASE
        default: return -3;
      }
    }
    if (fs != nullptr) {
      const int64_t n = (int64_t)N * D;
      GDN_LAUNCH(kKernConvState, st, (conv1d_final_state_kernel<T>), dim3((unsigned)((n + 255) / 256)), dim3(256),
                         0, st, (const T*)x, (const T*)init, cu, (T*)fs, T_len, N, D, W);
    }
    return (int)hipGetLastError();
  }
  static int bwd(const void* x, const void* dy, const void* weight, const void* bias, const void* init,
                 const void* dht, const int64_t* cu, void* dx, float* dw, float* db, void* dh0, float* workspace,
                 int B, int T_len, int N, int D, int W, int silu, hipStream_t st) {
    constexpr int V = Elem<T>::kVec;
    const int64_t total = (int64_t)B * T_len;
    const int tile = 256;
    const int ntiles = (int)((total + tile - 1) / tile);
    const int64_t nblocks = (int64_t)((D / V + kConvThreads - 1) / kConvThreads) * ntiles;
    if (nblocks > 0x7fffffffLL) return -3;
    dim3 grid((unsigned)nblocks);
    if (total > 0) {
      switch (W) {
#define GDN_CASE(W_)                                                                                              \
  case W_:                                                                                                        \
    GDN_LAUNCH(kKernConvBwd, st, (conv1d_bwd_kernel<T, W_>), grid, dim3(kConvThreads), 0, st, (const T*)x,   \
                       (const T*)dy, (const T*)weight, (const T*)bias, (const T*)init, (const T*)dht, cu, (T*)dx, \
                       workspace, total, T_len, N, D, tile, silu);                                                \
    break;
        GDN_CASE(1) GDN_CASE(2) GDN_CASE(3) GDN_CASE(4) GDN_CASE(5) GDN_CASE(6) GDN_CASE(7) GDN_CASE(8)
#undef GDN_CASE
        default: return -3;
      }
    }
    const int64_t nred = (int64_t)(W + 1) * D;
    GDN_LAUNCH(kKernConvReduce, st, conv1d_reduce_kernel, dim3((unsigned)((nred + 255) / 256)), dim3(256), 0, st, workspace, dw, db,
                       ntiles, W, D);
    if (dh0 != nullptr) {
      const int64_t n = (int64_t)N * D;
      GDN_LAUNCH(kKernConvDh0, st, (conv1d_dh0_kernel<T>), dim3((unsigned)((n + 255) / 256)), dim3(256), 0, st,
                         (const T*)x, (const T*)dy, (const T*)weight, (const T*)bias, (const T*)init, (const T*)dht,
                         cu, (T*)dh0, T_len, N, D, W, silu);
    }
    return (int)hipGetLastError();
  }
  static int update(const void* hidden, void* state, const void* weight, const void* bias, void* out, int B,
                    int T_len, int D, int W, int S, int silu, hipStream_t st) {
    const int64_t n = (int64_t)B * D;
    const dim3 grid((unsigned)((n + 255) / 256));
    const bool aligned = (((uintptr_t)state | (uintptr_t)weight) & 15) == 0;
    if (S == W && aligned && W * (int)sizeof(T) == 8) {
      GDN_LAUNCH(kKernConvUpdate, st, (conv1d_update_rows_kernel<T, 8 / (int)sizeof(T)>), grid, dim3(256), 0, st,
                 (const T*)hidden, (T*)state, (const T*)weight, (const T*)bias, (T*)out, B, T_len, D, silu);
    } else if (S == W && aligned && W * (int)sizeof(T) == 16) {
      GDN_LAUNCH(kKernConvUpdate, st, (conv1d_update_rows_kernel<T, 16 / (int)sizeof(T)>), grid, dim3(256), 0, st,
                 (const T*)hidden, (T*)state, (const T*)weight, (const T*)bias, (T*)out, B, T_len, D, silu);
    } else {
      GDN_LAUNCH(kKernConvUpdate, st, (conv1d_update_kernel<T>), grid, dim3(256), 0, st, (const T*)hidden, (T*)state,
                 (const T*)weight, (const T*)bias, (T*)out, B, T_len, D, W, S, silu);
    }
    return (int)hipGetLastError();
  }
};

static int conv_check(int B, int T_len, int N, int D, int W, int dtype) {
  if (B <= 0 || T_len < 0 || N <= 0 || D <= 0) return -2;
  if (W < 1 || W > 8) return -3;
  const int V = dtype == 0 ? 4 : 8;
  if (D % V != 0) return -3;
  if (dtype < 0 || dtype > 2) return -4;
  return 0;
}

}  // namespace gdn

extern "C" int64_t gdn_conv1d_bwd_workspace_bytes(int B, int T, int D, int W) {
  const int64_t total = (int64_t)B * T;
  const int64_t ntiles = (total + 255) / 256;
  return (ntiles > 0 ? ntiles : 1) * (int64_t)(W + 1) * D * (int64_t)sizeof(float);
}

extern "C" int gdn_conv1d_fwd(const void* x, const void* weight, const void* bias, const void* residual,
                              const void* initial_state, const int64_t* cu_seqlens, void* y, void* final_state, int B,
                              int T, int N, int D, int W, int activation, int dtype, void* stream) {
  if (!x || !weight || !y) return -1;
  if (int e = gdn::conv_check(B, T, N, D, W, dtype)) return e;
  if (cu_seqlens != nullptr && B != 1) return -2;
  hipStream_t s = (hipStream_t)stream;
  if (dtype == 0) return gdn::ConvLaunch<float>::fwd(x, weight, bias, residual, initial_state, cu_seqlens, y, final_state, B, T, N, D, W, activation, s);
  if (dtype == 1) return gdn::ConvLaunch<gdn::bf16_t>::fwd(x, weight, bias, residual, initial_state, cu_seqlens, y, final_state, B, T, N, D, W, activation, s);
  return gdn::ConvLaunch<gdn::f16_t>::fwd(x, weight, bias, residual, initial_state, cu_seqlens, y, final_state, B, T, N, D, W, activation, s);
}

extern "C" int gdn_conv1d_bwd(const void* x, const void* dy, const void* weight, const void* bias,
                              const void* initial_state, const void* d_final_state, const int64_t* cu_seqlens,
                              void* dx, float* dw, float* db, void* d_initial_state, void* workspace,
                              int64_t workspace_bytes, int B, int T, int N, int D, int W, int activation, int dtype,
                              void* stream) {
  if (!x || !dy || !weight || !dx || !dw || !workspace) return -1;
  if (int e = gdn::conv_check(B, T, N, D, W, dtype)) return e;
  if (cu_seqlens != nullptr && B != 1) return -2;
  if (workspace_bytes < gdn_conv1d_bwd_workspace_bytes(B, T, D, W)) return -5;
  hipStream_t s = (hipStream_t)stream;
  float* ws = (float*)workspace;
  if (dtype == 0) return gdn::ConvLaunch<float>::bwd(x, dy, weight, bias, initial_state, d_final_state, cu_seqlens, dx, dw, db, d_initial_state, ws, B, T, N, D, W, activation, s);
  if (dtype == 1) return gdn::ConvLaunch<gdn::bf16_t>::bwd(x, dy, weight, bias, initial_state, d_final_state, cu_seqlens, dx, dw, db, d_initial_state, ws, B, T, N, D, W, activation, s);
  return gdn::ConvLaunch<gdn::f16_t>::bwd(x, dy, weight, bias, initial_state, d_final_state, cu_seqlens, dx, dw, db, d_initial_state, ws, B, T, N, D, W, activation, s);
}

extern "C" int gdn_conv1d_update(const void* hidden, void* conv_state, const void* weight, const void* bias, void* out,
                                 int B, int T, int D, int W, int state_len, int activation, int dtype, void* stream) {
  if (!hidden || !conv_state || !weight || !out) return -1;
  if (B <= 0 || T < 0 || D <= 0) return -2;
  if (W < 1 || W > 8 || state_len < 1 || state_len > 16 || state_len < W - 1) return -3;
  if (dtype < 0 || dtype > 2) return -4;
  hipStream_t s = (hipStream_t)stream;
  if (dtype == 0) return gdn::ConvLaunch<float>::update(hidden, conv_state, weight, bias, out, B, T, D, W, state_len, activation, s);
  if (dtype == 1) return gdn::ConvLaunch<gdn::bf16_t>::update(hidden, conv_state, weight, bias, out, B, T, D, W, state_len, activation, s);
  return gdn::ConvLaunch<gdn::f16_t>::update(hidden, conv_state, weight, bias, out, B, T, D, W, state_len, activation, s);
}
