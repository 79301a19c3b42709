// Chunked gated delta rule, forward pass (chunk = 64 tokens).  Per sequence and value head, with
// G the chunk-local cumulative log decay and Gam_ij = e^{G_i - G_j}:
//     L  = strict_tril(beta_i (k_i.k_j) Gam_ij)          Tm = (I + L)^-1
//     W  = Tm (beta e^G . K)      U = Tm (beta . V)
//     V' = U - W S                O = scale [ (e^G . Q) S + tril(Q K^T . Gam) V' ]
//     S <- e^{G_last} S + (e^{G_last - G} . K)^T V'
// Math: mindspeed_mm/fsdp/models/qwen3_5/modeling_qwen3_5.py:398-475; stage split as in
// mindspeed_mm/fsdp/ops/gdn/chunk_gated_delta_rule.py:30-85 (cumsum, KK^T, tril solve, W/U, state
// recurrence, output), fused here into three launches:
//     chunk_prep_kernel      per (chunk, head):        G, Tm, W, U           -- MFMA + fp32 block solve
//     chunk_state_kernel     per (sequence, head, V-slab), sequential in chunks: V', S per chunk
//     chunk_out_kernel       per (chunk, head, V-slab): O
// A ragged last chunk is zero padded in LDS (k = v = beta = g = 0 is exact for this recurrence).
#include "gdn_chunk.h"
#include "gdn_common.h"
#include "gdn_profile.h"

namespace gdn {

constexpr int kLF = 68;  // leading dimension of the fp32 64x64 solve buffers

// 16x16x4 fp32 matrix-core step used by the triangular solve: lane l feeds A[l%16][l/16], B[l/16][l%16]
// and owns C[4*(l/16)+r][l%16], r = 0..3.
__device__ __forceinline__ f32x4 mfma16_f32(f32x4 acc, float a, float b) {
  return __builtin_amdgcn_mfma_f32_16x16x4f32(a, b, acc, 0, 0, 0);
}

// ---------------------------------------------------------------------------------------------
// packed-sequence chunk table: chunk_offsets[n] = sum_{m<n} ceil(len_m / 64)
// ---------------------------------------------------------------------------------------------
__global__ void chunk_table_kernel(const int64_t* __restrict__ cu, int* __restrict__ chunk_offsets, int N) {
  __shared__ int part[kThreads];
  const int tid = threadIdx.x;
  const int per = (N + kThreads - 1) / kThreads;
  const int lo = imin(tid * per, N), hi = imin(lo + per, N);
  int s = 0;
  for (int n = lo; n < hi; ++n) s += (int)((cu[n + 1] - cu[n] + kChunk - 1) / kChunk);
  part[tid] = s;
  __syncthreads();
  if (tid == 0) {
    int run = 0;
    for (int i = 0; i < kThreads; ++i) { const int t = part[i]; part[i] = run; run += t; }
    chunk_offsets[N] = run;
  }
  __syncthreads();
  int run = part[tid];
  for (int n = lo; n < hi; ++n) {
    chunk_offsets[n] = run;
    run += (int)((cu[n + 1] - cu[n] + kChunk - 1) / kChunk);
  }
}

// ---------------------------------------------------------------------------------------------
// y = x * rsqrt(sum(x^2) + 1e-6) over the last axis (modeling_qwen3_5.py:392-395); rows of DK elements
// ---------------------------------------------------------------------------------------------
template <typename T, int DK>
__global__ void l2norm_fwd_kernel(const T* __restrict__ x0, const T* __restrict__ x1, T* __restrict__ y0,
                                  T* __restrict__ y1, int64_t rows) {
  constexpr int V = Elem<T>::kVec, LPR = DK / V;  // lanes per row (a power of two <= 32)
  const T* x = blockIdx.y == 0 ? x0 : x1;
  T* y = blockIdx.y == 0 ? y0 : y1;
  const int64_t row = (int64_t)blockIdx.x * (kThreads / LPR) + threadIdx.x / LPR;
  const int c = threadIdx.x % LPR;
  const bool ok = row < rows;
  Vec16<T> v = ok ? ld16(x + row * DK + c * V) : zero16<T>();
  float ss = 0.f;
#pragma unroll
  for (int e = 0; e < V; ++e) { const float f = v.get(e); ss += f * f; }
#pragma unroll
  for (int m = 1; m < LPR; m <<= 1) ss += __shfl_xor(ss, m);
  const float r = rsqrtf(ss + 1e-6f);
#pragma unroll
  for (int e = 0; e < V; ++e) v.set(e, v.get(e) * r);
  if (ok) st16(y + row * DK + c * V, v);
}

// ---------------------------------------------------------------------------------------------
// chunk_prep_kernel
// ---------------------------------------------------------------------------------------------
template <typename T, int DK, int BV> struct PrepSmem {
  static constexpr int LDK = lds_ld<T>(DK), LDV = lds_ld<T>(BV), L64 = lds_ld<T>(64);
  static constexpr int kv_elems = 64 * (LDK > LDV ? LDK : LDV);
  static constexpr int off_ks = 0;  // K tile, later the (beta V) tile
  static constexpr int off_kb = off_ks + kv_elems * (int)sizeof(T);
  static constexpr int off_as = off_kb + 64 * LDK * (int)sizeof(T);
  static constexpr int off_ti = off_as + 64 * kLF * 4;
  static constexpr int off_tms = off_ti + 64 * kLF * 4;
  static constexpr int off_misc = off_tms + 64 * L64 * (int)sizeof(T);
  static constexpr int bytes = off_misc + 3 * 64 * 4;
};

template <typename T, int DK, int BV>
__global__ __launch_bounds__(kThreads) void chunk_prep_kernel(
    const T* __restrict__ k, const T* __restrict__ v, const float* __restrict__ g, const float* __restrict__ beta,
    const int64_t* __restrict__ cu, const int* __restrict__ chunk_offsets, float* __restrict__ G_out,
    T* __restrict__ Ai_out, T* __restrict__ W_out, T* __restrict__ U_out, int T_len, int N, int Hqk, int Hv, int V) {
  using SM = PrepSmem<T, DK, BV>;
  constexpr int LDK = SM::LDK, LDV = SM::LDV, L64 = SM::L64, VEC = Elem<T>::kVec;
  T* Ks = reinterpret_cast<T*>(gdn_smem + SM::off_ks);
  T* Vb = Ks;
  T* Kb = reinterpret_cast<T*>(gdn_smem + SM::off_kb);
  float* As = reinterpret_cast<float*>(gdn_smem + SM::off_as);
  float* Ti = reinterpret_cast<float*>(gdn_smem + SM::off_ti);
  T* Tms = reinterpret_cast<T*>(gdn_smem + SM::off_tms);
  float* Gs = reinterpret_cast<float*>(gdn_smem + SM::off_misc);
  float* bs = Gs + 64;
  float* egs = bs + 64;

  const SeqInfo s = locate_chunk(blockIdx.x, cu, chunk_offsets, N, T_len);
  if (s.nvalid <= 0) return;
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int h = blockIdx.y, hq = h / (Hv / Hqk), nvalid = s.nvalid;
  const int64_t tok0 = s.bos + (int64_t)s.chunk * kChunk;

  // ---- phase 0: cumulative decay (one lane per token), beta ----
  if (wave == 0) {
    float x = lane < nvalid ? g[(tok0 + lane) * Hv + h] : 0.f;
#pragma unroll
    for (int d = 1; d < 64; d <<= 1) {
      const float t = __shfl_up(x, d);
      if (lane >= d) x += t;
    }
    const float b = lane < nvalid ? beta[(tok0 + lane) * Hv + h] : 0.f;
    Gs[lane] = x;
    bs[lane] = b;
    egs[lane] = b * __expf(x);
    if (lane < nvalid) G_out[(tok0 + lane) * Hv + h] = x;
  }
  for (int i = tid; i < 64 * kLF; i += kThreads) Ti[i] = 0.f;
  __syncthreads();

  // ---- phase 1: K tile, plain and scaled by beta e^G ----
  {
    constexpr int CPR = DK / VEC;
    const T* kg = k + (tok0 * Hqk + hq) * DK;
    for (int c = tid; c < 64 * CPR; c += kThreads) {
      const int row = c / CPR, cc = c % CPR;
      Vec16<T> x = zero16<T>(), xs = zero16<T>();
      if (row < nvalid) {
        x = ld16(kg + (int64_t)row * Hqk * DK + cc * VEC);
        const float sc = egs[row];
#pragma unroll
        for (int e = 0; e < VEC; ++e) xs.set(e, x.get(e) * sc);
      }
      st16(Ks + row * LDK + cc * VEC, x);
      st16(Kb + row * LDK + cc * VEC, xs);
    }
  }
  __syncthreads();

  // ---- phase 2: A = strict_tril(beta_i k_i.k_j e^{G_i-G_j}), one 32x32 tile per wave ----
  {
    const int ti = wave >> 1, tj = wave & 1;
    f32x16 acc = acc_zero();
    if (tj <= ti) mma32<T, DK, true, true>(acc, Ks + 32 * ti * LDK, LDK, Ks + 32 * tj * LDK, LDK);
    const int j = 32 * tj + acc_col();
#pragma unroll
    for (int r = 0; r < 16; ++r) {
      const int i = 32 * ti + acc_row(r);
      As[i * kLF + j] = i > j ? bs[i] * acc[r] * __expf(Gs[i] - Gs[j]) : 0.f;
    }
  }
  __syncthreads();

  // (beta V) tile of the first V block goes into the dead K tile while the solve runs
  const T* vg = v + (tok0 * Hv + h) * V;
  load_tile_scaled<T, BV>(Vb, LDV, vg, (int64_t)Hv * V, nvalid, bs, tid);

  // ---- phase 3a: invert the four 16x16 diagonal blocks by forward substitution (fp32) ----
  if (lane < 16) {
    const int o = 16 * wave, j = lane;
    float tcol[16];
#pragma unroll
    for (int i = 0; i < 16; ++i) {
      float x = (i == j) ? 1.f : 0.f;
#pragma unroll
      for (int m = 0; m < i; ++m) x -= As[(o + i) * kLF + o + m] * tcol[m];
      tcol[i] = x;
    }
#pragma unroll
    for (int i = 0; i < 16; ++i) Ti[(o + i) * kLF + o + j] = tcol[i];
  }
  __syncthreads();

  // ---- phase 3b: 16 -> 32 merges  X = -T22 (A21 T11); the zero upper triangle of As is scratch ----
  {
    const int p = wave & 1;           // waves 0,1 compute; 2,3 repeat the same values (benign)
    const int C0 = 32 * p, R0 = C0 + 16;
    const int li = lane & 15, lk = lane >> 4;
    f32x4 y = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int kk = 0; kk < 4; ++kk)
      y = mfma16_f32(y, As[(R0 + li) * kLF + C0 + 4 * kk + lk], Ti[(C0 + 4 * kk + lk) * kLF + C0 + li]);
    __syncthreads();  // every wave has read its A21 before the scratch next to it is written
    if (wave < 2) {
#pragma unroll
      for (int r = 0; r < 4; ++r) As[(C0 + 4 * lk + r) * kLF + R0 + li] = y[r];
    }
    __syncthreads();
    f32x4 x = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int kk = 0; kk < 4; ++kk)
      x = mfma16_f32(x, Ti[(R0 + li) * kLF + R0 + 4 * kk + lk], As[(C0 + 4 * kk + lk) * kLF + R0 + li]);
    if (wave < 2) {
#pragma unroll
      for (int r = 0; r < 4; ++r) Ti[(R0 + 4 * lk + r) * kLF + C0 + li] = -x[r];
    }
  }
  __syncthreads();

  // ---- phase 3c: 32 -> 64 merge, one 16x16 tile of the 32x32 block per wave ----
  {
    const int ta = wave >> 1, tb = wave & 1;
    const int li = lane & 15, lk = lane >> 4;
    f32x4 y = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int kk = 0; kk < 8; ++kk)
      y = mfma16_f32(y, As[(32 + 16 * ta + li) * kLF + 4 * kk + lk], Ti[(4 * kk + lk) * kLF + 16 * tb + li]);
    // scratch: upper-right 32x32 quadrant of As (never read as part of A)
#pragma unroll
    for (int r = 0; r < 4; ++r) As[(16 * ta + 4 * lk + r) * kLF + 32 + 16 * tb + li] = y[r];
    __syncthreads();
    f32x4 x = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int kk = 0; kk < 8; ++kk)
      x = mfma16_f32(x, Ti[(32 + 16 * ta + li) * kLF + 32 + 4 * kk + lk], As[(4 * kk + lk) * kLF + 32 + 16 * tb + li]);
#pragma unroll
    for (int r = 0; r < 4; ++r) Ti[(32 + 16 * ta + 4 * lk + r) * kLF + 16 * tb + li] = -x[r];
  }
  __syncthreads();

  // ---- phase 4: Tm in operand precision, kept for the backward pass ----
  {
    constexpr int CPR = 64 / VEC;
    T* ag = Ai_out + (tok0 * Hv + h) * 64;
    for (int c = tid; c < 64 * CPR; c += kThreads) {
      const int row = c / CPR, cc = c % CPR;
      Vec16<T> x = zero16<T>();
#pragma unroll
      for (int e = 0; e < VEC; ++e) x.set(e, Ti[row * kLF + cc * VEC + e]);
      st16(Tms + row * L64 + cc * VEC, x);
      if (row < nvalid) st16(ag + (int64_t)row * Hv * 64 + cc * VEC, x);
    }
  }
  __syncthreads();

  // ---- phase 5: W = Tm (beta e^G K) ----
  {
    T* wg = W_out + (tok0 * Hv + h) * DK;
    for (int tt = wave; tt < 2 * (DK / 32); tt += 4) {
      const int ri = tt & 1, cj = tt >> 1;
      f32x16 acc = acc_zero();
      mma32<T, 64, true, false>(acc, Tms + 32 * ri * L64, L64, Kb + 32 * cj, LDK);
      acc_to_global(acc, wg, (int64_t)Hv * DK, 32 * ri, 32 * cj, nvalid);
    }
  }
  // ---- phase 6: U = Tm (beta V), V block by V block ----
  for (int vb = 0; vb < V / BV; ++vb) {
    if (vb > 0) {
      __syncthreads();
      load_tile_scaled<T, BV>(Vb, LDV, vg + vb * BV, (int64_t)Hv * V, nvalid, bs, tid);
      __syncthreads();
    }
    T* ug = U_out + (tok0 * Hv + h) * V + vb * BV;
    for (int tt = wave; tt < 2 * (BV / 32); tt += 4) {
      const int ri = tt & 1, cj = tt >> 1;
      f32x16 acc = acc_zero();
      mma32<T, 64, true, false>(acc, Tms + 32 * ri * L64, L64, Vb + 32 * cj, LDV);
      acc_to_global(acc, ug, (int64_t)Hv * V, 32 * ri, 32 * cj, nvalid);
    }
  }
}

// ---------------------------------------------------------------------------------------------
// chunk_state_kernel: the inter-chunk recurrence.  The workgroup keeps the transposed state slab
// S^T[BV, DK] in fp32 accumulators for the whole sequence; a copy in operand precision is staged in
// LDS once per chunk (B operand of W S) and streamed to HBM for the output and backward kernels.
// ---------------------------------------------------------------------------------------------
template <typename T, int DK, int BV> struct StateSmem {
  static constexpr int LDK = lds_ld<T>(DK), L64 = lds_ld<T>(64);
  static constexpr int off_ws = 0;
  static constexpr int off_ks = off_ws + 64 * LDK * (int)sizeof(T);
  static constexpr int off_sb = off_ks + 64 * LDK * (int)sizeof(T);
  static constexpr int off_vpt = off_sb + BV * LDK * (int)sizeof(T);
  static constexpr int off_gs = off_vpt + BV * L64 * (int)sizeof(T);
  static constexpr int bytes = off_gs + 64 * 4;
};

template <typename T, int DK, int BV>
__global__ __launch_bounds__(kThreads) void chunk_state_kernel(
    const T* __restrict__ k, const T* __restrict__ w, T* vn, const float* __restrict__ G,
    const float* __restrict__ h0, float* __restrict__ ht, T* __restrict__ hbuf, const int64_t* __restrict__ cu,
    const int* __restrict__ chunk_offsets, int T_len, int Hqk, int Hv, int V) {
  using SM = StateSmem<T, DK, BV>;
  constexpr int LDK = SM::LDK, L64 = SM::L64;
  constexpr int MT = BV / 32, NTC = DK / 32, NS = (MT * NTC + 3) / 4;  // state tiles per wave
  T* Ws = reinterpret_cast<T*>(gdn_smem + SM::off_ws);
  T* Ks = reinterpret_cast<T*>(gdn_smem + SM::off_ks);
  T* Sb = reinterpret_cast<T*>(gdn_smem + SM::off_sb);
  T* VpT = reinterpret_cast<T*>(gdn_smem + SM::off_vpt);
  float* Gs = reinterpret_cast<float*>(gdn_smem + SM::off_gs);

  const int tid = threadIdx.x, wave = tid >> 6;
  const int n = blockIdx.x / Hv, h = blockIdx.x % Hv, hq = h / (Hv / Hqk);
  const int v0 = blockIdx.y * BV;
  const int64_t bos = cu ? cu[n] : (int64_t)n * T_len;
  const int len = cu ? (int)(cu[n + 1] - bos) : T_len;
  const int nchunks = (len + kChunk - 1) / kChunk;
  const int64_t chunk_base = cu ? chunk_offsets[n] : (int64_t)n * ((T_len + kChunk - 1) / kChunk);

  // state tile tt of this wave: rows (v) 32*mi.., cols (k) 32*ni..
  f32x16 S[NS];
#pragma unroll
  for (int i = 0; i < NS; ++i) {
    const int tt = wave + 4 * i;
    S[i] = acc_zero();
    if (tt < MT * NTC && h0 != nullptr) {
      const int mi = tt % MT, ni = tt / MT;
      const int kcol = 32 * ni + acc_col();
#pragma unroll
      for (int r = 0; r < 16; ++r)
        S[i][r] = h0[(((int64_t)n * Hv + h) * DK + kcol) * V + v0 + 32 * mi + acc_row(r)];
    }
  }

  for (int c = 0; c < nchunks; ++c) {
    const int64_t tok0 = bos + (int64_t)c * kChunk;
    const int nvalid = imin(kChunk, len - c * kChunk);
    T* hg = hbuf + (((chunk_base + c) * Hv + h) * V + v0) * DK;
    // (a) state before this chunk -> LDS (operand precision) and HBM
#pragma unroll
    for (int i = 0; i < NS; ++i) {
      const int tt = wave + 4 * i;
      if (tt < MT * NTC) {
        const int mi = tt % MT, ni = tt / MT;
        acc_to_lds(S[i], Sb, LDK, 32 * mi, 32 * ni);
        acc_to_global(S[i], hg, (int64_t)DK, 32 * mi, 32 * ni, BV);
      }
    }
    // (b) operands of this chunk
    load_tile<T, DK>(Ws, LDK, w + (tok0 * Hv + h) * DK, (int64_t)Hv * DK, nvalid, tid);
    load_tile<T, DK>(Ks, LDK, k + (tok0 * Hqk + hq) * DK, (int64_t)Hqk * DK, nvalid, tid);
    if (tid < 64) Gs[tid] = G[(tok0 + imin(tid, nvalid - 1)) * Hv + h];
    __syncthreads();
    const float glast = Gs[63];
    // (c) V' = U - W S; the copy for the state update is scaled by e^{G_last - G} and transposed
    T* vg = vn + (tok0 * Hv + h) * V + v0;
    for (int tt = wave; tt < 2 * MT; tt += 4) {
      const int ri = tt & 1, cj = tt >> 1;
      f32x16 ws = acc_zero();
      mma32<T, DK, true, true>(ws, Ws + 32 * ri * LDK, LDK, Sb + 32 * cj * LDK, LDK);
      f32x16 vp = acc_from_global(vg, (int64_t)Hv * V, 32 * ri, 32 * cj, nvalid);
#pragma unroll
      for (int r = 0; r < 16; ++r) vp[r] -= ws[r];
      acc_to_global(vp, vg, (int64_t)Hv * V, 32 * ri, 32 * cj, nvalid);
#pragma unroll
      for (int r = 0; r < 16; ++r) vp[r] *= __expf(glast - Gs[32 * ri + acc_row(r)]);
      acc_to_lds_t(vp, VpT, L64, 32 * ri, 32 * cj);
    }
    __syncthreads();
    // (d) S^T <- e^{G_last} S^T + V'^T K
    const float eg = __expf(glast);
#pragma unroll
    for (int i = 0; i < NS; ++i) {
      const int tt = wave + 4 * i;
      if (tt < MT * NTC) {
        const int mi = tt % MT, ni = tt / MT;
#pragma unroll
        for (int r = 0; r < 16; ++r) S[i][r] *= eg;
        mma32<T, 64, true, false>(S[i], VpT + 32 * mi * L64, L64, Ks + 32 * ni, LDK);
      }
    }
    __syncthreads();
  }

  if (ht != nullptr) {
#pragma unroll
    for (int i = 0; i < NS; ++i) {
      const int tt = wave + 4 * i;
      if (tt < MT * NTC) {
        const int mi = tt % MT, ni = tt / MT;
        const int kcol = 32 * ni + acc_col();
#pragma unroll
        for (int r = 0; r < 16; ++r)
          ht[(((int64_t)n * Hv + h) * DK + kcol) * V + v0 + 32 * mi + acc_row(r)] = S[i][r];
      }
    }
  }
}

// ---------------------------------------------------------------------------------------------
// chunk_out_kernel:  O = scale [ e^G . (Q S) + tril(Q K^T . Gam) V' ]
// ---------------------------------------------------------------------------------------------
template <typename T, int DK, int BV> struct OutSmem {
  static constexpr int LDK = lds_ld<T>(DK), LDV = lds_ld<T>(BV), L64 = lds_ld<T>(64);
  static constexpr int off_qs = 0;
  static constexpr int off_ks = off_qs + 64 * LDK * (int)sizeof(T);
  static constexpr int off_sb = off_ks + 64 * LDK * (int)sizeof(T);
  static constexpr int off_vp = off_sb + BV * LDK * (int)sizeof(T);
  static constexpr int off_aq = off_vp + 64 * LDV * (int)sizeof(T);
  static constexpr int off_gs = off_aq + 64 * L64 * (int)sizeof(T);
  static constexpr int bytes = off_gs + 64 * 4;
};

template <typename T, int DK, int BV>
__global__ __launch_bounds__(kThreads) void chunk_out_kernel(
    const T* __restrict__ q, const T* __restrict__ k, const T* __restrict__ vn, const T* __restrict__ hbuf,
    const float* __restrict__ G, T* __restrict__ o, const int64_t* __restrict__ cu,
    const int* __restrict__ chunk_offsets, int T_len, int N, int Hqk, int Hv, int V, float scale) {
  using SM = OutSmem<T, DK, BV>;
  constexpr int LDK = SM::LDK, LDV = SM::LDV, L64 = SM::L64, MT = BV / 32;
  T* Qs = reinterpret_cast<T*>(gdn_smem + SM::off_qs);
  T* Ks = reinterpret_cast<T*>(gdn_smem + SM::off_ks);
  T* Sb = reinterpret_cast<T*>(gdn_smem + SM::off_sb);
  T* Vp = reinterpret_cast<T*>(gdn_smem + SM::off_vp);
  T* Aq = reinterpret_cast<T*>(gdn_smem + SM::off_aq);
  float* Gs = reinterpret_cast<float*>(gdn_smem + SM::off_gs);

  const SeqInfo s = locate_chunk(blockIdx.x, cu, chunk_offsets, N, T_len);
  if (s.nvalid <= 0) return;
  const int tid = threadIdx.x, wave = tid >> 6;
  const int h = blockIdx.y, hq = h / (Hv / Hqk), nvalid = s.nvalid, v0 = blockIdx.z * BV;
  const int64_t tok0 = s.bos + (int64_t)s.chunk * kChunk;

  load_tile<T, DK>(Qs, LDK, q + (tok0 * Hqk + hq) * DK, (int64_t)Hqk * DK, nvalid, tid);
  load_tile<T, DK>(Ks, LDK, k + (tok0 * Hqk + hq) * DK, (int64_t)Hqk * DK, nvalid, tid);
  load_tile<T, DK, BV>(Sb, LDK, hbuf + (((int64_t)blockIdx.x * Hv + h) * V + v0) * DK, (int64_t)DK, BV, tid);
  load_tile<T, BV>(Vp, LDV, vn + (tok0 * Hv + h) * V + v0, (int64_t)Hv * V, nvalid, tid);
  if (tid < 64) Gs[tid] = G[(tok0 + imin(tid, nvalid - 1)) * Hv + h];
  __syncthreads();

  {  // intra-chunk scores, one 32x32 tile per wave
    const int ti = wave >> 1, tj = wave & 1;
    f32x16 acc = acc_zero();
    if (tj <= ti) mma32<T, DK, true, true>(acc, Qs + 32 * ti * LDK, LDK, Ks + 32 * tj * LDK, LDK);
    const int j = 32 * tj + acc_col();
#pragma unroll
    for (int r = 0; r < 16; ++r) {
      const int i = 32 * ti + acc_row(r);
      Aq[i * L64 + j] = Elem<T>::from_f(i >= j ? acc[r] * __expf(Gs[i] - Gs[j]) : 0.f);
    }
  }
  constexpr int NO = (2 * MT + 3) / 4;
  f32x16 O[NO];
#pragma unroll
  for (int i = 0; i < NO; ++i) {
    const int tt = wave + 4 * i;
    O[i] = acc_zero();
    if (tt < 2 * MT) {
      const int ri = tt & 1, cj = tt >> 1;
      mma32<T, DK, true, true>(O[i], Qs + 32 * ri * LDK, LDK, Sb + 32 * cj * LDK, LDK);
#pragma unroll
      for (int r = 0; r < 16; ++r) O[i][r] *= __expf(Gs[32 * ri + acc_row(r)]);
    }
  }
  __syncthreads();
  T* og = o + (tok0 * Hv + h) * V + v0;
#pragma unroll
  for (int i = 0; i < NO; ++i) {
    const int tt = wave + 4 * i;
    if (tt < 2 * MT) {
      const int ri = tt & 1, cj = tt >> 1;
      mma32<T, 64, true, false>(O[i], Aq + 32 * ri * L64, L64, Vp + 32 * cj, LDV);
#pragma unroll
      for (int r = 0; r < 16; ++r) O[i][r] *= scale;
      acc_to_global(O[i], og, (int64_t)Hv * V, 32 * ri, 32 * cj, nvalid);
    }
  }
}

// ---------------------------------------------------------------------------------------------
// host side
// ---------------------------------------------------------------------------------------------
template <typename K> static int set_lds(K kernel, int bytes) {
  return (int)hipFuncSetAttribute(reinterpret_cast<const void*>(kernel), hipFuncAttributeMaxDynamicSharedMemorySize,
                                  bytes);
}

template <typename T, int DK, int BVP, int BVS, int BVO>
static int chunk_fwd_launch(const ChunkDims& d, const ChunkWorkspace& L, const void* q, const void* k, const void* v,
                            const float* g, const float* beta, const float* h0, const int64_t* cu, void* o, float* ht,
                            unsigned char* ws, float scale, int l2norm, hipStream_t st) {
  const int64_t tok = d.tokens();
  const int nc = (int)d.max_chunks();
  int* chunk_offsets = reinterpret_cast<int*>(ws + L.chunk_offsets);
  const T* qq = (const T*)q;
  const T* kk = (const T*)k;
  if (cu != nullptr) GDN_LAUNCH(kKernChunkTable, st, chunk_table_kernel, dim3(1), dim3(kThreads), 0, st, cu, chunk_offsets, d.N);
  if (l2norm) {
    constexpr int LPR = DK / Elem<T>::kVec;
    const int64_t rows = tok * d.Hqk;
    T* qn = reinterpret_cast<T*>(ws + L.qn);
    T* kn = reinterpret_cast<T*>(ws + L.kn);
    GDN_LAUNCH(kKernL2Norm, st, (l2norm_fwd_kernel<T, DK>),
                       dim3((unsigned)((rows + kThreads / LPR - 1) / (kThreads / LPR)), 2), dim3(kThreads), 0, st, qq,
                       kk, qn, kn, rows);
    qq = qn;
    kk = kn;
  }
  float* G = reinterpret_cast<float*>(ws + L.G);
  T* Ai = reinterpret_cast<T*>(ws + L.Ai);
  T* W = reinterpret_cast<T*>(ws + L.W);
  T* VN = reinterpret_cast<T*>(ws + L.VN);
  T* H = reinterpret_cast<T*>(ws + L.H);
  {
    auto kern = chunk_prep_kernel<T, DK, BVP>;
    constexpr int smem = PrepSmem<T, DK, BVP>::bytes;
    if (int e = set_lds(kern, smem)) return e;
    GDN_LAUNCH(kKernPrep, st, kern, dim3(nc, d.Hv), dim3(kThreads), smem, st, kk, (const T*)v, g, beta, cu,
                       (const int*)chunk_offsets, G, Ai, W, VN, d.T, d.N, d.Hqk, d.Hv, d.V);
  }
  {
    auto kern = chunk_state_kernel<T, DK, BVS>;
    constexpr int smem = StateSmem<T, DK, BVS>::bytes;
    if (int e = set_lds(kern, smem)) return e;
    GDN_LAUNCH(kKernStateFwd, st, kern, dim3(d.N * d.Hv, d.V / BVS), dim3(kThreads), smem, st, kk, (const T*)W, VN,
                       (const float*)G, h0, ht, H, cu, (const int*)chunk_offsets, d.T, d.Hqk, d.Hv, d.V);
  }
  {
    auto kern = chunk_out_kernel<T, DK, BVO>;
    constexpr int smem = OutSmem<T, DK, BVO>::bytes;
    if (int e = set_lds(kern, smem)) return e;
    GDN_LAUNCH(kKernOut, st, kern, dim3(nc, d.Hv, d.V / BVO), dim3(kThreads), smem, st, qq, kk, (const T*)VN, (const T*)H,
                       (const float*)G, (T*)o, cu, (const int*)chunk_offsets, d.T, d.N, d.Hqk, d.Hv, d.V, scale);
  }
  return (int)hipGetLastError();
}

}  // namespace gdn

extern "C" int64_t gdn_chunk_workspace_bytes(int B, int T, int N, int Hqk, int Hv, int K, int V, int dtype,
                                             int with_backward) {
  // one layout for padded and packed input: the packed chunk bound is the larger of the two
  gdn::ChunkDims d{B, T, N, Hqk, Hv, K, V, true};
  const gdn::ChunkWorkspace w = gdn::chunk_workspace_layout(d, dtype == 0 ? 4 : 2);
  return with_backward ? w.total_bytes : w.fwd_bytes;
}

extern "C" int gdn_chunk_fwd(const void* q, const void* k, const void* v, const float* g, const float* beta,
                             const float* initial_state, const int64_t* cu_seqlens, void* o, float* final_state,
                             void* workspace, int64_t workspace_bytes, int B, int T, int N, int Hqk, int Hv, int K,
                             int V, float scale, int use_qk_l2norm, int dtype, void* stream) {
  using namespace gdn;
  if (!q || !k || !v || !g || !beta || !o || !workspace) return -1;
  ChunkDims d{B, T, N, Hqk, Hv, K, V, cu_seqlens != nullptr};
  if (int e = chunk_check_dims(d, dtype)) return e;
  ChunkDims dl = d;
  dl.varlen = true;  // one layout for both modes (the packed bound is the larger)
  const ChunkWorkspace L = chunk_workspace_layout(dl, dtype == 0 ? 4 : 2);
  if (workspace_bytes < L.fwd_bytes) return -5;
  if ((reinterpret_cast<uintptr_t>(workspace) & 255) != 0) return -5;
  unsigned char* ws = static_cast<unsigned char*>(workspace);
  hipStream_t st = (hipStream_t)stream;
#define GDN_FWD(T_, DK_, BVP_, BVS_, BVO_) \
  return chunk_fwd_launch<T_, DK_, BVP_, BVS_, BVO_>(d, L, q, k, v, g, beta, initial_state, cu_seqlens, o, final_state, ws, scale, use_qk_l2norm, st)
  const bool wide = (V % 128 == 0);
  if (dtype == 1) {
    if (K == 128 && wide) GDN_FWD(bf16_t, 128, 128, 64, 128);
    if (K == 128) GDN_FWD(bf16_t, 128, 64, 64, 64);
    if (K == 64 && wide) GDN_FWD(bf16_t, 64, 128, 64, 128);
    GDN_FWD(bf16_t, 64, 64, 64, 64);
  } else {
    if (K == 128) GDN_FWD(float, 128, 64, 64, 64);
    GDN_FWD(float, 64, 64, 64, 64);
  }
#undef GDN_FWD
}
