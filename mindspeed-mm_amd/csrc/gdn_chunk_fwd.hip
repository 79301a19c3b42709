// Chunked gated delta rule, forward pass (chunk = 64 tokens).  Per sequence and value head, with
// G the chunk-local cumulative log decay and Gam_ij = e^{G_i - G_j}:
//     L  = strict_tril(beta_i (k_i.k_j) Gam_ij)          Tm = (I + L)^-1
//     W  = Tm (beta e^G . K)      U = Tm (beta . V)
//     V' = U - W S                O = scale [ (e^G . Q) S + tril(Q K^T . Gam) V' ]
//     S <- e^{G_last} S + (e^{G_last - G} . K)^T V'
// Math: mindspeed_mm/fsdp/models/qwen3_5/modeling_qwen3_5.py:398-475; stage split as in
// mindspeed_mm/fsdp/ops/gdn/chunk_gated_delta_rule.py:30-85 (cumsum, KK^T, tril solve, W/U, state
// recurrence, output), fused here into two launches:
//     chunk_prep_kernel   per (chunk, head):  G, Tm, W, U, tril(QK^T . Gam)      -- MFMA + fp32 block solve
//     chunk_fwd_kernel    per (sequence, head, 32-column state slab), sequential in chunks: V', O, S
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
// chunk_prep_kernel: everything that is independent across chunks.
//   G (cumulative decay), Tm = (I+L)^-1, W = Tm (beta e^G K), U = Tm (beta V), Aq = tril(Q K^T . Gam)
// U is written in accumulator-fragment order -- for tile (32-row block ri, 32-column block vb) lane l stores its 16
// accumulator values as 16/VEC vectors at U[chunk][head][vb][ri][part][l][0..VEC) -- which is exactly how the
// recurrence kernel reads it back (straight copy to LDS, conflict-free 16-byte fragment reads).
// ---------------------------------------------------------------------------------------------
template <typename T, int DK, int BV> struct PrepSmem {
  static constexpr int LDK = lds_ld<T>(DK), LDV = lds_ld<T>(BV), L64 = lds_ld<T>(64);
  static constexpr int kv_elems = 64 * (LDK > LDV ? LDK : LDV);
  static constexpr int off_ks = 0;  // K tile, scaled in place to beta e^G K after the score tiles
  static constexpr int off_qs = off_ks + 64 * LDK * (int)sizeof(T);  // Q tile, later the (beta V) tile
  static constexpr int off_as = off_qs + kv_elems * (int)sizeof(T);
  static constexpr int off_ti = off_as + 64 * kLF * 4;
  static constexpr int off_tms = off_ti + 64 * kLF * 4;
  static constexpr int off_misc = off_tms + 64 * L64 * (int)sizeof(T);
  static constexpr int bytes = off_misc + 3 * 64 * 4;
};

template <typename T, int DK, int BV>
__global__ __launch_bounds__(kThreads) void chunk_prep_kernel(
    const T* __restrict__ q, const T* __restrict__ k, const T* __restrict__ v, const float* __restrict__ g,
    const float* __restrict__ beta, const int64_t* __restrict__ cu, const int* __restrict__ chunk_offsets,
    float* __restrict__ G_out, T* __restrict__ Ai_out, T* __restrict__ W_out, T* __restrict__ U_out,
    T* __restrict__ Aq_out, int T_len, int N, int Hqk, int Hv, int V) {
  using SM = PrepSmem<T, DK, BV>;
  constexpr int LDK = SM::LDK, LDV = SM::LDV, L64 = SM::L64, VEC = Elem<T>::kVec;
  T* Ks = reinterpret_cast<T*>(gdn_smem + SM::off_ks);
  T* Kb = Ks;
  T* Qs = reinterpret_cast<T*>(gdn_smem + SM::off_qs);
  T* Vb = Qs;
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

  // ---- phase 0: cumulative decay (one lane per token), beta; K and Q tiles ----
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
  load_tile<T, DK>(Ks, LDK, k + (tok0 * Hqk + hq) * DK, (int64_t)Hqk * DK, nvalid, tid);
  load_tile<T, DK>(Qs, LDK, q + (tok0 * Hqk + hq) * DK, (int64_t)Hqk * DK, nvalid, tid);
  __syncthreads();

  // ---- phase 1: A = strict_tril(beta_i k_i.k_j Gam_ij) and Aq = tril(q_i.k_j Gam_ij), one 32x32 tile per wave ----
  {
    const int ti = wave >> 1, tj = wave & 1;
    f32x16 acc = acc_zero(), aq = acc_zero();
    if (tj <= ti) {
      mma32<T, DK, true, true>(acc, Ks + 32 * ti * LDK, LDK, Ks + 32 * tj * LDK, LDK);
      mma32<T, DK, true, true>(aq, Qs + 32 * ti * LDK, LDK, Ks + 32 * tj * LDK, LDK);
    }
    const int j = 32 * tj + acc_col();
    T* aqg = Aq_out + (tok0 * Hv + h) * 64;
#pragma unroll
    for (int r = 0; r < 16; ++r) {
      const int i = 32 * ti + acc_row(r);
      const float gam = i >= j ? __expf(Gs[i] - Gs[j]) : 0.f;
      As[i * kLF + j] = i > j ? bs[i] * acc[r] * gam : 0.f;
      if (i < nvalid) aqg[(int64_t)i * Hv * 64 + j] = Elem<T>::from_f(aq[r] * gam);
    }
  }
  __syncthreads();

  // K tile -> beta e^G K in place; (beta V) tile of the first V block replaces Q while the solve runs
  {
    constexpr int CPR = DK / VEC;
    for (int c = tid; c < 64 * CPR; c += kThreads) {
      const int row = c / CPR, cc = c % CPR;
      Vec16<T> x = ld16(Ks + row * LDK + cc * VEC);
      const float sc = egs[row];
#pragma unroll
      for (int e = 0; e < VEC; ++e) x.set(e, x.get(e) * sc);
      st16(Kb + row * LDK + cc * VEC, x);
    }
  }
  const T* vg = v + (tok0 * Hv + h) * V;
  load_tile_scaled<T, BV>(Vb, LDV, vg, (int64_t)Hv * V, nvalid, bs, tid);

  // ---- phase 2a: invert the four 16x16 diagonal blocks by forward substitution (fp32) ----
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

  // ---- phase 2b: 16 -> 32 merges  X = -T22 (A21 T11); the zero upper triangle of As is scratch ----
  {
    const int p = wave & 1;           // waves 0,1 write; 2,3 repeat the same values (benign)
    const int C0 = 32 * p, R0 = C0 + 16;
    const int li = lane & 15, lk = lane >> 4;
    f32x4 y = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int kk = 0; kk < 4; ++kk)
      y = mfma16_f32(y, As[(R0 + li) * kLF + C0 + 4 * kk + lk], Ti[(C0 + 4 * kk + lk) * kLF + C0 + li]);
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

  // ---- phase 2c: 32 -> 64 merge, one 16x16 tile of the 32x32 block per wave ----
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

  // ---- phase 3: Tm in operand precision, kept for the backward pass ----
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

  // ---- phase 4: W = Tm (beta e^G K) ----
  {
    T* wg = W_out + (tok0 * Hv + h) * DK;
    for (int tt = wave; tt < 2 * (DK / 32); tt += 4) {
      const int ri = tt & 1, cj = tt >> 1;
      f32x16 acc = acc_zero();
      mma32<T, 64, true, false>(acc, Tms + 32 * ri * L64, L64, Kb + 32 * cj, LDK);
      acc_to_global(acc, wg, (int64_t)Hv * DK, 32 * ri, 32 * cj, nvalid);
    }
  }
  // ---- phase 5: U = Tm (beta V), V block by V block, stored in fragment order ----
  for (int vb = 0; vb < V / BV; ++vb) {
    if (vb > 0) {
      __syncthreads();
      load_tile_scaled<T, BV>(Vb, LDV, vg + vb * BV, (int64_t)Hv * V, nvalid, bs, tid);
      __syncthreads();
    }
    for (int tt = wave; tt < 2 * (BV / 32); tt += 4) {
      const int ri = tt & 1, cj = tt >> 1;
      f32x16 acc = acc_zero();
      mma32<T, 64, true, false>(acc, Tms + 32 * ri * L64, L64, Vb + 32 * cj, LDV);
      const int vblk = vb * (BV / 32) + cj;
      T* ug = U_out + ((((int64_t)blockIdx.x * Hv + h) * (V / 32) + vblk) * 2 + ri) * (64 * 16);
#pragma unroll
      for (int c = 0; c < 16 / VEC; ++c) {
        Vec16<T> x = zero16<T>();
#pragma unroll
        for (int e = 0; e < VEC; ++e) x.set(e, acc[c * VEC + e]);
        st16(ug + (c * 64 + lane) * VEC, x);
      }
    }
  }
}

// ---------------------------------------------------------------------------------------------
// chunk_fwd_kernel: the inter-chunk recurrence fused with the output.  One wave owns a 32-column slab of the
// state S[K, 32] in fp32 accumulators for the whole sequence, and for every chunk does
//     V' = U - W S        O = scale [ e^G . (Q S) + Aq V' ]        S <- e^{G_last} S + K^T (e^{G_last-G} . V')
// Every B operand (S, V') is taken straight from accumulator registers (see frag_b_from_acc), so the waves
// of a workgroup never exchange data and the chain W S -> V' -> S needs no LDS round trip.  The A operands
// (W, Q, Aq row-major, K transposed) are staged in LDS by NW dedicated loader waves of the same workgroup; with
// STAGES = 2 they run one chunk ahead of the NW compute waves and the two roles meet at one barrier per chunk.
// ---------------------------------------------------------------------------------------------
template <typename T, int DK, int NW, int STAGES> struct FwdSmem {
  static constexpr int LDK = lds_ld<T>(DK), L64 = lds_ld<T>(64);
  static constexpr int off_ws = 0;
  static constexpr int off_qs = off_ws + 64 * LDK * (int)sizeof(T);
  static constexpr int off_kt = off_qs + 64 * LDK * (int)sizeof(T);
  static constexpr int off_aq = off_kt + DK * L64 * (int)sizeof(T);
  static constexpr int off_uf = off_aq + 64 * L64 * (int)sizeof(T);
  static constexpr int off_gs = off_uf + NW * 2 * 64 * 16 * (int)sizeof(T);
  static constexpr int stage = off_gs + 2 * 64 * 4;
  static constexpr int bytes = STAGES * stage;
};

template <typename T, int DK, int NW, int STAGES>
__global__ __launch_bounds__(128 * NW) void chunk_fwd_kernel(
    const T* __restrict__ q, const T* __restrict__ k, const T* __restrict__ w, const T* __restrict__ ufrag,
    const T* __restrict__ aqk, const float* __restrict__ G, const float* __restrict__ h0, float* __restrict__ ht,
    T* __restrict__ o, T* __restrict__ vn, T* __restrict__ hbuf, const int64_t* __restrict__ cu,
    const int* __restrict__ chunk_offsets, int T_len, int Hqk, int Hv, int V, float scale) {
  using SM = FwdSmem<T, DK, NW, STAGES>;
  constexpr int LDK = SM::LDK, L64 = SM::L64, NT = 64 * NW, VEC = Elem<T>::kVec;
  constexpr int NKT = DK / 32;                                  // state tiles of a compute wave (rows of S)
  constexpr int CW = 64 * (DK / VEC) / NT, CA = 64 * (64 / VEC) / NT, CU = 16 / VEC;
  constexpr int CUL = NW * 2 * 64 * 16 / VEC / NT;              // U vectors copied by a loader thread
  static_assert(64 * (DK / VEC) % NT == 0 && 64 * (64 / VEC) % NT == 0, "tile chunks must divide over the loaders");

  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6, l32 = lane & 31;
  const int n = blockIdx.x / Hv, h = blockIdx.x % Hv, hq = h / (Hv / Hqk);
  const int64_t bos = cu ? cu[n] : (int64_t)n * T_len;
  const int len = cu ? (int)(cu[n + 1] - bos) : T_len;
  const int nchunks = (len + kChunk - 1) / kChunk;
  const int64_t chunk_base = cu ? chunk_offsets[n] : (int64_t)n * ((T_len + kChunk - 1) / kChunk);

  if (wave >= NW) {
    // ================= loader waves: global -> LDS stage, one chunk ahead of the compute waves =================
    const int lt = tid - NT;
    for (int c = 0; c < nchunks; ++c) {
      const int buf = (STAGES == 2) ? (c & 1) : 0;
      if (STAGES == 1 && c > 0) __syncthreads();              // (B) the single stage is free again
      unsigned char* base = gdn_smem + buf * SM::stage;
      T* Ws = reinterpret_cast<T*>(base + SM::off_ws);
      T* Qs = reinterpret_cast<T*>(base + SM::off_qs);
      T* KT = reinterpret_cast<T*>(base + SM::off_kt);
      T* Aq = reinterpret_cast<T*>(base + SM::off_aq);
      T* Uf = reinterpret_cast<T*>(base + SM::off_uf);
      float* Gs = reinterpret_cast<float*>(base + SM::off_gs);
      const int64_t tok0 = bos + (int64_t)c * kChunk;
      const int nvalid = imin(kChunk, len - c * kChunk);
      Vec16<T> pw[CW], pq[CW], pk[CW], pa[CA], pu[CUL];
      const float g_last = G[(tok0 + nvalid - 1) * Hv + h];
#pragma unroll
      for (int i = 0; i < CW; ++i) {
        const int id = lt + i * NT;
        const int row = id / (DK / VEC), cc = id % (DK / VEC);          // row-major tiles: W, Q
        pw[i] = row < nvalid ? ld16(w + ((tok0 + row) * Hv + h) * DK + cc * VEC) : zero16<T>();
        pq[i] = row < nvalid ? ld16(q + ((tok0 + row) * Hqk + hq) * DK + cc * VEC) : zero16<T>();
        const int rowt = id % kChunk, cct = id / kChunk;                 // K goes in transposed: rows fastest
        pk[i] = rowt < nvalid ? ld16(k + ((tok0 + rowt) * Hqk + hq) * DK + cct * VEC) : zero16<T>();
      }
#pragma unroll
      for (int i = 0; i < CA; ++i) {
        const int id = lt + i * NT;
        const int row = id / (64 / VEC), cc = id % (64 / VEC);
        pa[i] = row < nvalid ? ld16(aqk + ((tok0 + row) * Hv + h) * 64 + cc * VEC) : zero16<T>();
      }
      const T* ug = ufrag + (((chunk_base + c) * Hv + h) * (V / 32) + blockIdx.y * NW) * (2 * 64 * 16);
#pragma unroll
      for (int i = 0; i < CUL; ++i) pu[i] = ld16(ug + (lt + i * NT) * VEC);
      // every loader lane owns token lt%64 in the transposed K staging: its decay towards the chunk end
      const float kdec = __expf(g_last - G[(tok0 + imin(lt & 63, nvalid - 1)) * Hv + h]);
      if (lt < 64) Gs[lt] = G[(tok0 + imin(lt, nvalid - 1)) * Hv + h];
#pragma unroll
      for (int i = 0; i < CW; ++i) {
        const int id = lt + i * NT;
        const int row = id / (DK / VEC), cc = id % (DK / VEC);
        st16(Ws + row * LDK + cc * VEC, pw[i]);
        st16(Qs + row * LDK + cc * VEC, pq[i]);
        const int rowt = id % kChunk, cct = id / kChunk;      // rowt == lt % 64 because NT is a multiple of 64
#pragma unroll
        for (int e = 0; e < VEC; ++e) KT[(cct * VEC + e) * L64 + rowt] = Elem<T>::from_f(pk[i].get(e) * kdec);
      }
#pragma unroll
      for (int i = 0; i < CUL; ++i) st16(Uf + (lt + i * NT) * VEC, pu[i]);
#pragma unroll
      for (int i = 0; i < CA; ++i) {
        const int id = lt + i * NT;
        const int row = id / (64 / VEC), cc = id % (64 / VEC);
        st16(Aq + row * L64 + cc * VEC, pa[i]);
      }
      __syncthreads();                                         // (A) chunk c is staged
    }
    return;
  }

  // ================= compute waves: one 32-column slab of the state each =================
  const int vblk = blockIdx.y * NW + wave, v0 = 32 * vblk;
  f32x16 S[NKT];
#pragma unroll
  for (int kt = 0; kt < NKT; ++kt) {
    S[kt] = acc_zero();
    if (h0 != nullptr) {
#pragma unroll
      for (int r = 0; r < 16; ++r)
        S[kt][r] = h0[(((int64_t)n * Hv + h) * DK + 32 * kt + acc_row(r)) * V + v0 + acc_col()];
    }
  }
  for (int c = 0; c < nchunks; ++c) {
    const int buf = (STAGES == 2) ? (c & 1) : 0;
    __syncthreads();                       // (A) stage `buf` holds chunk c
    unsigned char* base = gdn_smem + buf * SM::stage;
    const T* Ws = reinterpret_cast<const T*>(base + SM::off_ws);
    const T* Qs = reinterpret_cast<const T*>(base + SM::off_qs);
    const T* KT = reinterpret_cast<const T*>(base + SM::off_kt);
    const T* Aq = reinterpret_cast<const T*>(base + SM::off_aq);
    const T* Uf = reinterpret_cast<const T*>(base + SM::off_uf) + wave * (2 * 64 * 16);
    const float* Gs = reinterpret_cast<const float*>(base + SM::off_gs);
    const int64_t tok0 = bos + (int64_t)c * kChunk;
    const int nvalid = imin(kChunk, len - c * kChunk);
    const float glast = Gs[63];
    int64_t row_v = V, row_hv = (int64_t)Hv * V;   // row strides of the h / o,v_new stores
    GDN_OPAQUE(row_v);
    GDN_OPAQUE(row_hv);

    AccB<T> Sb[NKT];
#pragma unroll
    for (int kt = 0; kt < NKT; ++kt) Sb[kt].pack(S[kt]);
    if (hbuf != nullptr) {                 // state before this chunk, for the backward pass
      T* hg = hbuf + (((chunk_base + c) * Hv + h) * DK) * V + v0;
#pragma unroll
      for (int kt = 0; kt < NKT; ++kt) acc_to_global(S[kt], hg, row_v, 32 * kt, 0, DK);
    }
    GDN_PHASE_FENCE();
    // V' = U - W S, then packed as a B operand (for O and for the state update)
    AccB<T> Vb[2];
    T* vg = vn != nullptr ? vn + (tok0 * Hv + h) * V + v0 : nullptr;
#pragma unroll
    for (int ri = 0; ri < 2; ++ri) {
      f32x16 p = acc_zero();
#pragma unroll
      for (int kt = 0; kt < NKT; ++kt) mma32_accb<T>(p, Ws + (32 * ri + l32) * LDK + 32 * kt, Sb[kt]);
      f32x16 vp;
#pragma unroll
      for (int i = 0; i < CU; ++i) {
        const Vec16<T> u = ld16(Uf + ((ri * CU + i) * 64 + lane) * VEC);
#pragma unroll
        for (int e = 0; e < VEC; ++e) vp[i * VEC + e] = u.get(e) - p[i * VEC + e];
      }
      if (vg != nullptr) acc_to_global(vp, vg, row_hv, 32 * ri, 0, nvalid);
      Vb[ri].pack(vp);
      GDN_PHASE_FENCE();
    }
    // O = scale [ e^G . (Q S) + Aq V' ]
    T* og = o + (tok0 * Hv + h) * V + v0;
#pragma unroll
    for (int ri = 0; ri < 2; ++ri) {
      f32x16 oa = acc_zero();
#pragma unroll
      for (int kt = 0; kt < NKT; ++kt) mma32_accb<T>(oa, Qs + (32 * ri + l32) * LDK + 32 * kt, Sb[kt]);
#pragma unroll
      for (int r = 0; r < 16; ++r) oa[r] *= __expf(Gs[32 * ri + acc_row(r)]);
#pragma unroll
      for (int tj = 0; tj <= ri; ++tj) mma32_accb<T>(oa, Aq + (32 * ri + l32) * L64 + 32 * tj, Vb[tj]);
#pragma unroll
      for (int r = 0; r < 16; ++r) oa[r] *= scale;
      acc_to_global(oa, og, row_hv, 32 * ri, 0, nvalid);
      GDN_PHASE_FENCE();
    }
    // S <- e^{G_last} S + (e^{G_last - G} . K)^T V'   (the loaders staged K already scaled)
    const float eg = __expf(glast);
#pragma unroll
    for (int kt = 0; kt < NKT; ++kt) {
#pragma unroll
      for (int r = 0; r < 16; ++r) S[kt][r] *= eg;
#pragma unroll
      for (int tj = 0; tj < 2; ++tj) mma32_accb<T>(S[kt], KT + (32 * kt + l32) * L64 + 32 * tj, Vb[tj]);
      GDN_PHASE_FENCE();
    }
    if (STAGES == 1 && c + 1 < nchunks) __syncthreads();      // (B) done with the single stage
  }

  if (ht != nullptr) {
#pragma unroll
    for (int kt = 0; kt < NKT; ++kt)
#pragma unroll
      for (int r = 0; r < 16; ++r)
        ht[(((int64_t)n * Hv + h) * DK + 32 * kt + acc_row(r)) * V + v0 + acc_col()] = S[kt][r];
  }
}

// ---------------------------------------------------------------------------------------------
// host side
// ---------------------------------------------------------------------------------------------
template <typename K> static int set_lds(K kernel, int bytes) {
  return (int)hipFuncSetAttribute(reinterpret_cast<const void*>(kernel), hipFuncAttributeMaxDynamicSharedMemorySize,
                                  bytes);
}

template <typename T, int DK, int BVP, int NW, int STAGES>
static int chunk_fwd_launch(const ChunkDims& d, const ChunkWorkspace& L, const void* q, const void* k, const void* v,
                            const float* g, const float* beta, const float* h0, const int64_t* cu, void* o, float* ht,
                            unsigned char* ws, float scale, int l2norm, bool keep_for_backward, hipStream_t st) {
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
               dim3((unsigned)((rows + kThreads / LPR - 1) / (kThreads / LPR)), 2), dim3(kThreads), 0, st, qq, kk, qn,
               kn, rows);
    qq = qn;
    kk = kn;
  }
  float* G = reinterpret_cast<float*>(ws + L.G);
  T* Ai = reinterpret_cast<T*>(ws + L.Ai);
  T* W = reinterpret_cast<T*>(ws + L.W);
  T* AQ = reinterpret_cast<T*>(ws + L.AQ);
  T* U = reinterpret_cast<T*>(ws + L.U);
  T* VN = keep_for_backward ? reinterpret_cast<T*>(ws + L.VN) : nullptr;
  T* H = keep_for_backward ? reinterpret_cast<T*>(ws + L.H) : nullptr;
  {
    auto kern = chunk_prep_kernel<T, DK, BVP>;
    constexpr int smem = PrepSmem<T, DK, BVP>::bytes;
    if (int e = set_lds(kern, smem)) return e;
    GDN_LAUNCH(kKernPrep, st, kern, dim3(nc, d.Hv), dim3(kThreads), smem, st, qq, kk, (const T*)v, g, beta, cu,
               (const int*)chunk_offsets, G, Ai, W, U, AQ, d.T, d.N, d.Hqk, d.Hv, d.V);
  }
  {
    auto kern = chunk_fwd_kernel<T, DK, NW, STAGES>;
    constexpr int smem = FwdSmem<T, DK, NW, STAGES>::bytes;
    if (int e = set_lds(kern, smem)) return e;
    GDN_LAUNCH(kKernStateFwd, st, kern, dim3(d.N * d.Hv, d.V / (32 * NW)), dim3(128 * NW), smem, st, qq, kk,
               (const T*)W, (const T*)U, (const T*)AQ, (const float*)G, h0, ht, (T*)o, VN, H, cu,
               (const int*)chunk_offsets, d.T, d.Hqk, d.Hv, d.V, scale);
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
  const bool keep = workspace_bytes >= L.total_bytes;   // a workspace sized for backward also receives v_new and the states
  if ((reinterpret_cast<uintptr_t>(workspace) & 255) != 0) return -5;
  unsigned char* ws = static_cast<unsigned char*>(workspace);
  hipStream_t st = (hipStream_t)stream;
#define GDN_FWD(T_, DK_, BVP_, NW_, ST_)                                                                          \
  return chunk_fwd_launch<T_, DK_, BVP_, NW_, ST_>(d, L, q, k, v, g, beta, initial_state, cu_seqlens, o, final_state, \
                                                   ws, scale, use_qk_l2norm, keep, st)
  const bool wide = (V % 128 == 0);
  if (dtype == 1) {
    if (K == 128 && wide) GDN_FWD(bf16_t, 128, 128, 4, 2);
    if (K == 128) GDN_FWD(bf16_t, 128, 64, 2, 1);
    if (K == 64 && wide) GDN_FWD(bf16_t, 64, 128, 4, 2);
    GDN_FWD(bf16_t, 64, 64, 2, 1);
  } else {
    if (K == 128 && wide) GDN_FWD(float, 128, 64, 4, 1);
    if (K == 128) GDN_FWD(float, 128, 64, 2, 1);
    if (wide) GDN_FWD(float, 64, 64, 4, 1);
    GDN_FWD(float, 64, 64, 2, 1);
  }
#undef GDN_FWD
}
