// Chunked gated delta rule, forward pass (chunk = 64 tokens).  Per sequence and value head, with
// G the chunk-local cumulative log decay and Gam_ij = e^{G_i - G_j}:
//     L  = strict_tril(beta_i (k_i.k_j) Gam_ij)          Tm = (I + L)^-1
//     W  = Tm (beta e^G . K)      U = Tm (beta . V)
//     V' = U - W S                O = scale [ (e^G . Q) S + tril(Q K^T . Gam) V' ]
//     S <- e^{G_last} S + (e^{G_last - G} . K)^T V'
// Math: mindspeed_mm/fsdp/models/qwen3_5/modeling_qwen3_5.py:398-475; stage split as in
// mindspeed_mm/fsdp/ops/gdn/chunk_gated_delta_rule.py:30-85 (cumsum, KK^T, tril solve, W/U, state
// recurrence, output), fused here into three launches:
//     chunk_prep_kernel   per (chunk, head):  G, Tm, W, U, tril(QK^T . Gam)      -- MFMA + fp32 block solve
//     chunk_state_kernel  per (sequence, head, 32-column state slab), sequential in chunks: V', S
//     chunk_out_kernel    per (chunk, head, 32-column block): O
// A ragged last chunk is zero padded in LDS (k = v = beta = g = 0 is exact for this recurrence).
#include "gdn_chunk.h"
#include "gdn_common.h"
#include "gdn_profile.h"
#include "gdn_rmsnorm_gated.h"

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

// A [64, DK] q or k tile on its way into LDS, in two steps so that the requests of both tiles (and of the gates) are
// in flight together instead of one 16-byte piece at a time: tile_qk_request() issues this thread's loads (rows past
// the end of the sequence are zero), tile_qk_finish() applies the optional l2 norm (y = x rsqrt(sum x^2 + 1e-6) over
// the row, modeling_qwen3_5.py:392-395; fp32 arithmetic, result rounded to T; a row sits on DK/VEC neighbouring lanes
// that combine their partial sums with data-parallel-primitive moves), writes the tile to
// LDS and, on request, the normalised rows (row stride y_stride) and 1/|x| (stride rstd_stride) to global memory.
template <typename T, int DK> struct TileQK {
  static constexpr int V = Elem<T>::kVec, CPR = DK / V, PT = 64 * CPR / kThreads;   // lanes per row; pieces per thread
  static_assert((64 * CPR) % kThreads == 0, "every thread takes the same number of pieces");
  Vec16<T> x[PT];
};
template <typename T, int DK>
__device__ __forceinline__ void tile_qk_request(TileQK<T, DK>& t, const T* g, int64_t row_stride, int nvalid, int tid) {
  constexpr int V = TileQK<T, DK>::V, CPR = TileQK<T, DK>::CPR;
#pragma unroll
  for (int i = 0; i < TileQK<T, DK>::PT; ++i) {
    const int c = tid + i * kThreads, row = c / CPR, cc = c % CPR;
    t.x[i] = ld16(g + (int64_t)imin(row, nvalid - 1) * row_stride + cc * V);   // the same load on every path
  }
}
template <typename T, int DK>
__device__ __forceinline__ void tile_qk_finish(TileQK<T, DK>& t, T* lds, int ld, int nvalid, int tid, bool l2norm,
                                               T* y_out, int64_t y_stride, float* rstd_out, int64_t rstd_stride) {
  constexpr int V = TileQK<T, DK>::V, CPR = TileQK<T, DK>::CPR;
#pragma unroll
  for (int i = 0; i < TileQK<T, DK>::PT; ++i) {
    const int c = tid + i * kThreads, row = c / CPR, cc = c % CPR;
    const bool ok = row < nvalid;
    Vec16<T> x = ok ? t.x[i] : zero16<T>();
    if (l2norm) {   // uniform: every lane takes part in the shuffles
      float f[V], ss = 0.f;
      unpack16<T>(x, f);
#pragma unroll
      for (int e = 0; e < V; ++e) ss += f[e] * f[e];
      ss = lane_group_sum<CPR>(ss);
      const float r = rsqrtf(ss + 1e-6f);
#pragma unroll
      for (int e = 0; e < V; ++e) f[e] *= r;
      x = pack16<T>(f);
      if (ok && y_out != nullptr) st16(y_out + (int64_t)row * y_stride + cc * V, x);
      if (ok && rstd_out != nullptr && cc == 0) rstd_out[(int64_t)row * rstd_stride] = r;
    }
    st16(lds + row * ld + cc * V, x);
  }
}

// ---------------------------------------------------------------------------------------------
// chunk_prep_kernel: everything that is independent across chunks.
//   G (cumulative decay), Tm = (I+L)^-1, -W = -Tm (beta e^G K), U = Tm (beta V), Aq = scale tril(Q K^T . Gam),
//   per q/k group the K^T, K and Q^T tiles of the recurrence kernels
// U is written in fragment order (AccB<>): tile (32-token block ri) x (32-column block vb) at
// U[chunk][head][vb][ri][1024], 16 bytes per lane per k-group -- the recurrence kernel copies it straight to LDS.
// Three quarters of the kernel's traffic are stores, issued all along the way; its barriers order LDS traffic only
// (GDN_LDS_BARRIER), because a __syncthreads() would also wait until every store issued so far has been acknowledged.
// ---------------------------------------------------------------------------------------------
template <typename T, int DK, int BV> struct PrepSmem {
  static constexpr int LDK = lds_ld<T>(DK), LDV = lds_ld<T>(BV), L64 = lds_ld<T>(64);
  static constexpr int cmax(int a, int b) { return a > b ? a : b; }
  // Two regions, each reused once its tenant is dead, so that four workgroups (bf16) fit a CU's LDS:
  //   region 1: K tile -> Tm (fp32, solve output) -> beta e^G K (parked in registers during the solve) -> (beta V) tile
  //   region 2: Q tile -> A (fp32, solve input) -> Tm in T
  static constexpr int off_ks = 0;
  static constexpr int r1_bytes = cmax(cmax(64 * LDK * (int)sizeof(T), 64 * kLF * 4), 64 * LDV * (int)sizeof(T));
  static constexpr int off_qs = off_ks + r1_bytes;
  static constexpr int qs_bytes = cmax(cmax(64 * LDK * (int)sizeof(T), 64 * kLF * 4), 64 * L64 * (int)sizeof(T));
  static constexpr int off_ti = off_ks;
  static constexpr int off_misc = off_qs + qs_bytes;
  static constexpr int bytes = off_misc + 3 * 64 * 4;
};

template <typename T, int DK, int BV>
__global__ __launch_bounds__(kThreads) GDN_WAVES_PER_SIMD(sizeof(T) == 2 ? 4 : 3) void chunk_prep_kernel(
    const T* __restrict__ q, const T* __restrict__ k, const T* __restrict__ v, const float* __restrict__ g,
    const float* __restrict__ beta, const int64_t* __restrict__ cu, const int* __restrict__ chunk_offsets,
    float* __restrict__ G_out, T* __restrict__ Ai_out, T* __restrict__ W_out, T* __restrict__ U_out,
    T* __restrict__ Aq_out, T* __restrict__ KT_out, T* __restrict__ WF_out, T* __restrict__ KA_out,
    T* __restrict__ QT_out, float* __restrict__ rstd_q_out, float* __restrict__ rstd_k_out,
    int T_len, int N, int Hqk, int Hv, int V, float scale, int l2norm, TokenStrides ts) {
  using SM = PrepSmem<T, DK, BV>;
  constexpr int LDK = SM::LDK, LDV = SM::LDV, L64 = SM::L64, VEC = Elem<T>::kVec;
  T* Ks = reinterpret_cast<T*>(gdn_smem + SM::off_ks);
  T* Kb = Ks;                                                     // after Tm (fp32)
  T* Qs = reinterpret_cast<T*>(gdn_smem + SM::off_qs);
  float* As = reinterpret_cast<float*>(gdn_smem + SM::off_qs);    // after Q
  T* Tms = reinterpret_cast<T*>(gdn_smem + SM::off_qs);          // after A
  float* Ti = reinterpret_cast<float*>(gdn_smem + SM::off_ti);
  T* Vb = reinterpret_cast<T*>(gdn_smem + SM::off_ti);           // after beta e^G K
  float* Gs = reinterpret_cast<float*>(gdn_smem + SM::off_misc);
  float* bs = Gs + 64;
  float* egs = bs + 64;

  const SeqInfo s = locate_chunk(blockIdx.x, cu, chunk_offsets, N, T_len);
  if (s.nvalid <= 0) return;
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int h = blockIdx.y, hq = h / (Hv / Hqk), nvalid = s.nvalid;
  const int64_t tok0 = s.bos + (int64_t)s.chunk * kChunk;

  // ---- phase 0: cumulative decay (one lane per token), beta; K and Q tiles.  All requests first. ----
  TileQK<T, DK> kt, qt;
  tile_qk_request<T, DK>(kt, k + tok0 * ts.k + hq * DK, ts.k, nvalid, tid);
  tile_qk_request<T, DK>(qt, q + tok0 * ts.q + hq * DK, ts.q, nvalid, tid);
  if (wave == 0) {
    float x = lane < nvalid ? g[(tok0 + lane) * Hv + h] : 0.f;
    const float b = lane < nvalid ? beta[(tok0 + lane) * Hv + h] : 0.f;
#pragma unroll
    for (int d = 1; d < 64; d <<= 1) {
      const float t = __shfl_up(x, d);
      if (lane >= d) x += t;
    }
    Gs[lane] = x;
    bs[lane] = b;
    egs[lane] = b * __expf(x);
    G_out[((int64_t)blockIdx.x * Hv + h) * 64 + lane] = x;   // 64 contiguous values per chunk and head
  }
  {
    // q and k arrive raw; with the in-kernel l2 norm they are normalised on the way into LDS.  The first value head
    // of each q/k group also leaves 1/|q|, 1/|k| (for the output kernel, which scales q itself, and the backward pass).
    const bool keep = l2norm && (h % (Hv / Hqk)) == 0;
    const int64_t roff = ((int64_t)blockIdx.x * Hqk + hq) * 64;   // 64 contiguous values per chunk and q/k head
    tile_qk_finish<T, DK>(kt, Ks, LDK, nvalid, tid, l2norm != 0, nullptr, 0, keep ? rstd_k_out + roff : nullptr, 1);
    tile_qk_finish<T, DK>(qt, Qs, LDK, nvalid, tid, l2norm != 0, nullptr, 0, keep ? rstd_q_out + roff : nullptr, 1);
  }
  GDN_LDS_BARRIER();

  // ---- phase 1: A = strict_tril(beta_i k_i.k_j Gam_ij) and Aq = tril(q_i.k_j Gam_ij), one 32x32 tile per wave ----
  f32x16 a_tile = acc_zero();   // goes to LDS (over the Q tile) once every wave is done with Q
  {
    const int ti = wave >> 1, tj = wave & 1;
    f32x16 aq = acc_zero();
    if (tj <= ti) {
      mma32<T, DK, true, true>(a_tile, Ks + 32 * ti * LDK, LDK, Ks + 32 * tj * LDK, LDK);
      mma32<T, DK, true, true>(aq, Qs + 32 * ti * LDK, LDK, Ks + 32 * tj * LDK, LDK);
    }
    const int j = 32 * tj + acc_col();
    const float gj = Gs[j];
    const f32x16 gi = rows_ld(Gs, 32 * ti), bi = rows_ld(bs, 32 * ti);
#pragma unroll
    for (int r = 0; r < 16; ++r) {   // branch-free: where the mask discards the value the exponent is set to 0 first
      const int i = 32 * ti + acc_row(r);
      const float e = __expf(i >= j ? gi[r] - gj : 0.f);
      const float gam = i >= j ? e : 0.f;
      a_tile[r] = i > j ? bi[r] * a_tile[r] * gam : 0.f;
      aq[r] *= gam * scale;
    }
    // scale tril(Q K^T . Gam) leaves as four 32x32 tiles in fragment order, packed as they sit in the accumulator
    // (lane <-> column j, registers <-> row i): the A operand of Aq^T dO as is, of Aq V' after one turn
    AccB<T> af;
    af.pack(aq);
    af.store_stream(Aq_out + (((int64_t)blockIdx.x * Hv + h) * 4 + wave) * 1024);
  }
  // K^T as A-operand fragments for the state update: K tile fragments (lane <-> token) turned through the matrix
  // core into (lane <-> K column, registers <-> token), stored in fragment order (the decay is applied by the reader)
  {
    IdentityFrag<T> id;
    id.init();
    const bool group_first = (h % (Hv / Hqk)) == 0;   // K and Q^T tiles are shared by the value heads of a q/k group
    for (int tt = wave; tt < 2 * (DK / 32); tt += 4) {
      const int tj = tt & 1, kt = tt >> 1;
      const int64_t gtile = ((((int64_t)blockIdx.x * Hqk + hq) * (DK / 32) + kt) * 2 + tj) * 1024;
      AccB<T> kf;
      frags_from_lds<T>(kf, Ks + (32 * tj + (lane & 31)) * LDK + 32 * kt);
      if (KA_out != nullptr && group_first) kf.store_stream(KA_out + gtile);   // K as an A operand (lane <-> token)
      if (group_first) {   // K^T as an A operand (lane <-> K column), for the state update
        kf.pack(mfma_transpose<T>(kf, id));
        kf.store_stream(KT_out + gtile);
      }
      if (QT_out != nullptr && group_first) {   // Q^T as an A operand (lane <-> K column), for the backward pass
        frags_from_lds<T>(kf, Qs + (32 * tj + (lane & 31)) * LDK + 32 * kt);
        kf.pack(mfma_transpose<T>(kf, id));
        kf.store_stream(QT_out + gtile);
      }
    }
  }
  // beta e^G K, this thread's pieces of the K tile, parked in registers: the K tile's space takes the fp32 Tm first
  constexpr int KPT = 64 * (DK / VEC) / kThreads;
  Vec16<T> kreg[KPT];
#pragma unroll
  for (int i = 0; i < KPT; ++i) {
    const int c = tid + i * kThreads, row = c / (DK / VEC), cc = c % (DK / VEC);
    kreg[i] = scale16<T>(ld16(Ks + row * LDK + cc * VEC), egs[row]);
  }
  GDN_LDS_BARRIER();   // Q and K are consumed: their space takes A and Tm

  {
    const int ti = wave >> 1, tj = wave & 1, j = 32 * tj + acc_col();
#pragma unroll
    for (int r = 0; r < 16; ++r) As[(32 * ti + acc_row(r)) * kLF + j] = a_tile[r];
  }
  for (int i = tid; i < 64 * kLF; i += kThreads) Ti[i] = 0.f;
  // the first V block is requested now and parked in registers until the fp32 Tm has been consumed
  const T* vg = v + tok0 * ts.v + h * V;
  constexpr int VPT = 64 * (BV / VEC) / kThreads;   // 16-byte pieces of the V tile per thread
  Vec16<T> vreg[VPT];
#pragma unroll
  for (int i = 0; i < VPT; ++i) {
    const int c = tid + i * kThreads, row = c / (BV / VEC), cc = c % (BV / VEC);
    vreg[i] = ld16(vg + imin(row, nvalid - 1) * ts.v + cc * VEC);   // rows past the end: beta = 0 will clear them
  }
  GDN_LDS_BARRIER();

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
  GDN_LDS_BARRIER();

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
    GDN_LDS_BARRIER();
    f32x4 x = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int kk = 0; kk < 4; ++kk)
      x = mfma16_f32(x, Ti[(R0 + li) * kLF + R0 + 4 * kk + lk], As[(C0 + 4 * kk + lk) * kLF + R0 + li]);
    if (wave < 2) {
#pragma unroll
      for (int r = 0; r < 4; ++r) Ti[(R0 + 4 * lk + r) * kLF + C0 + li] = -x[r];
    }
  }
  GDN_LDS_BARRIER();

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
    GDN_LDS_BARRIER();
    f32x4 x = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int kk = 0; kk < 8; ++kk)
      x = mfma16_f32(x, Ti[(32 + 16 * ta + li) * kLF + 32 + 4 * kk + lk], As[(4 * kk + lk) * kLF + 32 + 16 * tb + li]);
#pragma unroll
    for (int r = 0; r < 4; ++r) Ti[(32 + 16 * ta + 4 * lk + r) * kLF + 16 * tb + li] = -x[r];
  }
  GDN_LDS_BARRIER();

  // ---- phase 3: Tm in operand precision, kept for the backward pass ----
  {
    constexpr int CPR = 64 / VEC;
    for (int c = tid; c < 64 * CPR; c += kThreads) {
      const int row = c / CPR, cc = c % CPR;
      float f[VEC];
#pragma unroll
      for (int e = 0; e < VEC; ++e) f[e] = Ti[row * kLF + cc * VEC + e];
      st16(Tms + row * L64 + cc * VEC, pack16<T>(f));
    }
  }
  GDN_LDS_BARRIER();
  // the fp32 Tm is consumed: its space takes the beta e^G K tile parked in registers
#pragma unroll
  for (int i = 0; i < KPT; ++i) {
    const int c = tid + i * kThreads, row = c / (DK / VEC), cc = c % (DK / VEC);
    st16(Kb + row * LDK + cc * VEC, kreg[i]);
  }
  // The V block requested above has long arrived.  Waiting for it here, before the stores of the next phases are
  // issued, keeps its first use from waiting for those stores as well (loads and stores are counted in one order).
  GDN_WAIT_VMEM();
  if (Ai_out != nullptr) {  // the four 32x32 tiles of Tm as A operands (lane <-> row, registers <-> column), for the backward
    AccB<T> tf;
    frags_from_lds<T>(tf, Tms + (32 * (wave >> 1) + (lane & 31)) * L64 + 32 * (wave & 1));
    tf.store_stream(Ai_out + (((int64_t)blockIdx.x * Hv + h) * 4 + wave) * 1024);
  }
  GDN_LDS_BARRIER();

  // ---- phase 4: W = Tm (beta e^G K), handed on in fragment order only ----
  {
    IdentityFrag<T> id;
    id.init();
    for (int tt = wave; tt < 2 * (DK / 32); tt += 4) {
      const int ri = tt & 1, cj = tt >> 1;
      f32x16 acc = acc_zero();
      mma32<T, 64, true, false>(acc, Tms + 32 * ri * L64, L64, Kb + 32 * cj, LDK);
      const int64_t tile = (((int64_t)blockIdx.x * Hv + h) * (DK / 32) + cj) * 2 + ri;
      AccB<T> wf;
      wf.pack(acc);              // (lane <-> K column, registers <-> token): -W^T as an A operand, for the backward pass
      wf.negate();               // both uses subtract the product (U - W S, dS - W^T dV')
      if (WF_out != nullptr) wf.store_stream(WF_out + tile * 1024);
      const f32x16 wt = mfma_transpose<T>(wf, id);
      wf.pack(wt);               // (lane <-> token, registers <-> K column): -W as an A operand, for U - W S
      wf.store_stream(W_out + tile * 1024);
    }
  }
  // ---- phase 5: U = Tm (beta V), V block by V block, stored in fragment order ----
  for (int vb = 0; vb < V / BV; ++vb) {
    GDN_LDS_BARRIER();   // the tile in region 1 (beta e^G K, or the previous V block) is consumed
    if (vb == 0) {     // the first (beta V) block was parked in registers
#pragma unroll
      for (int i = 0; i < VPT; ++i) {
        const int c = tid + i * kThreads, row = c / (BV / VEC), cc = c % (BV / VEC);
        st16(Vb + row * LDV + cc * VEC, scale16<T>(vreg[i], bs[row]));
      }
    } else {
      load_tile_scaled<T, BV>(Vb, LDV, vg + vb * BV, ts.v, nvalid, bs, tid);
    }
    GDN_LDS_BARRIER();
    for (int tt = wave; tt < 2 * (BV / 32); tt += 4) {
      const int ri = tt & 1, cj = tt >> 1;
      f32x16 acc = acc_zero();
      mma32<T, 64, true, false>(acc, Tms + 32 * ri * L64, L64, Vb + 32 * cj, LDV);
      const int vblk = vb * (BV / 32) + cj;
      AccB<T> uf;
      uf.pack(acc);
      uf.store_stream(U_out + ((((int64_t)blockIdx.x * Hv + h) * (V / 32) + vblk) * 2 + ri) * 1024);
    }
  }
}

// ---------------------------------------------------------------------------------------------
// chunk_state_kernel: the inter-chunk recurrence, kept as lean as possible because it is the only part of the
// forward pass that is sequential in the chunks.  One compute wave owns a 32-column slab of the state S[K, 32] in
// fp32 registers for the whole sequence and per chunk does
//     V' = U - W S            S <- e^{G_last} S + K^T (e^{G_last-G} . V')
// Both B operands (S, V') are taken straight from accumulator registers (frag_b_from_acc), so the chain
// W S -> V' -> S never touches LDS and the compute waves of a workgroup never exchange data.  S (before the chunk)
// and V' leave the kernel in fragment order, 16 bytes per lane per k-group, for chunk_out_kernel and the backward
// pass.  The A operands (-W per value head, K^T per q/k group) and U arrive in fragment order, one contiguous 16 KB
// block per chunk prepared by chunk_prep_kernel (token-major tiles would be 64 rows scattered 8 KB apart), and are
// copied to LDS in 16-byte pieces by NL loader waves of the same workgroup, which run ahead of the NW compute
// waves: loads for chunks c+2 and c+3 are in flight in registers while chunk c+1 sits in the other LDS stage; the
// two roles meet at one barrier per chunk.
// ---------------------------------------------------------------------------------------------
template <typename T, int DK, int NW, int STAGES> struct StateSmem {
  static constexpr int off_ws = 0;
  static constexpr int off_kt = off_ws + 64 * DK * (int)sizeof(T);
  static constexpr int off_uf = off_kt + DK * 64 * (int)sizeof(T);
  static constexpr int off_gl = off_uf + NW * 2048 * (int)sizeof(T);   // e^{G_last - G_t} [64], G_last
  static constexpr int stage = off_gl + 64 * 4 + 16;
  static constexpr int bytes = STAGES * stage;
};

template <typename T, int DK, int NW, int NL, int STAGES>
__global__ __launch_bounds__(64 * (NW + NL)) GDN_WAVES_PER_SIMD(sizeof(T) == 2 ? 2 : 1) void chunk_state_kernel(
    const T* __restrict__ ktf, const T* __restrict__ w, const T* __restrict__ uf, const float* __restrict__ G,
    const float* __restrict__ h0, float* __restrict__ ht, T* __restrict__ vf, T* __restrict__ hf,
    const int64_t* __restrict__ cu, const int* __restrict__ chunk_offsets, int T_len, int Hqk, int Hv, int V) {
  using SM = StateSmem<T, DK, NW, STAGES>;
  constexpr int NT = 64 * NL, VEC = Elem<T>::kVec;   // loader threads
  constexpr int NKT = DK / 32;
  constexpr int CW = 64 * (DK / VEC) / NT, CUL = NW * 2048 / VEC / NT;
  static_assert(64 * (DK / VEC) % NT == 0 && (NW * 2048 / VEC) % NT == 0, "tile chunks must divide over the loaders");
  static_assert(STAGES == 1 || STAGES == 2, "one or two LDS stages");

  const int tid = threadIdx.x, wave = tid >> 6;
  const int nh = xcd_grouped_head(blockIdx.x, gridDim.x, Hv / Hqk), n = nh / Hv, h = nh % Hv;
  const int64_t bos = cu ? cu[n] : (int64_t)n * T_len;
  const int len = cu ? (int)(cu[n + 1] - bos) : T_len;
  const int nchunks = (len + kChunk - 1) / kChunk;
  const int64_t chunk_base = cu ? chunk_offsets[n] : (int64_t)n * ((T_len + kChunk - 1) / kChunk);

  if (wave >= NW) {
    // ================= loader waves: straight 16-byte copies =================
    const int lt = tid - 64 * NW;
    // DEPTH register sets: chunk j sits in set j % DEPTH from the iteration that requests it (j - DEPTH - 1) to the
    // one that copies it to LDS (j - 1), so global loads have DEPTH chunk periods to arrive
    constexpr int DEPTH = (STAGES == 2) ? 2 : 1;
    Vec16<T> pw[DEPTH][CW], pk[DEPTH][CW], pu[DEPTH][CUL];
    float glast[DEPTH], pdec[DEPTH];
    auto issue = [&](int c, int set) {      // global -> registers
      const int nvalid = imin(kChunk, len - c * kChunk);
#pragma unroll
      for (int i = 0; i < CW; ++i) {
        const int id = lt + i * NT;
        pw[set][i] = ld16(w + ((chunk_base + c) * Hv + h) * (64 * DK) + id * VEC);
        pk[set][i] = ld16(ktf + ((chunk_base + c) * Hqk + h / (Hv / Hqk)) * (64 * DK) + id * VEC);   // shared by the group
      }
      const T* ug = uf + (((chunk_base + c) * Hv + h) * (V / 32) + blockIdx.y * NW) * 2048;
#pragma unroll
      for (int i = 0; i < CUL; ++i) pu[set][i] = ld16(ug + (lt + i * NT) * VEC);
      const float* gc = G + ((chunk_base + c) * Hv + h) * 64;
      glast[set] = gc[nvalid - 1];          // raw values only: arithmetic here would wait for every load issued so far
      pdec[set] = gc[imin(lt & 63, nvalid - 1)];
    };
    auto commit = [&](int set, int buf) {   // registers -> LDS stage
      unsigned char* base = gdn_smem + buf * SM::stage;
      T* Ws = reinterpret_cast<T*>(base + SM::off_ws);
      T* KT = reinterpret_cast<T*>(base + SM::off_kt);
      T* Uf = reinterpret_cast<T*>(base + SM::off_uf);
#pragma unroll
      for (int i = 0; i < CW; ++i) {
        const int id = lt + i * NT;
        st16(Ws + id * VEC, pw[set][i]);
        st16(KT + id * VEC, pk[set][i]);
      }
#pragma unroll
      for (int i = 0; i < CUL; ++i) st16(Uf + (lt + i * NT) * VEC, pu[set][i]);
      float* dec = reinterpret_cast<float*>(base + SM::off_gl);
      if (lt < 64) dec[lt] = __expf(glast[set] - pdec[set]);
      if (lt == 0) dec[64] = glast[set];
    };
    if (STAGES == 2) {
      // Every path through this loop issues the same loads in the same order (chunk indices past the end are clamped
      // and their data is never used), so that the number of loads in flight at each wait is a compile-time fact and
      // the waits before the LDS writes of one register set leave the younger sets in flight.
      if (nchunks == 0) return;
      issue(0, 0);
      commit(0, 0);
#pragma unroll
      for (int j = 1; j <= DEPTH; ++j) issue(imin(j, nchunks - 1), j % DEPTH);
      for (int c0 = 0;; c0 += DEPTH) {
#pragma unroll
        for (int u = 0; u < DEPTH; ++u) {
          const int c = c0 + u;
          if (c >= nchunks) return;
          GDN_LDS_BARRIER();                // (A) chunk c staged; the other stage (chunk c-1) is free
          commit((u + 1) % DEPTH, (c + 1) & 1);
          issue(imin(c + 1 + DEPTH, nchunks - 1), (u + 1) % DEPTH);
        }
      }
    } else {
      for (int c = 0; c < nchunks; ++c) {
        if (c > 0) GDN_LDS_BARRIER();       // (B) the single stage is free again
        issue(c, 0);
        commit(0, 0);
        GDN_LDS_BARRIER();                  // (A)
      }
    }
    return;
  }

  // ================= compute waves =================
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
  // The wave issues its instructions in order and a matrix instruction occupies the matrix pipe for 32 cycles, in
  // which eight vector instructions can issue: the loop body is written so that the vector work which does not
  // depend on the running product (decay of S, packing S for the next chunk, unpacking U) sits between the matrix
  // instructions instead of before or after them.
  AccB<T> Sb[NKT];
#pragma unroll
  for (int kt = 0; kt < NKT; ++kt) Sb[kt].pack(S[kt]);
  for (int c = 0; c < nchunks; ++c) {
    const int buf = (STAGES == 2) ? (c & 1) : 0;
    GDN_LDS_BARRIER();                        // (A) stage `buf` holds chunk c
    unsigned char* base = gdn_smem + buf * SM::stage;
    const T* Ws = reinterpret_cast<const T*>(base + SM::off_ws);
    const T* KT = reinterpret_cast<const T*>(base + SM::off_kt);
    const T* Uf = reinterpret_cast<const T*>(base + SM::off_uf) + wave * 2048;
    const float* dec = reinterpret_cast<const float*>(base + SM::off_gl);
    const int64_t tile0 = ((chunk_base + c) * Hv + h) * (V / 32) + vblk;

    constexpr int NP = NKT / 2;             // K tiles are processed two at a time
    AccB<T> Wf[2][2][2];                    // [buffer][32-token block][K tile of the pair]
    AccB<T> Kf[2][2][2];                    // [buffer][K tile of the pair][32-token block]
    auto load_w = [&](int b, int kp) {
#pragma unroll
      for (int ri = 0; ri < 2; ++ri)
#pragma unroll
        for (int j = 0; j < 2; ++j) Wf[b][ri][j].load(Ws + ((2 * kp + j) * 2 + ri) * 1024);
    };
    auto load_k = [&](int b, int kp) {
#pragma unroll
      for (int j = 0; j < 2; ++j)
#pragma unroll
        for (int tj = 0; tj < 2; ++tj) Kf[b][j][tj].load(KT + ((2 * kp + j) * 2 + tj) * 1024);
    };
    AccB<T> Vb[2];
    Vb[0].load(Uf);
    Vb[1].load(Uf + 1024);
    load_w(0, 0);
    if (NP > 1) load_w(1, 1);
    const float eg = __expf(dec[64]);
#pragma unroll
    for (int kt = 0; kt < NKT; ++kt) Sb[kt].store_stream(hf + (tile0 * NKT + kt) * 1024);
    // V' = U - W S: the accumulators start from U and the W tiles arrive negated; the two 32-token blocks are
    // independent accumulation chains.  The decay of S rides between the matrix instructions.
    f32x16 p0 = Vb[0].unpack(), p1 = Vb[1].unpack();
    GDN_SCHED_FENCE();
#pragma unroll
    for (int kp = 0; kp < NP; ++kp) {
#pragma unroll
      for (int j = 0; j < 2; ++j) {
        mma32_ff<T>(p0, Wf[kp & 1][0][j], Sb[2 * kp + j]);
        mma32_ff<T>(p1, Wf[kp & 1][1][j], Sb[2 * kp + j]);
#pragma unroll
        for (int r = 0; r < 16; ++r) S[2 * kp + j][r] *= eg;
        GDN_INTERLEAVE_MFMA_VALU(2 * AccK<T>::kGroups, 16 / (2 * AccK<T>::kGroups));
      }
      GDN_SCHED_FENCE();
      if (kp + 2 < NP) load_w(kp & 1, kp + 2);
      if (kp == (NP > 1 ? NP - 2 : 0)) load_k(0, 0);
      if (kp == NP - 1 && NP > 1) load_k(1, 1);
      GDN_SCHED_FENCE();
    }
    const f32x16 d0 = rows_ld(dec, 0), d1 = rows_ld(dec, 32);
    Vb[0].pack(p0);
    Vb[1].pack(p1);
    Vb[0].store_stream(vf + (tile0 * 2 + 0) * 1024);
    Vb[1].store_stream(vf + (tile0 * 2 + 1) * 1024);
    // the decay of the state update rides on V': (e^{G_last - G} . K)^T V' = K^T (e^{G_last - G} . V'), so that the
    // K^T tiles are the same for every value head of a q/k group
#pragma unroll
    for (int r = 0; r < 16; ++r) { p0[r] *= d0[r]; p1[r] *= d1[r]; }
    Vb[0].pack(p0);
    Vb[1].pack(p1);
    GDN_SCHED_FENCE();
    // S <- e^{G_last} S + K^T (e^{G_last - G} . V'); a finished tile of S is packed for the next chunk while the
    // matrix pipe works on the following ones
#pragma unroll
    for (int kp = 0; kp < NP; ++kp) {
#pragma unroll
      for (int j = 0; j < 2; ++j) {
        const int kt = 2 * kp + j;
        mma32_ff<T>(S[kt], Kf[kp & 1][j][0], Vb[0]);
        mma32_ff<T>(S[kt], Kf[kp & 1][j][1], Vb[1]);
        if (kt >= 2) Sb[kt - 2].pack(S[kt - 2]);
      }
      GDN_SCHED_FENCE();
      if (kp + 2 < NP) { load_k(kp & 1, kp + 2); GDN_SCHED_FENCE(); }
    }
#pragma unroll
    for (int kt = (NKT >= 2 ? NKT - 2 : 0); kt < NKT; ++kt) Sb[kt].pack(S[kt]);
    if (STAGES == 1 && c + 1 < nchunks) GDN_LDS_BARRIER();      // (B) done with the single stage
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
// chunk_out_kernel:  O = scale e^G . (Q S) + (scale Aq) V', parallel over (chunk, head, 32-column block).
// S and V' arrive in fragment order and go from global memory straight into B-operand registers.
// NORM: the workgroup's NW waves hold whole rows of a head (V = 32 NW) and the gated RMSNorm that follows the rule
// in the layer (modeling_qwen3_5.py:897-900) is applied to the rows before they leave: y = norm(o) * silu(gate),
// with the stand-alone operator's arithmetic on the same 16-byte pieces and its order of additions (pieces of a
// row: neighbouring lanes pairwise, then the waves pairwise), so both give the same bits.  o itself and 1/rms are
// written only on request (a backward pass needs them).
// ---------------------------------------------------------------------------------------------
template <typename T, int DK, int NW> struct OutSmem {
  static constexpr int LDK = lds_ld<T>(DK);
  static constexpr int off_qs = 0;
  static constexpr int off_patch = off_qs + 64 * LDK * (int)sizeof(T);
  static constexpr int off_eg = off_patch + NW * Patch<T>::kElems * (int)sizeof(T);
  static constexpr int off_ss = off_eg + 64 * 4;       // NORM: sums of squares [NW waves][64 rows]
  static constexpr int bytes = off_ss + NW * 64 * 4;
};

// operands of the fused norm: gate and y [tokens, Hv, V] in T, weight [V] in TW; o_opt, rstd_opt may be null
template <typename T, typename TW> struct OutNorm {
  const T* gate;
  const TW* weight;
  T* y;
  float* rstd_opt;
  float eps;
};

template <typename T, int DK, int NW, bool NORM, typename TW>
__global__ __launch_bounds__(64 * NW) GDN_WAVES_PER_SIMD(sizeof(T) == 2 ? 4 : 2) void chunk_out_kernel(
    const T* __restrict__ q, const T* __restrict__ aqf, const T* __restrict__ vf, const T* __restrict__ hf,
    const float* __restrict__ G, T* __restrict__ o, const int64_t* __restrict__ cu,
    const int* __restrict__ chunk_offsets, int T_len, int N, int Hqk, int Hv, int V, float scale, int64_t q_stride,
    const float* __restrict__ rstd_q, OutNorm<T, TW> nm) {
  using SM = OutSmem<T, DK, NW>;
  constexpr int LDK = SM::LDK, NT = 64 * NW, VEC = Elem<T>::kVec, NKT = DK / 32;
  T* Qs = reinterpret_cast<T*>(gdn_smem + SM::off_qs);
  float* Eg = reinterpret_cast<float*>(gdn_smem + SM::off_eg);
  const SeqInfo s = locate_chunk(blockIdx.x, cu, chunk_offsets, N, T_len);
  if (s.nvalid <= 0) return;
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6, l32 = lane & 31;
  const int h = blockIdx.y, hq = h / (Hv / Hqk), nvalid = s.nvalid;
  const int vblk = blockIdx.z * NW + wave, v0 = 32 * vblk;
  const int64_t tok0 = s.bos + (int64_t)s.chunk * kChunk;
  const int64_t ch = (int64_t)blockIdx.x * Hv + h;
  const int64_t tile0 = ch * (V / 32) + vblk;
  T* patch = reinterpret_cast<T*>(gdn_smem + SM::off_patch) + wave * Patch<T>::kElems;

  // operands that come in fragment order are requested first, the LDS tile while they are in flight
  AccB<T> Sb[NKT], Vb[2], Af[3];
#pragma unroll
  for (int kt = 0; kt < NKT; ++kt) Sb[kt].load(hf + (tile0 * NKT + kt) * 1024);
  Vb[0].load(vf + tile0 * 2048);
  Vb[1].load(vf + tile0 * 2048 + 1024);
  Af[0].load(aqf + (ch * 4 + 0) * 1024);   // tiles (0,0), (1,0), (1,1) of tril(Q K^T . Gam)
  Af[1].load(aqf + (ch * 4 + 2) * 1024);
  Af[2].load(aqf + (ch * 4 + 3) * 1024);
  // q arrives raw; with the in-kernel l2 norm its rows are scaled by the 1/|q| the prep kernel left (the same fp32
  // product and rounding it applied itself: no normalised copy of q is kept in memory)
  constexpr int QPT = 64 * (DK / VEC) / NT;   // pieces of the Q tile per thread: all requested before the first is used
  static_assert(64 * (DK / VEC) % NT == 0, "every thread takes the same number of pieces of the Q tile");
  Vec16<T> qreg[QPT];
  float qs[QPT];
#pragma unroll
  for (int i = 0; i < QPT; ++i) {
    const int c = tid + i * NT, row = imin(c / (DK / VEC), nvalid - 1), cc = c % (DK / VEC);
    qreg[i] = ld16(q + (tok0 + row) * q_stride + hq * DK + cc * VEC);
    qs[i] = rstd_q != nullptr ? rstd_q[((int64_t)blockIdx.x * Hqk + hq) * 64 + row] : 1.f;
  }
  const float gval = G[ch * 64 + imin(tid & 63, nvalid - 1)];
#pragma unroll
  for (int i = 0; i < QPT; ++i) {
    const int c = tid + i * NT, row = c / (DK / VEC), cc = c % (DK / VEC);
    Vec16<T> x = zero16<T>();
    if (row < nvalid) x = rstd_q != nullptr ? scale16<T>(qreg[i], qs[i]) : qreg[i];
    st16(Qs + row * LDK + cc * VEC, x);
  }
  if (tid < 64) Eg[tid] = scale * __expf(gval);
  IdentityFrag<T> id;
  id.init();
#pragma unroll
  for (int t = 0; t < 3; ++t) Af[t].pack(mfma_transpose<T>(Af[t], id));   // now (lane <-> row i, registers <-> column j)
  __syncthreads();

  auto out_tile = [&](int ri) {
    f32x16 oa = acc_zero();
#pragma unroll
    for (int kt = 0; kt < NKT; ++kt) mma32_accb<T>(oa, Qs + (32 * ri + l32) * LDK + 32 * kt, Sb[kt]);
    const f32x16 eg = rows_ld(Eg, 32 * ri);
#pragma unroll
    for (int r = 0; r < 16; ++r) oa[r] *= eg[r];
#pragma unroll
    for (int tj = 0; tj <= ri; ++tj) mma32_ff<T>(oa, Af[ri + tj], Vb[tj]);
    return oa;
  };
  if constexpr (!NORM) {
    T* og = o + (tok0 * Hv + h) * V + v0;
#pragma unroll
    for (int ri = 0; ri < 2; ++ri)
      acc_store_rows<T, false>(out_tile(ri), id, patch, og + (int64_t)32 * ri * Hv * V, (int64_t)Hv * V, nvalid - 32 * ri);
  } else {
    // the wave's 32 columns of a row are PPR 16-byte pieces on PPR neighbouring lanes; a lane holds PPL pieces per tile
    constexpr int PLD = Patch<T>::kLd, PPR = 32 / VEC, PPL = PPR / 2;
    float* ssw = reinterpret_cast<float*>(gdn_smem + SM::off_ss);
    const int cc = lane % PPR;
    Vec16<T> xs[2][PPL], gs[2][PPL];
#pragma unroll
    for (int ri = 0; ri < 2; ++ri) {
      const f32x16 oa = out_tile(ri);
      GDN_WAVE_LDS_SYNC();   // earlier readers of the patch are done
      acc_to_lds_rm(oa, id, patch, PLD, 0, 0);
      GDN_WAVE_LDS_SYNC();
#pragma unroll
      for (int i = 0; i < PPL; ++i) {
        const int rowl = (lane + 64 * i) / PPR;
        xs[ri][i] = ld16(patch + rowl * PLD + cc * VEC);
        const float ss = lane_group_sum<PPR>(piece_sumsq<T>(xs[ri][i]));
        if (cc == 0) ssw[wave * 64 + 32 * ri + rowl] = ss;
      }
    }
    // gate and weight are requested only now, when the operands of the products no longer occupy registers
    float w[VEC];
    load_weight<T, TW>(w, nm.weight + v0 + cc * VEC);
#pragma unroll
    for (int ri = 0; ri < 2; ++ri)
#pragma unroll
      for (int i = 0; i < PPL; ++i) {
        const int row = 32 * ri + (lane + 64 * i) / PPR;
        gs[ri][i] = row < nvalid ? ld16(nm.gate + ((tok0 + row) * Hv + h) * V + v0 + cc * VEC) : zero16<T>();
      }
    __syncthreads();
#pragma unroll
    for (int ri = 0; ri < 2; ++ri)
#pragma unroll
      for (int i = 0; i < PPL; ++i) {
        const int row = 32 * ri + (lane + 64 * i) / PPR;
        float ss = ssw[row] + ssw[64 + row];
        if constexpr (NW == 4) ss += ssw[128 + row] + ssw[192 + row];
        const float rstd = rsqrtf(ss * (1.f / (32 * NW)) + nm.eps);
        if (row < nvalid) {
          const int64_t at = ((tok0 + row) * Hv + h) * V + v0 + cc * VEC;
          const Vec16<T> yv = rmsnorm_gated_piece<T, TW>(xs[ri][i], gs[ri][i], w, rstd);
          __builtin_nontemporal_store(yv.raw, reinterpret_cast<u32x4*>(nm.y + at));
          if (o != nullptr) st16(o + at, xs[ri][i]);
          if (nm.rstd_opt != nullptr && wave == 0 && cc == 0) nm.rstd_opt[(tok0 + row) * Hv + h] = rstd;
        }
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

// the gated RMSNorm applied by the output kernel (null y: none); weight in fp32 or in the rule's dtype
struct FwdNorm {
  const void* gate;
  const void* weight;
  void* y;
  float* rstd;
  float eps;
  bool weight_fp32;
};

template <typename T, int DK, int BVP, int NW, int NWS, int NLS, int STAGES>
static int chunk_fwd_launch(const ChunkDims& d, const ChunkWorkspace& L, const void* q, const void* k, const void* v,
                            const float* g, const float* beta, const float* h0, const int64_t* cu, void* o, float* ht,
                            unsigned char* ws, float scale, int l2norm, bool with_backward, const FwdNorm& fn,
                            hipStream_t st) {
  const int nc = (int)d.max_chunks();
  int* chunk_offsets = reinterpret_cast<int*>(ws + L.chunk_offsets);
  const T* qq = (const T*)q;
  const T* kk = (const T*)k;
  if (cu != nullptr) GDN_LAUNCH(kKernChunkTable, st, chunk_table_kernel, dim3(1), dim3(kThreads), 0, st, cu, chunk_offsets, d.N);
  float* rstd = reinterpret_cast<float*>(ws + L.rstd);
  float* G = reinterpret_cast<float*>(ws + L.G);
  T* Ai = with_backward ? reinterpret_cast<T*>(ws + L.Ai) : nullptr;
  T* W = reinterpret_cast<T*>(ws + L.WAF);
  T* AQ = reinterpret_cast<T*>(ws + L.AQ);
  T* UF = reinterpret_cast<T*>(ws + L.UF);
  T* KTF = reinterpret_cast<T*>(ws + L.KTF);
  T* WF = with_backward ? reinterpret_cast<T*>(ws + L.WF) : nullptr;
  T* KAF = with_backward ? reinterpret_cast<T*>(ws + L.KAF) : nullptr;
  T* QTF = with_backward ? reinterpret_cast<T*>(ws + L.QTF) : nullptr;
  T* VF = reinterpret_cast<T*>(ws + L.VF);
  T* HF = reinterpret_cast<T*>(ws + L.HF);
  {
    auto kern = chunk_prep_kernel<T, DK, BVP>;
    constexpr int smem = PrepSmem<T, DK, BVP>::bytes;
    if (int e = set_lds(kern, smem)) return e;
    GDN_LAUNCH(kKernPrep, st, kern, dim3(nc, d.Hv), dim3(kThreads), smem, st, qq, kk, (const T*)v, g, beta, cu,
               (const int*)chunk_offsets, G, Ai, W, UF, AQ, KTF, WF, KAF, QTF, rstd, rstd + (int64_t)nc * 64 * d.Hqk, d.T, d.N, d.Hqk,
               d.Hv, d.V, scale, l2norm, d.strides());
  }
  {
    auto kern = chunk_state_kernel<T, DK, NWS, NLS, STAGES>;
    constexpr int smem = StateSmem<T, DK, NWS, STAGES>::bytes;
    if (int e = set_lds(kern, smem)) return e;
    GDN_LAUNCH(kKernStateFwd, st, kern, dim3(d.N * d.Hv, d.V / (32 * NWS)), dim3(64 * (NWS + NLS)), smem, st,
               (const T*)KTF, (const T*)W, (const T*)UF, (const float*)G, h0, ht, VF, HF, cu,
               (const int*)chunk_offsets, d.T, d.Hqk, d.Hv, d.V);
  }
  auto launch_out = [&](auto kern, auto nm) -> int {
    constexpr int smem = OutSmem<T, DK, NW>::bytes;
    if (int e = set_lds(kern, smem)) return e;
    GDN_LAUNCH(kKernOut, st, kern, dim3(nc, d.Hv, d.V / (32 * NW)), dim3(64 * NW), smem, st, qq,
               (const T*)AQ, (const T*)VF, (const T*)HF, (const float*)G, (T*)o, cu, (const int*)chunk_offsets, d.T, d.N, d.Hqk,
               d.Hv, d.V, scale, d.strides().q, l2norm ? (const float*)rstd : (const float*)nullptr, nm);
    return 0;
  };
  if (fn.y == nullptr) {
    if (int e = launch_out(chunk_out_kernel<T, DK, NW, false, T>, OutNorm<T, T>{})) return e;
  } else if (d.V != 32 * NW) {
    return -3;   // a workgroup of the output kernel must hold whole rows
  } else if (fn.weight_fp32) {
    if (int e = launch_out(chunk_out_kernel<T, DK, NW, true, float>,
                           OutNorm<T, float>{(const T*)fn.gate, (const float*)fn.weight, (T*)fn.y, fn.rstd, fn.eps}))
      return e;
  } else {
    if (int e = launch_out(chunk_out_kernel<T, DK, NW, true, T>,
                           OutNorm<T, T>{(const T*)fn.gate, (const T*)fn.weight, (T*)fn.y, fn.rstd, fn.eps}))
      return e;
  }
  return (int)hipGetLastError();
}

}  // namespace gdn

namespace gdn {
int device_compute_units() {
  static int cus = 0;   // one device type per process; a wrong guess only costs speed
  if (cus == 0) {
    int dev = 0, n = 0;
    if (hipGetDevice(&dev) == hipSuccess &&
        hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, dev) == hipSuccess && n > 0)
      cus = n;
    else
      cus = 256;
  }
  return cus;
}
}  // namespace gdn

extern "C" int64_t gdn_chunk_workspace_bytes(int B, int T, int N, int Hqk, int Hv, int K, int V, int dtype,
                                             int with_backward) {
  // one layout for padded and packed input: the packed chunk bound is the larger of the two
  gdn::ChunkDims d{B, T, N, Hqk, Hv, K, V, true};
  const gdn::ChunkWorkspace w = gdn::chunk_workspace_layout(d, dtype == 0 ? 4 : 2);
  return with_backward ? w.total_bytes : w.fwd_bytes;
}

namespace gdn {
static int chunk_fwd_entry(const void* q, const void* k, const void* v, int64_t q_stride, int64_t k_stride,
                           int64_t v_stride, const float* g, const float* beta, const float* initial_state,
                           const int64_t* cu_seqlens, void* o, float* final_state, void* workspace,
                           int64_t workspace_bytes, int B, int T, int N, int Hqk, int Hv, int K, int V, float scale,
                           int use_qk_l2norm, int dtype, const FwdNorm& fn, void* stream) {
  if (!q || !k || !v || !g || !beta || !workspace) return -1;
  if (fn.y == nullptr ? !o : (!fn.gate || !fn.weight)) return -1;
  ChunkDims d{B, T, N, Hqk, Hv, K, V, cu_seqlens != nullptr};
  d.ts = {q_stride, k_stride, v_stride, 0, 0, 0};
  if (int e = chunk_check_dims(d, dtype)) return e;
  if (((uintptr_t)q | (uintptr_t)k | (uintptr_t)v | (uintptr_t)o | (uintptr_t)fn.y | (uintptr_t)fn.gate |
       (uintptr_t)fn.weight) & 15)
    return -6;
  ChunkDims dl = d;
  dl.varlen = true;  // one layout for both modes (the packed bound is the larger)
  const ChunkWorkspace L = chunk_workspace_layout(dl, dtype == 0 ? 4 : 2);
  if (workspace_bytes < L.fwd_bytes) return -5;
  const bool with_bwd = workspace_bytes >= L.total_bytes;   // a workspace sized for backward also receives W^T fragments
  if ((reinterpret_cast<uintptr_t>(workspace) & 255) != 0) return -5;
  unsigned char* ws = static_cast<unsigned char*>(workspace);
  hipStream_t st = (hipStream_t)stream;
#define GDN_FWD(T_, DK_, BVP_, NW_, NWS_, NLS_, ST_)                                                                        \
  return chunk_fwd_launch<T_, DK_, BVP_, NW_, NWS_, NLS_, ST_>(d, L, q, k, v, g, beta, initial_state, cu_seqlens, o, final_state, \
                                                   ws, scale, use_qk_l2norm, with_bwd, fn, st)
  const bool wide = (V % 128 == 0);
  const bool solo = one_slab_per_workgroup(d, device_compute_units());
  if (dtype == 1) {
    if (K == 128 && wide && solo) GDN_FWD(bf16_t, 128, 128, 4, 1, 2, 2);
    if (K == 128 && wide) GDN_FWD(bf16_t, 128, 128, 4, 2, 2, 2);
    if (K == 128) GDN_FWD(bf16_t, 128, 64, 2, 2, 2, 2);
    if (K == 64 && wide) GDN_FWD(bf16_t, 64, 128, 4, 2, 2, 2);
    GDN_FWD(bf16_t, 64, 64, 2, 2, 2, 2);
  } else {
    if (K == 128 && wide) GDN_FWD(float, 128, 64, 4, 4, 4, 1);
    if (K == 128) GDN_FWD(float, 128, 64, 2, 2, 2, 1);
    if (wide) GDN_FWD(float, 64, 64, 4, 4, 4, 2);
    GDN_FWD(float, 64, 64, 2, 2, 2, 2);
  }
#undef GDN_FWD
}
}  // namespace gdn

extern "C" int gdn_chunk_fwd_strided(const void* q, const void* k, const void* v, int64_t q_stride, int64_t k_stride,
                                     int64_t v_stride, const float* g, const float* beta, const float* initial_state,
                                     const int64_t* cu_seqlens, void* o, float* final_state, void* workspace,
                                     int64_t workspace_bytes, int B, int T, int N, int Hqk, int Hv, int K, int V,
                                     float scale, int use_qk_l2norm, int dtype, void* stream) {
  return gdn::chunk_fwd_entry(q, k, v, q_stride, k_stride, v_stride, g, beta, initial_state, cu_seqlens, o, final_state,
                              workspace, workspace_bytes, B, T, N, Hqk, Hv, K, V, scale, use_qk_l2norm, dtype,
                              gdn::FwdNorm{}, stream);
}

extern "C" int gdn_chunk_fwd_norm_strided(const void* q, const void* k, const void* v, int64_t q_stride,
                                          int64_t k_stride, int64_t v_stride, const float* g, const float* beta,
                                          const float* initial_state, const int64_t* cu_seqlens, const void* gate,
                                          const void* norm_weight, void* o, void* y, float* rstd, float* final_state,
                                          void* workspace, int64_t workspace_bytes, int B, int T, int N, int Hqk,
                                          int Hv, int K, int V, float scale, float eps, int use_qk_l2norm, int dtype,
                                          int weight_dtype, void* stream) {
  if (!y) return -1;
  if (weight_dtype != 0 && weight_dtype != dtype) return -4;
  if (V != 64 && V != 128) return -3;
  return gdn::chunk_fwd_entry(q, k, v, q_stride, k_stride, v_stride, g, beta, initial_state, cu_seqlens, o, final_state,
                              workspace, workspace_bytes, B, T, N, Hqk, Hv, K, V, scale, use_qk_l2norm, dtype,
                              gdn::FwdNorm{gate, norm_weight, y, rstd, eps, weight_dtype == 0}, stream);
}

extern "C" int gdn_chunk_fwd(const void* q, const void* k, const void* v, const float* g, const float* beta,
                             const float* initial_state, const int64_t* cu_seqlens, void* o, float* final_state,
                             void* workspace, int64_t workspace_bytes, int B, int T, int N, int Hqk, int Hv, int K,
                             int V, float scale, int use_qk_l2norm, int dtype, void* stream) {
  return gdn_chunk_fwd_strided(q, k, v, 0, 0, 0, g, beta, initial_state, cu_seqlens, o, final_state, workspace,
                               workspace_bytes, B, T, N, Hqk, Hv, K, V, scale, use_qk_l2norm, dtype, stream);
}
