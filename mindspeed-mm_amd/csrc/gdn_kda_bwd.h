// KDA (Kimi delta attention) backward.  Included at the end of gdn_chunk_bwd.hip: the reverse recurrence and the sums
// over V of the chunk-local pass are that file's kernels in their KDA modes (chunk_state_bwd_kernel,
// chunk_bwd_local_kernel, which also writes dv); this file turns those sums into the gradients of q, k, the gate input
// and beta, which is where the decay per key channel changes the algebra.  The reference differentiates its pure
// PyTorch statement with autograd (mindspeed_mm/fsdp/ops/kda/chunk_kda_naive.py:106-221); the equations below are the
// hand-derived backward of that statement.
//
// Forward, per chunk (G cumulative log decay [64,K], b = transformed beta, S the state before the chunk):
//   Kp = k . e^{G}   K1 = -b Kp   K2 = k . e^{G_last-G}   Qb = scale q . e^{G}
//   L_ij = b_i sum_d k_id k_jd e^{G_id-G_jd} (i>j)   Tm = (I+L)^-1   Aq_ij = scale sum_d q_id k_jd e^{G_id-G_jd} (i>=j)
//   z = b v + K1 S    V' = Tm z    O = Qb S + Aq V'    S' = e^{G_last} . S + K2^T V'
// What arrives (sums over V, rounded to T; dD in fp32): dQb = dO S^T, dK2 = V' dS'^T, P = dV' S^T, dAq = tril(dO V'^T), a2 = dV' V^T,
// dD = sum_v dS' . S.  Then
//   dTm = stril(b_j (a2 - P Kp^T))    dL = -stril(Tm^T dTm Tm^T)    dK1 = Tm^T P    <R_t, v_t> = sum_i Tm_it a2_it
//   U_i  = sum_{j<i}  dL_ij        k_j . e^{G_i-G_j}          Uq_i = sum_{j<=i} scale dAq_ij k_j . e^{G_i-G_j}
//   W_j  = sum_{i>=j} (dL_ij b_i k_i + scale dAq_ij q_i) . e^{G_i-G_j}
//   dq^ = scale e^{G} . dQb + Uq
//   dk^ = -b e^{G} . dK1 + e^{G_last-G} . dK2 + b U + W
//   dG  = q^ . dq^ + k^ . (-b e^{G} . dK1 + b U - e^{G_last-G} . dK2 - W)         per token and channel
//   dG_last = sum_i k^_i . e^{G_last-G_i} . dK2_i + dD . e^{G_last}               per channel
//   db_i = <R_i, v_i> + sum_d k^_id (U_id - e^{G_id} dK1_id)
//   dg_t = sum_{i>=t} dG_i + dG_last, then back through the gate, the l2 norm and the sigmoid of beta.
// The decay-weighted sums over a chunk use the recursive halving of the forward pass: a pair i > j belongs to one block
// of one level (64, 32, ..., 2 tokens), in which i lies in the second half and j in the first, and there
// e^{G_i-G_j} = e^{G_i-G_m} e^{G_m-G_j} with m the middle of the block, both factors at most 1.  For the levels of 8
// to 64 tokens the coefficients outside that level's pairs are masked away, the partner rows are rescaled in
// registers straight into the B-operand layout, the products run on the matrix cores and the rows of the result are
// scaled by their own factor.  The levels of 2 and 4 tokens stay inside a lane: a lane has one key channel and, per
// accumulator group, four consecutive tokens, which are one block of 4.  (For fp32 operands every pair is summed term
// by term in fp32 instead.)
// What the chunk-local kernel leaves (the workspace's DUMP): P as rows, dQb, dK2, dAq and a2 as 32x32 tiles in
// fragment order, which is how both kernels hold them in registers.
#pragma once
#include "gdn_kda_common.h"

namespace gdn {

template <typename T, int DK> struct KdaBwdSmem {
  static constexpr int LDK = lds_ld<T>(DK), LDG = DK + 4, L64 = lds_ld<T>(64);
  static constexpr bool FULL = sizeof(T) == 4;   // no rescaled images: every pair term by term
  static constexpr int tile = 64 * LDK * (int)sizeof(T), gmat = 64 * LDG * 4, mat = 64 * L64 * (int)sizeof(T);
  static constexpr int off_ks = 0;                   // k^ rows
  static constexpr int off_qs = off_ks + tile;       // P as T; FULL: then q^ rows
  static constexpr int off_gs = off_qs + tile;       // first Kp as T (64 rows), then G rows (fp32)
  static constexpr int off_m1 = off_gs + gmat;       // dTm, then dL; later, with the next one, the store patches
  static constexpr int off_m2 = off_m1 + mat;        // X = Tm^T dTm, then scale dAq
  static constexpr int off_tm = off_m2 + mat;        // Tm row-major
  static constexpr int off_m2t = off_tm + mat;       // scale dAq transposed (not FULL)
  // not FULL: q^ rows and dL transposed get places of their own, so that P and Tm live until dK1 = Tm^T P is formed
  // where it is used, after the decay-weighted sums, instead of occupying registers through them
  static constexpr int off_q2 = off_m2t + (FULL ? 0 : mat);
  static constexpr int off_m1t = off_q2 + (FULL ? 0 : tile);
  // not FULL: which entries of a coefficient fragment belong to a level's pairs: [5 levels][2 halves of the 32 columns]
  // [row = earlier | later token][64 lanes] masks of 16 bytes (only the levels of 8, 16 and 32 tokens are filled and
  // used).  They depend on nothing but the lane.
  static constexpr int off_keep = off_m1t + (FULL ? 0 : mat);
  static constexpr int off_row = off_keep + (FULL ? 0 : 5 * 2 * 2 * 64 * 16);
  // beta, 1/|q|, 1/|k| [64 each]; row sums <q^,dq^>, <k^,dk^>, db, <R,v> [256 each]; per-wave scalars [8]; what the
  // two waves of a channel block exchange: parts of dG_last and d(dt_bias) [8][32 each], sum of dG over tokens 32.. [4][32]
  // ... and the diagonal of scale dAq [64]
  static constexpr int bytes = off_row + (3 * 64 + 4 * 256 + 8 + 2 * 256 + 128 + 64) * 4;
  static_assert(tile <= gmat, "Kp fits where G will be");
  static_assert(8 * Patch<T>::kElems * (int)sizeof(T) <= 3 * mat, "store patches fit");
  static_assert(bytes <= 160 * 1024, "one CU's LDS");
};

// Eight waves, two per SIMD: the kernel is a chain of short dependent steps (LDS reads, exponentials, small matrix
// products), and a second wave on the SIMD fills the waits of the first.  Waves 0..3 each own a 32x32 tile of the 64x64
// matrices of phases A1..A4; in phase B wave w owns key channels 32 (w >> 1).. and tokens 32 (w & 1).. of the chunk.
constexpr int kFinThreads = 512;

// rowacc[i0 + i] += sum_j x[i][j] for the 32 rows of an accumulator tile (see rows_add; the caller picks the slot)
__device__ __forceinline__ void rows_add_at(const f32x16& x, float* rowacc, int i0) {
  float s = rows16_partial(x);
  s += __shfl_xor(s, 16);
  const int lane = threadIdx.x & 63;
  if ((lane & 16) == 0) rowacc[i0 + acc_row(lane & 15)] += s;
}

template <typename T, int DK>
__global__ __launch_bounds__(kFinThreads) void kda_bwd_finish_kernel(
    const T* __restrict__ q, const T* __restrict__ k, const void* __restrict__ g, const float* __restrict__ A_log,
    const float* __restrict__ dt_bias, const float* __restrict__ bhat,
    const T* __restrict__ TMR, const T* __restrict__ dumps, const float* __restrict__ dd, const int64_t* __restrict__ cu,
    const int* __restrict__ chunk_offsets, T* __restrict__ dq, T* __restrict__ dk, void* __restrict__ dg,
    void* __restrict__ dbeta, float* __restrict__ part, int T_len, int N, int H, float scale, KdaFlags fl) {
  using SM = KdaBwdSmem<T, DK>;
  constexpr int LDK = SM::LDK, LDG = SM::LDG, L64 = SM::L64, VEC = Elem<T>::kVec, CPR = DK / VEC, NKT = DK / 32;
  constexpr bool FULL = SM::FULL;
  T* Ks = reinterpret_cast<T*>(gdn_smem + SM::off_ks);
  T* Pt = reinterpret_cast<T*>(gdn_smem + SM::off_qs);
  T* Qs = FULL ? Pt : reinterpret_cast<T*>(gdn_smem + SM::off_q2);
  float* Gs = reinterpret_cast<float*>(gdn_smem + SM::off_gs);
  T* Kp = reinterpret_cast<T*>(gdn_smem + SM::off_gs);
  T* TmT = reinterpret_cast<T*>(gdn_smem + SM::off_tm);
  T* M1 = reinterpret_cast<T*>(gdn_smem + SM::off_m1);
  T* M2 = reinterpret_cast<T*>(gdn_smem + SM::off_m2);
  T* M1t = reinterpret_cast<T*>(gdn_smem + SM::off_m1t);
  T* M2t = reinterpret_cast<T*>(gdn_smem + SM::off_m2t);
  float* bs = reinterpret_cast<float*>(gdn_smem + SM::off_row);
  float* rsq = bs + 64;
  float* rsk = rsq + 64;
  float* rq = rsk + 64;     // row sums, a slot of 64 rows per block of 32 key channels (rows_add_at / rows_ld4)
  float* rk = rq + 256;
  float* rb = rk + 256;
  float* rv = rb + 256;     // <R_t, v_t>, a slot per tile wave
  float* wsum = rv + 256;   // [8]   per wave: its part of dA_log
  float* xgl = wsum + 8;    // [8][32] per wave and channel: its part of dG_last
  float* xdt = xgl + 256;   // [8][32] per wave and channel: its part of d(dt_bias)
  float* xblk = xdt + 256;  // [4][32] per channel: sum of dG over tokens 32..63
  float* dgq = xblk + 128;  // [64] scale dAq_ii: the pair i = j of the decay-weighted sums

  const SeqInfo s = locate_chunk(blockIdx.x, cu, chunk_offsets, N, T_len);
  if (s.nvalid <= 0) return;
  const int tid = threadIdx.x, lane = tid & 63, l32 = lane & 31;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);   // wave-uniform: branches and offsets from it are scalar
  const int h = blockIdx.y, nvalid = s.nvalid;
  const int64_t tok0 = s.bos + (int64_t)s.chunk * kChunk, hk = (int64_t)H * DK;
  const int64_t ch = (int64_t)blockIdx.x * H + h;
  const int ti = (wave >> 1) & 1, tj = wave & 1;
  const bool tile_wave = wave < 4, lower = tile_wave && tj <= ti;
  const int cj = wave >> 1, ri = wave & 1;
  const bool has_k = cj < NKT;
  const T* dump = dumps + ch * (3 * 64 * DK + 2 * 64 * 64);
  const T* dQb = dump, *dK2 = dump + 64 * DK, *Pm = dump + 2 * 64 * DK;
  const T* dAq = dump + 3 * 64 * DK, *a2m = dAq + 64 * 64;
  const float* dD = dd + ch * DK;

  // ---- phase A0: G from the gate input; k^ rows; P and Tm as operands; beta.  The tile waves request their tiles of
  //      a2 and dAq now ----
  // This thread's pieces of the 64 x DK operands: VEC consecutive channels of a row each.  The gate input goes first
  // (loads arrive in the order of their requests): the cumulative decay is rebuilt from it, with the forward pass's own
  // operations, while the other operands are on their way.  (As bits, one branch around the whole round of requests.)
  constexpr int NIT = 64 * CPR / kFinThreads, C64 = 64 / VEC, NTM = 64 * C64 / kFinThreads;
  static_assert(64 * CPR % kFinThreads == 0 && 64 * C64 % kFinThreads == 0 && VEC % 4 == 0, "whole rounds of 16-byte pieces");
  static_assert(kFinThreads % CPR == 0, "a thread's pieces share their channels");
  const bool g32 = sizeof(T) == 4 || fl.g_f32;
  u32x4 gw[NIT][VEC / 4];
  f32x4 bv[VEC / 4];
  if (g32) {
#pragma unroll
    for (int it = 0; it < NIT; ++it) {
      const int c = tid + it * kFinThreads, row = imin(c / CPR, nvalid - 1);
#pragma unroll
      for (int e = 0; e < VEC / 4; ++e)
        gw[it][e] = *reinterpret_cast<const u32x4*>(reinterpret_cast<const uint32_t*>(g) + (tok0 + row) * hk + h * DK +
                                                    (c % CPR) * VEC + 4 * e);
    }
  } else {
    if constexpr (sizeof(T) == 2) {   // VEC = 8 two-byte values: one 16-byte piece
#pragma unroll
      for (int it = 0; it < NIT; ++it) {
        const int c = tid + it * kFinThreads, row = imin(c / CPR, nvalid - 1);
        gw[it][0] = *reinterpret_cast<const u32x4*>(reinterpret_cast<const uint16_t*>(g) + (tok0 + row) * hk + h * DK +
                                                    (c % CPR) * VEC);
      }
    }
  }
  {
    // without a branch around the request (the compiler would wait for it at the join): with no bias the pieces come
    // from a place that is always there and are dropped
    const bool has_bias = fl.use_gate && dt_bias != nullptr;
    const float* bp = (has_bias ? dt_bias + h * DK : dD) + (tid % CPR) * VEC;
#pragma unroll
    for (int e = 0; e < VEC / 4; ++e) {
      const f32x4 x = *reinterpret_cast<const f32x4*>(bp + 4 * e);
      bv[e] = has_bias ? x : f32x4{0.f, 0.f, 0.f, 0.f};
    }
  }
  TileQK<T, DK, kFinThreads> kt;   // moved by every thread
  TileQK<T, DK> qt;                // moved by kThreads threads, see below
  tile_qk_request<T, DK>(kt, k + tok0 * hk + h * DK, hk, nvalid, tid);
  AccB<T> a2f, daf;
  u32x4* keepT = reinterpret_cast<u32x4*>(gdn_smem + SM::off_keep);
  if constexpr (!FULL) {
    // Which of 8 consecutive entries of a coefficient row belong to a level's pairs, as a mask over the fragment (two
    // 16-bit entries per register).  a: the row's token within the 32-token block, b: that of a column.  second: the
    // row index is the later token i (kept when i is in the second half of its block of 2^lg tokens and the column j
    // in the first half of the same block), else the row index is the earlier token j.
    // In terms of bits: i and j share the block and sit in different halves of it when (i ^ j) >> (lg - 1) == 1, and
    // the row's own half is bit lg - 1 of its index.  (Plain bit arithmetic: written with comparisons of the halves
    // the compiler turns every entry into a branch.)
    for (int idx = 2 * 2 * 2 * 64 + tid; idx < 5 * 2 * 2 * 64; idx += kFinThreads) {   // levels of 8, 16, 32 tokens
      const int ln = idx & 63, second = (idx >> 6) & 1, kg = (idx >> 7) & 1, sh = idx >> 8;   // sh = lg - 1
      const int a = ln & 31, b0 = 16 * kg + 8 * (ln >> 5);
      const uint32_t rok = ((a >> sh) & 1) == second ? 0xffffffffu : 0u;
      u32x4 w;
#pragma unroll
      for (int e = 0; e < 4; ++e) {
        const int b1 = b0 + 2 * e, b2 = b1 + 1;
        const uint32_t k1 = ((a ^ b1) >> sh) == 1 ? 0xffffu : 0u;
        const uint32_t k2 = ((a ^ b2) >> sh) == 1 ? 0xffff0000u : 0u;
        w[e] = (k1 | k2) & rok;
      }
      keepT[idx] = w;
    }
  }
  // this thread's pieces of P and Tm, all requested before the first wait
  f32x4 gk[NIT][VEC / 4];
  Vec16<T> pf[NIT], tmv[NTM];
#pragma unroll
  for (int it = 0; it < NIT; ++it) {
    const int c = tid + it * kFinThreads;
    pf[it] = ld16(Pm + (c / CPR) * DK + (c % CPR) * VEC);
  }
#pragma unroll
  for (int it = 0; it < NTM; ++it) {
    const int c = tid + it * kFinThreads;
    tmv[it] = ld16(TMR + ch * 4096 + (c / C64) * 64 + (c % C64) * VEC);
  }
  // beta: requested by every wave alike and with the early group (loads arrive in the order of their requests: the
  // store of the row vectors below then waits for P and Tm, not for the requests made behind the gate)
  const float bh = bhat[(tok0 + imin(lane, nvalid - 1)) * H + h];
  // G: the gate's log decay of every token and channel (0 on the rows past the end) into the place Kp will take,
  // summed down the tokens there, and back into this thread's registers until Kp is consumed
  {
    const float a = fl.use_gate ? __expf(A_log[h]) : 0.f;
    const float au = a * KdaDecay<T>::kUnit, lbu = fl.lower_bound * KdaDecay<T>::kUnit;
    auto gate_rows = [&](auto mode) {   // one copy of the loop per mode, as in the forward pass
      constexpr int MODE = decltype(mode)::value;
#pragma unroll
      for (int it = 0; it < NIT; ++it) {
        const int c = tid + it * kFinThreads, row = c / CPR, cc = c % CPR;
#pragma unroll
        for (int e4 = 0; e4 < VEC / 4; ++e4) {
          f32x4 y;
#pragma unroll
          for (int e = 0; e < 4; ++e) {
            const int idx = 4 * e4 + e;
            const float x = __uint_as_float(g32 ? gw[it][e4][e] : (gw[it][0][(idx >> 1) & 3] >> (16 * (idx & 1))) << 16);
            y[e] = row < nvalid ? kda_gate<T, MODE>(x, bv[e4][e], a, au, lbu) : 0.f;
          }
          *reinterpret_cast<f32x4*>(Gs + row * LDG + cc * VEC + 4 * e4) = y;
        }
      }
    };
    if (!fl.use_gate) gate_rows(IntConst<0>());
    else if (!fl.has_lower_bound) gate_rows(IntConst<1>());
    else gate_rows(IntConst<2>());
    GDN_LDS_BARRIER();
  }
  // a2 and dAq arrive as tiles in fragment order: a tile wave takes its own.  These requests come behind the gate: none
  // of them is needed before phase A1, and requested ahead of the gate their branches made every wave wait for all of
  // its earlier requests first.
  // q^ rows: in the 16-bit kernel they have a place of their own, and the waves that own no tile of the 64x64 phases
  // normalise them during those phases.
  // Every wave makes the same number of requests here (K = 128: four): the waits further down can then leave exactly
  // these in flight.  The wave of the tile above the diagonal, which nobody wrote, asks for tile (0,0) again (cached)
  // and drops it.
  constexpr bool Q_BY_OTHERS = !FULL;
  const bool q_wave = Q_BY_OTHERS ? !tile_wave : tile_wave;
  const int tile_at = lower ? (2 * ti + tj) * 1024 : 0;
  constexpr bool SAME_REQUESTS = Q_BY_OTHERS && TileQK<T, DK>::PT == 2 * AccB<T>::kG;
  if constexpr (SAME_REQUESTS) {
    // one set of requests, the choice made on the addresses (a branch with two arms does not survive the compiler as
    // such, and behind two separate branches it assumes the fewest requests in flight)
    const int t = tid & (kThreads - 1);
#pragma unroll
    for (int i = 0; i < TileQK<T, DK>::PT; ++i) {
      const int c = t + i * kThreads, row = imin(c / CPR, nvalid - 1), cc = c % CPR;
      const T* qa = q + (tok0 + row) * hk + h * DK + cc * VEC;
      const T* ta = (i < AccB<T>::kG ? a2m : dAq) + tile_at + frag_slot<T>(i % AccB<T>::kG, lane) * AccB<T>::kVecElems;
      qt.x[i] = ld16(tile_wave ? ta : qa);
    }
#pragma unroll
    for (int g = 0; g < AccB<T>::kG; ++g) { a2f.f[g] = qt.x[g].raw; daf.f[g] = qt.x[AccB<T>::kG + g].raw; }
  } else if constexpr (Q_BY_OTHERS) {
    if (tile_wave) {
      a2f.load(a2m + tile_at);
      daf.load(dAq + tile_at);
    } else {
      tile_qk_request<T, DK>(qt, q + tok0 * hk + h * DK, hk, nvalid, tid & (kThreads - 1));
    }
  } else {
    if (tile_wave) {
      a2f.load(a2m + tile_at);
      daf.load(dAq + tile_at);
      tile_qk_request<T, DK>(qt, q + tok0 * hk + h * DK, hk, nvalid, tid & (kThreads - 1));
    }
  }
  {
    constexpr int PARTS = kThreads / DK;   // the forward pass's split of the chunk, for the same rounding
    float* tot = xgl;                      // [PARTS][DK]: free until phase B
    static_assert(PARTS * DK <= 256, "the totals fit the vector they borrow");
    if (tid < kThreads) kda_cumsum_part<DK, LDG, PARTS>(Gs, tot, tid);
    GDN_LDS_BARRIER();
#pragma unroll
    for (int it = 0; it < NIT; ++it) {
      const int c = tid + it * kFinThreads, row = c / CPR, cc = c % CPR, part = row / (64 / PARTS);
#pragma unroll
      for (int e4 = 0; e4 < VEC / 4; ++e4) {
        gk[it][e4] = *reinterpret_cast<const f32x4*>(Gs + row * LDG + cc * VEC + 4 * e4);
#pragma unroll
        for (int e = 0; e < 4; ++e) gk[it][e4][e] += kda_cumsum_before<DK, PARTS>(tot, part, cc * VEC + 4 * e4 + e);
      }
    }
  }
  if (tid < 64) {
    bs[tid] = tid < nvalid ? bh : 0.f;
    rsq[tid] = 1.f;
    rsk[tid] = 1.f;
  }
  if (tid < 256) { rq[tid] = 0.f; rk[tid] = 0.f; rb[tid] = 0.f; rv[tid] = 0.f; }
#pragma unroll
  for (int it = 0; it < NIT; ++it) {
    const int c = tid + it * kFinThreads;
    st16(Pt + (c / CPR) * LDK + (c % CPR) * VEC, pf[it]);
  }
#pragma unroll
  for (int it = 0; it < NTM; ++it) {
    const int c = tid + it * kFinThreads;
    st16(TmT + (c / C64) * L64 + (c % C64) * VEC, tmv[it]);
  }
  GDN_LDS_BARRIER();   // the row vectors are initialised before the norm below writes 1/|k| over its entries; G is in registers
  tile_qk_finish<T, DK>(kt, Ks, LDK, nvalid, tid, fl.l2norm != 0, nullptr, 0, rsk, 1);
  GDN_LDS_BARRIER();
#pragma unroll
  for (int it = 0; it < NIT; ++it) {   // Kp = k^ . e^{G}
    const int c = tid + it * kFinThreads, row = c / CPR, cc = c % CPR;
    float f[VEC];
    unpack16<T>(ld16(Ks + row * LDK + cc * VEC), f);
#pragma unroll
    for (int e = 0; e < VEC; ++e) f[e] *= KdaDecay<T>::exp(gk[it][e / 4][e % 4]);
    st16(Kp + row * LDK + cc * VEC, pack16<T>(f));
  }
  GDN_LDS_BARRIER();

  if (Q_BY_OTHERS && q_wave) tile_qk_finish<T, DK>(qt, Qs, LDK, nvalid, tid & (kThreads - 1), fl.l2norm != 0, nullptr, 0, rsq, 1);
  // ---- phase A1: dTm = stril(b_j (a2 - P Kp^T)), one 32x32 tile per tile wave; <R_t, v_t> from Tm and a2 ----
  f32x16 a2t = acc_zero(), dat = acc_zero();
  if (lower) a2t = a2f.unpack();
  if (tile_wave) {
    f32x16 x = acc_zero();
    if (lower) mma32<T, DK, true, true>(x, Pt + 32 * ti * LDK, LDK, Kp + 32 * tj * LDK, LDK);
    const int j = 32 * tj + l32;
    const float bj = bs[j];
    float sv = 0.f;
    f32x16 tmt;   // this wave's tile of Tm as the accumulator holds a tile
    if constexpr (FULL) {
#pragma unroll
      for (int r = 0; r < 16; ++r) tmt[r] = TmT[(32 * ti + acc_row(r)) * L64 + j];
    } else {
      AccB<T> t;
      t.load_cols(TmT + 32 * ti * L64 + 32 * tj, L64);
      tmt = t.unpack();
    }
#pragma unroll
    for (int r = 0; r < 16; ++r) {
      const int i = 32 * ti + acc_row(r);
      const float a2v = a2t[r];
      sv += a2v * tmt[r];
      M1[i * L64 + j] = Elem<T>::from_f(i > j ? bj * (a2v - x[r]) : 0.f);
    }
    sv += __shfl_xor(sv, 32);
    if (lane < 32) rv[wave * 64 + 32 * tj + lane] = sv;
  }
  GDN_LDS_BARRIER();
  // ---- phase A2: X = Tm^T dTm (the tiles dL needs: a >= the column block) ----
  if (tile_wave) {
    f32x16 x = acc_zero();
    if (lower) mma32<T, 64, false, false>(x, TmT + 32 * ti, L64, M1 + 32 * tj, L64);
#pragma unroll
    for (int r = 0; r < 16; ++r) M2[(32 * ti + acc_row(r)) * L64 + 32 * tj + l32] = Elem<T>::from_f(x[r]);
  }
  GDN_LDS_BARRIER();
  // ---- phase A3: dL = -stril(X Tm^T); dK1 = Tm^T P for this wave's tokens and key channels; scale dAq ----
  f32x16 dK1 = acc_zero(), dl = acc_zero(), sa;
  if (lower) mma32<T, 64, true, true>(dl, M2 + 32 * ti * L64, L64, TmT + 32 * tj * L64, L64);
  if (FULL && has_k) mma32<T, 64, false, false>(dK1, TmT + 32 * ri, L64, Pt + 32 * cj, LDK);
  if (lower) dat = daf.unpack();
#pragma unroll
  for (int r = 0; r < 16; ++r) {
    const int i = 32 * ti + acc_row(r), j = 32 * tj + l32;
    dl[r] = i > j ? -dl[r] : 0.f;
    sa[r] = i >= j ? scale * dat[r] : 0.f;
  }
  GDN_LDS_BARRIER();   // dTm, X, Kp are consumed (FULL: P too)
  // ---- phase A4: the coefficient matrices in place of dTm and X; G in place of Kp; q^ rows (FULL: in place of P) ----
  if (tile_wave) {
    // the transposed dL carries the beta of its later token (its row in dL): the sum over i of dL_ij b_i k_i f_i then
    // takes the same rescaled rows k_i f_i as the sum over j
    const f32x16 bi = rows_ld(bs, 32 * ti);
#pragma unroll
    for (int r = 0; r < 16; ++r) {
      const int at = (32 * ti + acc_row(r)) * L64 + 32 * tj + l32;
      M1[at] = Elem<T>::from_f(dl[r]);
      M2[at] = Elem<T>::from_f(sa[r]);
      if constexpr (!FULL) {
        if (ti == tj && acc_row(r) == l32) dgq[32 * ti + l32] = Elem<T>::to_f(Elem<T>::from_f(sa[r]));
      }
    }
    if constexpr (!FULL) {   // the transposed copies: a lane's four consecutive rows of a group are four consecutive columns there
#pragma unroll
      for (int qd = 0; qd < 4; ++qd) {
        const int att = (32 * tj + l32) * L64 + 32 * ti + acc_row(4 * qd);
        u32x2 w1, w2;
#pragma unroll
        for (int m = 0; m < 2; ++m) {
          const int r = 4 * qd + 2 * m;
          w1[m] = f32x2_to_bf16x2(dl[r] * bi[r], dl[r + 1] * bi[r + 1]);
          w2[m] = f32x2_to_bf16x2(sa[r], sa[r + 1]);
        }
        *reinterpret_cast<u32x2*>(M1t + att) = w1;
        *reinterpret_cast<u32x2*>(M2t + att) = w2;
      }
    }
    if constexpr (!Q_BY_OTHERS) tile_qk_finish<T, DK>(qt, Qs, LDK, nvalid, tid, fl.l2norm != 0, nullptr, 0, rsq, 1);
  }
#pragma unroll
  for (int it = 0; it < NIT; ++it) {
    const int c = tid + it * kFinThreads;
#pragma unroll
    for (int e = 0; e < VEC / 4; ++e)
      *reinterpret_cast<f32x4*>(Gs + (c / CPR) * LDG + (c % CPR) * VEC + 4 * e) = gk[it][e];
  }
  GDN_LDS_BARRIER();

  // ---- phase B: the decay-weighted sums.  A lane has one key channel and the 16 rows of its accumulator registers
  //      in the wave's 32-token block ----
  const int d = 32 * cj + l32;
  float Gi[16], U[16], Uq[16], W[16];
  AccB<T> lqf, lkf;   // the sums over V of this lane's rows (dQb, dK2) for phase B3
  if (has_k) {
#pragma unroll
    for (int r = 0; r < 16; ++r) {
      Gi[r] = Gs[(32 * ri + acc_row(r)) * LDG + d];
      U[r] = 0.f; Uq[r] = 0.f; W[r] = 0.f;
    }
  }
  if constexpr (!FULL) {
    if (has_k) {
      const int half = lane >> 5;
      {
        // The partner rows this lane supplies as B operand, channel d, are tokens 32 ri + 16 kg + 8 half + e.
        {   // the pair i = j: no decay (dL has no diagonal).  This lane's rows of k^ and q^, channel d: four transposing
            // reads per tile instead of a two-byte read per row
          AccB<T> t;
          t.load_cols(Ks + 32 * ri * LDK + 32 * cj, LDK);
          const f32x16 kd = t.unpack();
          t.load_cols(Qs + 32 * ri * LDK + 32 * cj, LDK);
          const f32x16 qd = t.unpack();
          const f32x16 c = rows_ld(dgq, 32 * ri);
#pragma unroll
          for (int r = 0; r < 16; ++r) {
            Uq[r] += c[r] * kd[r];
            W[r] += c[r] * qd[r];
          }
          // The levels of 2 and 4 tokens inside the lane: the four rows of an accumulator group, tokens t0 .. t0 + 3, are
          // one block of 4, and every pair of these two levels has both of its rows there.  Level 2: pairs (1,0), (3,2),
          // reference row = the later token; level 4: i in {2,3}, j in {0,1}, reference row 2.  Coefficients: rows 1..3
          // of the block's 4x4 diagonal piece of dL and of scale dAq, 8 bytes each, the same for every lane of a
          // half-wave.  One exponential per pair member instead of one per row and level, and no matrix products.
          const f32x16 bo = rows_ld(bs, 32 * ri);
#pragma unroll
          for (int g4 = 0; g4 < 4; ++g4) {
            const int t0 = 32 * ri + 8 * g4 + 4 * half, r0 = 4 * g4;
            f32x4 cl[3], ca[3];
#pragma unroll
            for (int m = 1; m < 4; ++m) {
              const u32x2 wl = *reinterpret_cast<const u32x2*>(M1 + (t0 + m) * L64 + t0);
              const u32x2 wa = *reinterpret_cast<const u32x2*>(M2 + (t0 + m) * L64 + t0);
              cl[m - 1] = f32x4{__uint_as_float(wl[0] << 16), __uint_as_float(wl[0] & 0xffff0000u),
                                __uint_as_float(wl[1] << 16), __uint_as_float(wl[1] & 0xffff0000u)};
              ca[m - 1] = f32x4{__uint_as_float(wa[0] << 16), __uint_as_float(wa[0] & 0xffff0000u),
                                __uint_as_float(wa[1] << 16), __uint_as_float(wa[1] & 0xffff0000u)};
            }
            float bk[4];
#pragma unroll
            for (int m = 0; m < 4; ++m) bk[m] = bo[r0 + m] * kd[r0 + m];
            // rows t0 + i > t0 + j of the block, decay factor w = e^{G_i - G_j}
#define GDN_KDA_PAIR(i, j, w)                                                              \
            do {                                                                           \
              const float dl_ = cl[(i) - 1][j], sa_ = ca[(i) - 1][j], w_ = (w), kjw_ = kd[r0 + (j)] * w_; \
              U[r0 + (i)] += dl_ * kjw_;                                                   \
              Uq[r0 + (i)] += sa_ * kjw_;                                                  \
              W[r0 + (j)] += (dl_ * bk[i] + sa_ * qd[r0 + (i)]) * w_;                      \
            } while (0)
            GDN_KDA_PAIR(1, 0, KdaDecay<T>::exp(Gi[r0 + 1] - Gi[r0]));
            const float f3 = KdaDecay<T>::exp(Gi[r0 + 3] - Gi[r0 + 2]);
            GDN_KDA_PAIR(3, 2, f3);
            const float g0 = KdaDecay<T>::exp(Gi[r0 + 2] - Gi[r0]), g1 = KdaDecay<T>::exp(Gi[r0 + 2] - Gi[r0 + 1]);
            GDN_KDA_PAIR(2, 0, g0);
            GDN_KDA_PAIR(2, 1, g1);
            GDN_KDA_PAIR(3, 0, f3 * g0);
            GDN_KDA_PAIR(3, 1, f3 * g1);
#undef GDN_KDA_PAIR
          }
        }
        // The levels of 8, 16 and 32 tokens on the matrix cores.  A block is at least as long as the 8 partner rows a
        // half-wave holds per group and as the 8 rows that two of its accumulator groups span, so those rows share their
        // reference row: one read of it instead of eight (or four).
        // the partner rows of k^ and q^, channel d, as they lie (16 kg + 8 half + e): four transposing reads per tile,
        // packed pairs held through the levels
        AccB<T> kpart, qpart;
        kpart.load_cols_consecutive(Ks + 32 * ri * LDK + 32 * cj, LDK);
        qpart.load_cols_consecutive(Qs + 32 * ri * LDK + 32 * cj, LDK);
        float gpart[2][8];   // and their cumulative decays
#pragma unroll
        for (int kg = 0; kg < 2; ++kg)
#pragma unroll
          for (int e = 0; e < 8; ++e) gpart[kg][e] = Gs[(32 * ri + 16 * kg + 8 * half + e) * LDG + d];
        auto level = [&](int lg, auto wide_c) {
          constexpr bool WIDE = decltype(wide_c)::value != 0;
          const int n2 = (1 << lg) >> 1;
          asm volatile("" ::: "memory");   // the reads of a level stay inside it
          // The reference row of a token is the middle of its block of 2^lg tokens.  For the lane's 8 partner rows of a
          // group (and for the rows of its accumulator registers) it is a row that depends on the lane only through the
          // half-wave, and that only while the block is no larger than the group of rows the half-wave holds, plus an
          // offset that is the same for every lane: one addition per address instead of a shift, a mask and a product.
          const float* Gpm = Gs + (32 * ri + (lg <= 3 ? 8 * half : 0)) * LDG + d;
          const float* Gom = Gs + (32 * ri + (lg <= 2 ? 4 * half : 0)) * LDG + d;
          const u32x4* keepL = keepT + (lg - 1) * 4 * 64 + lane;
          f32x16 cu = acc_zero(), cq = acc_zero(), cw = acc_zero();
#pragma unroll
          for (int kg = 0; kg < 2; ++kg) {
            float xk[8], xq[8], kx[8], qx[8];
            { Vec16<T> v; v.raw = kpart.f[kg]; unpack16<T>(v, kx); v.raw = qpart.f[kg]; unpack16<T>(v, qx); }
            const float gmid = WIDE ? Gpm[((((16 * kg) >> lg) << lg) + n2) * LDG] : 0.f;
#pragma unroll
            for (int e = 0; e < 8; ++e) {
              const int sm = (((16 * kg + e) >> lg) << lg) + n2;
              const float f = KdaDecay<T>::exp(-fabsf(gpart[kg][e] - (WIDE ? gmid : Gpm[sm * LDG])));
              xk[e] = kx[e] * f; xq[e] = qx[e] * f;
            }
            const u32x4 bK = pack16<T>(xk).raw, bQ = pack16<T>(xq).raw;
            const int row = 32 * ri + l32, col0 = 32 * ri + 16 * kg + 8 * half;
            const u32x4 keep1 = keepL[2 * kg * 64], keep2 = keepL[(2 * kg + 1) * 64];
            mfma_kgroup<T>(cu, ld16(M1 + row * L64 + col0).raw & keep2, bK);     // sum_j dL_ij (k_j f_j)
            mfma_kgroup<T>(cq, ld16(M2 + row * L64 + col0).raw & keep2, bK);
            mfma_kgroup<T>(cw, ld16(M1t + row * L64 + col0).raw & keep1, bK);   // sum_i (dL_ij b_i) (k_i f_i)
            mfma_kgroup<T>(cw, ld16(M2t + row * L64 + col0).raw & keep1, bQ);
          }
#pragma unroll
          for (int qd = 0; qd < 4; ++qd) {   // every row by its own factor
            const float gq = WIDE ? Gom[((((8 * qd) >> lg) << lg) + n2) * LDG] : 0.f;
#pragma unroll
            for (int m = 0; m < 4; ++m) {
              const int r = 4 * qd + m, sm = (((8 * qd + m) >> lg) << lg) + n2;
              const float f = KdaDecay<T>::exp(-fabsf(Gi[r] - (WIDE ? gq : Gom[sm * LDG])));
              U[r] += f * cu[r];
              Uq[r] += f * cq[r];
              W[r] += f * cw[r];
            }
          }
        };
        // (phase B3's tiles are requested here, four levels ahead of their use: 16 registers)
        lqf.load(dQb + (ri * NKT + cj) * 1024);
        lkf.load(dK2 + (ri * NKT + cj) * 1024);
#pragma unroll 1
        for (int lg = 3; lg <= 5; ++lg) level(lg, IntConst<1>());
      }
      {   // the level of the whole chunk: tokens 32..63 against tokens 0..31, m = 32, every pair kept.  The wave of the
          // later tokens takes the sums over j (U, Uq), the wave of the earlier ones the sum over i (W)
        const float g32v = Gs[32 * LDG + d];
        f32x16 c1 = acc_zero(), c2 = acc_zero();
        // the rows of the other 32-token block, channel d, as they lie (transposing reads)
        AccB<T> kpart, qpart;
        kpart.load_cols_consecutive(Ks + 32 * (1 - ri) * LDK + 32 * cj, LDK);
        if (ri == 0) qpart.load_cols_consecutive(Qs + 32 * LDK + 32 * cj, LDK);
#pragma unroll
        for (int kg = 0; kg < 2; ++kg) {
          const int c0 = 16 * kg + 8 * half;
          float kx[8];
          { Vec16<T> v; v.raw = kpart.f[kg]; unpack16<T>(v, kx); }
          if (ri == 1) {
            float xk[8];
#pragma unroll
            for (int e = 0; e < 8; ++e) {
              const int j = c0 + e;
              xk[e] = kx[e] * KdaDecay<T>::exp(-fabsf(Gs[j * LDG + d] - g32v));
            }
            const u32x4 bK = pack16<T>(xk).raw;
            mfma_kgroup<T>(c1, ld16(M1 + (32 + l32) * L64 + c0).raw, bK);
            mfma_kgroup<T>(c2, ld16(M2 + (32 + l32) * L64 + c0).raw, bK);
          } else {
            float xb[8], xq[8], qx[8];
            { Vec16<T> v; v.raw = qpart.f[kg]; unpack16<T>(v, qx); }
#pragma unroll
            for (int e = 0; e < 8; ++e) {
              const int i = 32 + c0 + e;
              const float f = KdaDecay<T>::exp(-fabsf(Gs[i * LDG + d] - g32v));
              xb[e] = kx[e] * f;
              xq[e] = qx[e] * f;
            }
            mfma_kgroup<T>(c1, ld16(M1t + l32 * L64 + 32 + c0).raw, pack16<T>(xb).raw);
            mfma_kgroup<T>(c1, ld16(M2t + l32 * L64 + 32 + c0).raw, pack16<T>(xq).raw);
          }
        }
#pragma unroll
        for (int r = 0; r < 16; ++r) {
          const float f = KdaDecay<T>::exp(-fabsf(Gi[r] - g32v));
          if (ri == 1) { U[r] += f * c1[r]; Uq[r] += f * c2[r]; }
          else W[r] += f * c1[r];
        }
      }
    }
  }
  if (FULL && has_k) {
    // rows i of this lane against the earlier rows j of the chunk
    for (int jj = 0; jj <= 32 * ri + 31; ++jj) {
      const float gj = Gs[jj * LDG + d], kj = Elem<T>::to_f(Ks[jj * LDK + d]);
#pragma unroll
      for (int qd = 0; qd < 4; ++qd) {
        if (32 * ri + 8 * qd + 7 < jj) continue;   // none of the group's rows reaches jj (same for every lane)
#pragma unroll
        for (int m = 0; m < 4; ++m) {
          const int r = 4 * qd + m, i = 32 * ri + acc_row(r);
          const float t = kj * KdaDecay<T>::exp(i >= jj ? Gi[r] - gj : 0.f);
          U[r] += Elem<T>::to_f(M1[i * L64 + jj]) * t;    // coefficients are zero where i < jj
          Uq[r] += Elem<T>::to_f(M2[i * L64 + jj]) * t;
        }
      }
    }
    // rows j of this lane against the later rows i
    for (int ii = 32 * ri; ii <= 63; ++ii) {
      const float gi = Gs[ii * LDG + d], kb = bs[ii] * Elem<T>::to_f(Ks[ii * LDK + d]), qv = Elem<T>::to_f(Qs[ii * LDK + d]);
#pragma unroll
      for (int qd = 0; qd < 4; ++qd) {
        if (32 * ri + 8 * qd > ii) continue;
#pragma unroll
        for (int m = 0; m < 4; ++m) {
          const int r = 4 * qd + m, j = 32 * ri + acc_row(r);
          const float e = KdaDecay<T>::exp(ii >= j ? gi - Gi[r] : 0.f);
          W[r] += (Elem<T>::to_f(M1[ii * L64 + j]) * kb + Elem<T>::to_f(M2[ii * L64 + j]) * qv) * e;
        }
      }
    }
  }
  // ---- phase B3: the gradients of q^, k^, G per token and channel; row sums for beta and the l2 norm ----
  // (the loads below stay below: moved above the sums, which leave no register free, their results would be spilled)
  asm volatile("" ::: "memory");
  f32x16 dqh, dkh, dGv;
  float ki[16], qi[16];
  // suffix sums down the tokens come later.  Rows of a block in token order: group qd = 0..3, half-wave 0 then 1,
  // m = 0..3; so[qd] is this lane's sum of a group, sx[qd] that of the other half-wave
  float so[4], sx[4];
  if (has_k) {
    const float glast = Gs[63 * LDG + d];
    float gl_sum = 0.f, blk = 0.f;
    // the sums over V of this lane's rows: all requested before the first is used, and used in two passes so that few
    // intermediate rows are alive at a time (a schedule that runs out of registers waits after every load)
    if constexpr (FULL) {   // (tiles in fragment order: token block ri, channel block cj)
      lqf.load(dQb + (ri * NKT + cj) * 1024);
      lkf.load(dK2 + (ri * NKT + cj) * 1024);
    }
    __builtin_amdgcn_sched_barrier(0);
    if constexpr (!FULL) mma32<T, 64, false, false>(dK1, TmT + 32 * ri, L64, Pt + 32 * cj, LDK);
    if constexpr (FULL) {
#pragma unroll
      for (int r = 0; r < 16; ++r) {
        const int i = 32 * ri + acc_row(r);
        ki[r] = Ks[i * LDK + d];
        qi[r] = Qs[i * LDK + d];
      }
    } else {
      AccB<T> t;
      t.load_cols(Ks + 32 * ri * LDK + 32 * cj, LDK);
      const f32x16 kd = t.unpack();
      t.load_cols(Qs + 32 * ri * LDK + 32 * cj, LDK);
      const f32x16 qd = t.unpack();
#pragma unroll
      for (int r = 0; r < 16; ++r) { ki[r] = kd[r]; qi[r] = qd[r]; }
    }
    const f32x16 lq = lqf.unpack(), lk = lkf.unpack();
    {
      f32x16 pq;
#pragma unroll
      for (int r = 0; r < 16; ++r) {
        dqh[r] = scale * KdaDecay<T>::exp(Gi[r]) * lq[r] + Uq[r];
        pq[r] = qi[r] * dqh[r];
        dGv[r] = pq[r];
      }
      rows_add_at(pq, rq + 64 * cj, 32 * ri);
    }
    {
      f32x16 pk, pb;
#pragma unroll
      for (int r = 0; r < 16; ++r) {
        const float eG = KdaDecay<T>::exp(Gi[r]), b = bs[32 * ri + acc_row(r)];
        const float t1 = -b * eG * dK1[r];
        const float t2 = KdaDecay<T>::exp(glast - Gi[r]) * lk[r];
        dkh[r] = t1 + t2 + b * U[r] + W[r];
        dGv[r] += ki[r] * (t1 + b * U[r] - t2 - W[r]);
        gl_sum += ki[r] * t2;
        pk[r] = ki[r] * dkh[r];
        pb[r] = ki[r] * (U[r] - eG * dK1[r]);
      }
      rows_add_at(pk, rk + 64 * cj, 32 * ri);
      rows_add_at(pb, rb + 64 * cj, 32 * ri);
    }
#pragma unroll
    for (int qd = 0; qd < 4; ++qd) {
      so[qd] = dGv[4 * qd] + dGv[4 * qd + 1] + dGv[4 * qd + 2] + dGv[4 * qd + 3];
      sx[qd] = __shfl_xor(so[qd], 32);
      blk += so[qd] + sx[qd];
    }
    gl_sum += __shfl_xor(gl_sum, 32);
    if (lane < 32) {
      xgl[wave * 32 + lane] = gl_sum;
      if (ri == 1) xblk[cj * 32 + lane] = blk;
    }
  }
  GDN_LDS_BARRIER();   // row sums are complete; the matrices are dead: their place takes the store patches

  // ---- phase B4: l2 norm backward, dq and dk out; dg by a reverse cumulative sum, back through the gate ----
  IdentityFrag<T> id;
  id.init();
  T* patch = M1 + wave * Patch<T>::kElems;
  float da_sum = 0.f;
  if (has_k) {
    // the raw gate input of this lane's rows, requested before the stores below
    // (as bits, widened after the loop: a conversion inside it would make every load wait for the one before)
    // (The 16-bit kernels need none for the softplus gate: there the gate's value and slope follow from G itself, below.)
    constexpr bool FROM_G = KdaDecay<T>::kBase2;
    uint32_t raws[16];
    if (fl.use_gate && !(FROM_G && !fl.has_lower_bound)) {
      if (g32) {
#pragma unroll
        for (int r = 0; r < 16; ++r)
          raws[r] = reinterpret_cast<const uint32_t*>(g)[(tok0 + imin(32 * ri + acc_row(r), nvalid - 1)) * hk + h * DK + d];
      } else {
#pragma unroll
        for (int r = 0; r < 16; ++r)
          raws[r] = reinterpret_cast<const uint16_t*>(g)[(tok0 + imin(32 * ri + acc_row(r), nvalid - 1)) * hk + h * DK + d];
      }
    }
    const int raw_shift = g32 ? 0 : 16;
    // ... and so are the two per-channel values of the gate's backward
    const float dDd = dD[d];
    const float bias = (fl.use_gate && dt_bias != nullptr) ? dt_bias[h * DK + d] : 0.f;
    if (fl.l2norm) {
      const f32x16 dotq = rows_ld4(rq, 32 * ri), dotk = rows_ld4(rk, 32 * ri);
      const f32x16 sq = rows_ld(rsq, 32 * ri), sk = rows_ld(rsk, 32 * ri);
#pragma unroll
      for (int r = 0; r < 16; ++r) {
        dqh[r] = (dqh[r] - dotq[r] * qi[r]) * sq[r];
        dkh[r] = (dkh[r] - dotk[r] * ki[r]) * sk[r];
      }
    }
    const int64_t at = (tok0 + 32 * ri) * hk + h * DK + 32 * cj;
    acc_store_rows<T, false>(dqh, id, patch, dq + at, hk, nvalid - 32 * ri);
    acc_store_rows<T, false>(dkh, id, patch, dk + at, hk, nvalid - 32 * ri);
    // dG_last: column sum over all rows of this channel, plus the decay of the state
    const float dglast = xgl[2 * cj * 32 + l32] + xgl[(2 * cj + 1) * 32 + l32] + dDd * KdaDecay<T>::exp(Gs[63 * LDG + d]);
    const bool first_half = lane < 32;
    const float a = fl.use_gate ? __expf(A_log[h]) : 0.f;
    float dt_sum = 0.f;
    // MODE 0: g is the log decay itself; 1: -e^{A_log} softplus(g + bias); 2: lower_bound sigmoid(e^{A_log} (g + bias)).
    // One copy of the loop per mode: a test of the options per element would cost as much as the gate.
    // MODE 1 in the 16-bit kernels: the token's own log decay is the difference of two rows of G (exact to half an ulp
    // of G: G_i was formed as the rounded sum of G_{i-1} and it), -e^{A_log} log2(e) softplus(raw), and the slope of the
    // softplus is 1 - e^{-softplus} = 1 - 2^{G_tok / e^{A_log}}: one exponential per element, and no second pass over
    // the gate input.
    const float inv_a = __builtin_amdgcn_rcpf(a);
    auto gate_back = [&](auto mode) {
      constexpr int MODE = decltype(mode)::value;
      f32x16 dgr;
      float later = ri == 0 ? xblk[cj * 32 + l32] : 0.f;     // everything after the group being handled
#pragma unroll
      for (int qd = 3; qd >= 0; --qd) {
        float run = later + (first_half ? sx[qd] : 0.f);
        float gprev = 0.f;   // G of the row before this group of four
        if (MODE == 1 && FROM_G) {
          const int i0 = 32 * ri + acc_row(4 * qd);
          gprev = i0 > 0 ? Gs[(i0 - 1) * LDG + d] : 0.f;
        }
#pragma unroll
        for (int m = 3; m >= 0; --m) {
          const int r = 4 * qd + m, i = 32 * ri + acc_row(r);
          run += dGv[r];
          float x = i < nvalid ? run + dglast : 0.f;     // d(log decay of token i, channel d)
          if (MODE == 1 && FROM_G) {
            const float gt = Gi[r] - (m > 0 ? Gi[r - 1] : gprev);
            da_sum += x * gt * (1.f / KdaDecay<T>::kUnit);
            x *= a * (__builtin_amdgcn_exp2f(gt * inv_a) - 1.f);
          } else if (MODE != 0) {
            const float raw = __uint_as_float(raws[r] << raw_shift) + bias;
            if (MODE == 2) {
              const float sg = kda_sigmoid(a * raw), ds_ = fl.lower_bound * sg * (1.f - sg);
              da_sum += x * ds_ * a * raw;
              x *= ds_ * a;
            } else {
              float sp, sg;
              kda_softplus_sigmoid(raw, sp, sg);
              da_sum -= x * a * sp;
              x *= -a * sg;
            }
          }
          dt_sum += x;
          dgr[r] = x;
        }
        later += so[qd] + sx[qd];
      }
      if (g32) {
#pragma unroll
        for (int r = 0; r < 16; ++r) {
          const int i = 32 * ri + acc_row(r);
          if (i < nvalid) reinterpret_cast<float*>(dg)[(tok0 + i) * hk + h * DK + d] = dgr[r];
        }
      } else {
        acc_store_rows<T, false>(dgr, id, patch, reinterpret_cast<T*>(dg) + (tok0 + 32 * ri) * hk + h * DK + 32 * cj, hk,
                                 nvalid - 32 * ri);
      }
    };
    if (!fl.use_gate) gate_back(IntConst<0>());
    else if (!fl.has_lower_bound) gate_back(IntConst<1>());
    else gate_back(IntConst<2>());
    dt_sum += __shfl_xor(dt_sum, 32);
    if (lane < 32) xdt[wave * 32 + lane] = dt_sum;
    da_sum = wave_sum(da_sum);
  }
  if (lane == 0) wsum[wave] = has_k ? da_sum : 0.f;
  GDN_LDS_BARRIER();
  if (tid == 0) {
    float x = 0.f;
#pragma unroll
    for (int w = 0; w < 8; ++w) x += wsum[w];
    part[ch * (1 + DK)] = x;
  }
  if (tid < DK) part[ch * (1 + DK) + 1 + tid] = xdt[2 * (tid >> 5) * 32 + (tid & 31)] + xdt[(2 * (tid >> 5) + 1) * 32 + (tid & 31)];
  if (tid < 64 && tid < nvalid) {
    float x = 0.f;
#pragma unroll
    for (int w = 0; w < 4; ++w) x += rb[w * 64 + tid] + rv[w * 64 + tid];
    if (fl.beta_sigmoid) { const float b = bs[tid]; x *= b * (1.f - (fl.beta_x2 ? 0.5f * b : b)); }
    gate_st<T>(dbeta, fl.beta_f32 ? 0 : 1, (tok0 + tid) * H + h, x);
  }
}

// dA_log [H] and d(dt_bias) [H*K] from the per-chunk partial sums.  A workgroup sums 32 of the 1 + K columns of one
// head: 8 threads per column take every 8th chunk, and their sums are added in a fixed order.
__global__ __launch_bounds__(kThreads) void kda_bwd_reduce_kernel(const float* __restrict__ part, const int64_t* cu,
                                                                 const int* __restrict__ chunk_offsets, int N, int nc,
                                                                 int H, int K, float* __restrict__ dA_log,
                                                                 float* __restrict__ ddt_bias) {
  __shared__ float seg_sum[8][32];
  const int h = blockIdx.x, col = 32 * blockIdx.y + (threadIdx.x & 31), seg = threadIdx.x >> 5;
  const int n = cu != nullptr ? chunk_offsets[N] : nc;
  float x = 0.f;
  if (col <= K) {
#pragma unroll 4
    for (int c = seg; c < n; c += 8) x += part[((int64_t)c * H + h) * (1 + K) + col];
  }
  seg_sum[seg][threadIdx.x & 31] = x;
  __syncthreads();
  if (seg != 0 || col > K) return;
#pragma unroll
  for (int i = 1; i < 8; ++i) x += seg_sum[i][threadIdx.x];
  if (col == 0) { if (dA_log != nullptr) dA_log[h] = x; }
  else if (ddt_bias != nullptr) ddt_bias[h * K + col - 1] = x;
}

template <typename T, int DK, int NWS, int NLS, int STAGES>
static int kda_bwd_launch(const ChunkDims& d, const KdaWorkspace& L, const void* q, const void* k, const void* v,
                          const void* g, const float* A_log, const float* dt_bias, const int64_t* cu, const void* dO,
                          const float* dht, void* dq, void* dk, void* dv, void* dg, void* dbeta, float* dA_log,
                          float* ddt_bias, float* dh0, unsigned char* ws, float scale, const KdaFlags& fl, hipStream_t st) {
  const int H = d.Hv;
  const int nc = (int)d.max_chunks();
  const int* chunk_offsets = reinterpret_cast<const int*>(ws + L.chunk_offsets);
  const float* bhat = reinterpret_cast<const float*>(ws + L.bhat);
  const float* dec = reinterpret_cast<const float*>(ws + L.dec);
  const T* Ai = reinterpret_cast<const T*>(ws + L.Ai);
  const T* AQ = reinterpret_cast<const T*>(ws + L.AQ);
  const T* K1F = reinterpret_cast<const T*>(ws + L.K1F);
  const T* K2F = reinterpret_cast<const T*>(ws + L.K2F);
  const T* VF = reinterpret_cast<const T*>(ws + L.VF);
  const T* HF = reinterpret_cast<const T*>(ws + L.HF);
  const T* TMR = reinterpret_cast<const T*>(ws + L.TMR);
  const T* QBT = reinterpret_cast<const T*>(ws + L.QBT);
  T* DVF = reinterpret_cast<T*>(ws + L.DVF);
  T* DHF = reinterpret_cast<T*>(ws + L.DHF);
  T* DUMP = reinterpret_cast<T*>(ws + L.DUMP);
  float* DD = reinterpret_cast<float*>(ws + L.DD);
  float* PART = reinterpret_cast<float*>(ws + L.PART);
  {
    auto kern = chunk_state_bwd_kernel<T, DK, NWS, NLS, STAGES, true>;
    constexpr int smem = StateBwdSmem<T, DK, NWS, STAGES, true>::bytes;
    if (int e = set_lds_b(kern, smem)) return e;
    GDN_LAUNCH(kKernStateBwd, st, kern, dim3(d.N * H, d.V / (32 * NWS)), dim3(64 * (NWS + NLS)), smem, st, K2F, K1F, QBT,
               Ai, AQ, (const T*)dO, dec, (const void*)bhat, 0, dht, dh0, DVF, DHF, cu, chunk_offsets, d.T, H, H, d.V, scale);
  }
  {
    auto kern = chunk_bwd_local_kernel<T, DK, true>;
    constexpr int smem = BwdLocalSmem<T, DK>::bytes;
    if (int e = set_lds_b(kern, smem)) return e;
    TokenStrides ts = d.strides();
    GDN_LAUNCH(kKernBwdLocal, st, kern, dim3(nc, H), dim3(kThreads), smem, st, QBT, K1F, (const T*)v, (const void*)bhat, 0,
               (const float*)nullptr, Ai, VF, (const T*)DVF, (const T*)dO, HF, (const T*)DHF, (const float*)nullptr,
               (const float*)nullptr, (T*)nullptr, (T*)nullptr, (T*)dv, (void*)nullptr, (float*)nullptr, cu, chunk_offsets, d.T,
               d.N, H, H, d.V, scale, 0, ts, DUMP, DD, device_compute_units());
  }
  {
    const int es = (int)sizeof(T), ge = fl.g_f32 ? 4 : es, be = fl.beta_f32 ? 4 : es;
    const int64_t kb = (int64_t)H * DK, vb = (int64_t)H * d.V;
    TailRows tail{{dq, dk, dv, dg, dbeta}, {kb * es, kb * es, vb * es, kb * ge, (int64_t)H * be},
                  {(int)(kb * es), (int)(kb * es), (int)(vb * es), (int)(kb * ge), H * be}};
    launch_zero_tail_rows(cu, d.N, d.tokens(), tail, st);
  }
  {
    auto kern = kda_bwd_finish_kernel<T, DK>;
    constexpr int smem = KdaBwdSmem<T, DK>::bytes;
    if (int e = set_lds_b(kern, smem)) return e;
    GDN_LAUNCH(kKernKdaBwdFinish, st, kern, dim3(nc, H), dim3(kFinThreads), smem, st, (const T*)q, (const T*)k, g, A_log, dt_bias,
               bhat, TMR, (const T*)DUMP, (const float*)DD, cu, chunk_offsets, (T*)dq, (T*)dk, dg, dbeta, PART, d.T, d.N, H, scale, fl);
  }
  if (fl.use_gate && (dA_log != nullptr || ddt_bias != nullptr))
    GDN_LAUNCH(kKernKdaBwdReduce, st, kda_bwd_reduce_kernel, dim3(H, (d.K + 32) / 32), dim3(kThreads), 0, st, (const float*)PART, cu,
               chunk_offsets, d.N, nc, H, d.K, dA_log, ddt_bias);
  return (int)hipGetLastError();
}

}  // namespace gdn

extern "C" int gdn_kda_bwd(const void* q, const void* k, const void* v, const void* g, const float* A_log,
                           const float* dt_bias, const int64_t* cu_seqlens, const void* d_o, const float* d_final_state,
                           void* dq, void* dk, void* dv, void* dg, void* dbeta, float* dA_log, float* ddt_bias,
                           float* d_initial_state, void* workspace, int64_t workspace_bytes, int B, int T, int N, int H,
                           int K, int V, float scale, int use_qk_l2norm, int use_gate, int has_lower_bound,
                           float lower_bound, int beta_sigmoid, int allow_neg_eigval, int dtype, int g_dtype,
                           int beta_dtype, void* stream) {
  using namespace gdn;
  if (!q || !k || !v || !g || !d_o || !dq || !dk || !dv || !dg || !dbeta || !workspace) return -1;
  if (use_gate && !A_log) return -1;
  ChunkDims d{B, T, N, H, H, K, V, cu_seqlens != nullptr};
  if (int e = chunk_check_dims(d, dtype)) return e;
  if ((g_dtype != 0 && g_dtype != dtype) || (beta_dtype != 0 && beta_dtype != dtype)) return -4;
  if (((uintptr_t)q | (uintptr_t)k | (uintptr_t)v | (uintptr_t)g | (uintptr_t)d_o | (uintptr_t)dq | (uintptr_t)dk |
       (uintptr_t)dv | (uintptr_t)dg) & 15)
    return -6;
  ChunkDims dl = d;
  dl.varlen = true;
  const KdaWorkspace L = kda_workspace_layout(dl, dtype == 0 ? 4 : 2);
  if (workspace_bytes < L.total_bytes || (reinterpret_cast<uintptr_t>(workspace) & 255) != 0) return -5;
  KdaFlags fl{use_qk_l2norm, use_gate, has_lower_bound, beta_sigmoid, allow_neg_eigval, g_dtype == 0, beta_dtype == 0, lower_bound};
  unsigned char* ws = static_cast<unsigned char*>(workspace);
  hipStream_t st = (hipStream_t)stream;
#define GDN_KDAB(T_, DK_, NWS_, NLS_, ST_)                                                                              \
  return kda_bwd_launch<T_, DK_, NWS_, NLS_, ST_>(d, L, q, k, v, g, A_log, dt_bias, cu_seqlens, d_o, d_final_state, dq, dk, dv, \
                                                  dg, dbeta, dA_log, ddt_bias, d_initial_state, ws, scale, fl, st)
  const bool one_slab = one_slab_per_workgroup(d, device_compute_units());
  if (dtype == 1) {
    if (K == 128) {
      if (one_slab) GDN_KDAB(bf16_t, 128, 1, 4, 2);
      GDN_KDAB(bf16_t, 128, 2, 4, 2);
    }
    GDN_KDAB(bf16_t, 64, 2, 2, 2);
  } else {
    if (K == 128) GDN_KDAB(float, 128, 2, 2, 1);
    GDN_KDAB(float, 64, 2, 2, 1);
  }
#undef GDN_KDAB
}
