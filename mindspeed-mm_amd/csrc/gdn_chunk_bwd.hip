// Chunked gated delta rule, backward pass.  Notation as in gdn_chunk_fwd.hip; S is the state BEFORE a
// chunk, dS' the gradient of the state AFTER it, Gam_ij = e^{G_i - G_j}, everything per (sequence, head):
//   dv_local = scale tril(Q K^T . Gam)^T dO                                   chunk_state_bwd_kernel
//   dV' = (K dS') . e^{G_last-G} + dv_local                                   chunk_state_bwd_kernel
//   dS  = e^{G_last} dS' + scale (Q . e^G)^T dO - W^T dV'                       (reverse recurrence)
//   ds  = scale tril(dO V'^T . Gam);  dQ = scale e^G . (dO S^T) + ds K          chunk_bwd_local_kernel
//   dK1 = e^{G_last-G} . (V' dS'^T) + ds^T Q;  dW = -dV' S^T
//   dG1_i = <q_i,dQ_i> - <k_i,dK1_i>  (+ e^{G_last}<S,dS'> + sum_j <k_j, dK_inter_j> at the last row)
//   back through W = Tm (beta e^G K), U = Tm (beta V), Tm = (I+L)^-1:           (same kernel)
//     P = Tm^T dW, R = Tm^T dV', dTm = strict_tril(dW Kb^T + dV' Vb^T), dM = -(Tm^T dTm Tm^T) . Gam
//     dK2 = P beta e^G + beta (dM K) + dM^T (beta K);  dv = R beta
//     dbeta = e^G<P,k> + <R,v> + <dM K, k>;  dG2 = beta e^G<P,k> + beta<dM K,k> - <dM^T(beta K),k>
//   dg = reverse chunk-local cumsum(dG1 + dG2); group sum of dq/dk over grouped heads and the
//   l2-norm backward dx = (dy - <dy,y> y) rstd                                  (same kernel)
// The equations are those of the reference's backward kernels (mindspeed_mm/fsdp/ops/gdn/triton/
// chunk_o.py:19-284, chunk_delta_h.py:307-513, wy_fast.py:17-141, chunk_gated_delta_rule.py:88-174), with
// the dG row/column sums rewritten as row dot products with dQ/dK so that Q K^T need not be rebuilt.
#include "gdn_chunk.h"
#include "gdn_common.h"
#include "gdn_profile.h"

namespace gdn {

// ---------------------------------------------------------------------------------------------
// chunk_state_bwd_kernel: the reverse recurrence, mirror of chunk_state_kernel.  One compute wave owns a 32-column
// slab of dS[K, 32] in fp32 accumulators and per chunk (last to first) does
//     dV' = e^{G_last-G} . (K dS) + (scale Aq)^T dO
//     R = Tm^T dV'        dS <- e^{G_last} dS + Q^T (scale e^G . dO) - K^T (beta e^G . R)
// (the last term is W^T dV' with W = Tm (beta e^G K) never materialised), dS, dV', R and the scaled dO used as B
// operands straight from registers.  dS (gradient of the state AFTER the chunk) and dV' leave in fragment order.
// Loader waves copy the A operands from contiguous fragment-order blocks: K and Q^T per q/k group, Tm and Aq per value
// head; K^T and Tm^T are the same images read with the transposing LDS read, and so are the slab's raw dO rows on
// their way into the B-operand layout.  The per-token factors never enter the compute wave's dependent chain: the
// loaders write K twice, rows scaled by e^{G_last-G} (for K dS) and by -beta e^G (for the K^T product), and dO twice,
// raw and with rows scaled by scale e^G.
// ---------------------------------------------------------------------------------------------
template <typename T, int DK, int NW, int STAGES, bool KDA = false> struct StateBwdSmem {
  // one stage, in elements of T
  static constexpr int off_k = 0;                        // K images [2][K/32][2] tiles: rows x e^{G_last-G}, rows x -beta e^G
  static constexpr int off_q = off_k + 2 * 64 * DK;      // Q^T image
  static constexpr int off_tm = off_q + 64 * DK;         // Tm tiles (0,0), (1,0), (1,1)
  static constexpr int off_aq = off_tm + 3 * 1024;       // Aq tiles (0,0), (1,0), (1,1)
  static constexpr int off_do = off_aq + 3 * 1024;       // dO rows of the slabs [2][64][32 NW]: raw, rows x scale e^G
  static constexpr int off_row = (off_do + 2 * 64 * 32 * NW) * (int)sizeof(T);   // bytes: G_last; KDA: e^{G_last} per key channel [DK]
  static constexpr int stage = off_row + (KDA ? DK * 4 : 16);
  static constexpr int bytes = STAGES * stage;
  static_assert(bytes <= 160 * 1024, "one CU's LDS");
};

template <int PIECES, int NT> struct DealB { static constexpr int kPer = (PIECES + NT - 1) / NT; };

// KDA (one decay per key channel): kaf and kaf2 hold the two K images ready-made (rows x e^{G_last-G} and rows x
// -beta e^{G}, channel by channel), qtf the transposed rows of q with scale and decay already applied (so dO is used
// as it is), G holds e^{G_last} [chunks,Hv,DK]; the rows of dS decay each by their own factor.
template <typename T, int DK, int NW, int NL, int STAGES, bool KDA = false>
__global__ __launch_bounds__(64 * (NW + NL)) GDN_WAVES_PER_SIMD((sizeof(T) == 2 && NL >= 4) ? 2 : 1) void chunk_state_bwd_kernel(
    const T* __restrict__ kaf, const T* __restrict__ kaf2, const T* __restrict__ qtf, const T* __restrict__ ai, const T* __restrict__ aqf,
    const T* __restrict__ dO, const float* __restrict__ G, const void* __restrict__ beta, int beta_same,
    const float* __restrict__ dht,
    float* __restrict__ dh0, T* __restrict__ dvf, T* __restrict__ dhf, const int64_t* __restrict__ cu,
    const int* __restrict__ chunk_offsets, int T_len, int Hqk, int Hv, int V, float scale) {
  using SM = StateBwdSmem<T, DK, NW, STAGES, KDA>;
  static_assert(!KDA || 64 * NL >= DK, "a loader thread per key channel");
  constexpr int NT = 64 * NL, VEC = Elem<T>::kVec, NKT = DK / 32;   // NT loader threads
  constexpr int PK = 64 * DK / VEC, PTM = 3 * 1024 / VEC, PD = 64 * 32 * NW / VEC, DPR = 32 * NW / VEC;
  constexpr int CK = DealB<PK, NT>::kPer, CTM = DealB<PTM, NT>::kPer, CD = DealB<PD, NT>::kPer;
  static_assert(STAGES == 1 || STAGES == 2, "one or two LDS stages");

  const int tid = threadIdx.x;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);   // wave-uniform: the roles branch on a scalar
  const int nh = xcd_grouped_head(blockIdx.x, gridDim.x, Hv / Hqk), n = nh / Hv, h = nh % Hv;
  const int64_t bos = cu ? cu[n] : (int64_t)n * T_len;
  const int len = cu ? (int)(cu[n + 1] - bos) : T_len;
  const int nchunks = (len + kChunk - 1) / kChunk;
  const int64_t chunk_base = cu ? chunk_offsets[n] : (int64_t)n * ((T_len + kChunk - 1) / kChunk);

  // step s = 0 .. nchunks-1 handles chunk nchunks-1-s
  if (wave >= NW) {
    // ================= loader waves =================
    const int lt = tid - 64 * NW;
    constexpr int DEPTH = (STAGES == 2) ? 2 : 1;
    Vec16<T> pk[DEPTH][CK], pk2[DEPTH][KDA ? CK : 1], pq[DEPTH][CK], ptm[DEPTH][CTM], pa[DEPTH][CTM], pd[DEPTH][CD];
    float pgl[DEPTH], pgk[DEPTH][2], pgd[DEPTH][CD];
    uint32_t pbk[DEPTH][2];   // beta as fetched
    int pnv[DEPTH];
    static_assert(NT % (sizeof(T) == 2 ? 128 : 32) == 0, "a thread's pieces sit at one place of their tiles");
    const int krow = frag_piece_row<T>(lt & 127);
    auto tm_src = [&](int idc) {   // piece of the three kept tiles -> its place among the four stored ones
      const int t = idc / (1024 / VEC);
      return (t == 0 ? 0 : t + 1) * (1024 / VEC) + idc % (1024 / VEC);
    };
    auto issue = [&](int st, int set) {
      const int c = nchunks - 1 - st;
      const int64_t tok0 = bos + (int64_t)c * kChunk;
      const int nvalid = imin(kChunk, len - c * kChunk);
      const int64_t ch = (chunk_base + c) * Hv + h, chq = (chunk_base + c) * Hqk + h / (Hv / Hqk);
#pragma unroll
      for (int i = 0; i < CK; ++i) {
        const int idc = imin(lt + i * NT, PK - 1);
        pk[set][i] = ld16(kaf + chq * (64 * DK) + idc * VEC);
        if constexpr (KDA) pk2[set][i] = ld16(kaf2 + chq * (64 * DK) + idc * VEC);
        pq[set][i] = ld16(qtf + chq * (64 * DK) + idc * VEC);
      }
#pragma unroll
      for (int i = 0; i < CTM; ++i) {
        const int src = tm_src(imin(lt + i * NT, PTM - 1));
        ptm[set][i] = ld16(ai + ch * 4096 + src * VEC);
        pa[set][i] = ld16(aqf + ch * 4096 + src * VEC);
      }
#pragma unroll
      for (int i = 0; i < CD; ++i) {   // dO rows of the slabs; rows past the end repeat the last one and are cleared below
        const int idc = imin(lt + i * NT, PD - 1), row = imin(idc / DPR, nvalid - 1), cc = idc % DPR;
        pd[set][i] = ld16(dO + ((tok0 + row) * Hv + h) * V + blockIdx.y * (32 * NW) + cc * VEC);
        if constexpr (!KDA) pgd[set][i] = G[ch * 64 + row];
      }
      pnv[set] = nvalid;
      if constexpr (KDA) {
        pgl[set] = G[ch * DK + imin(lt, DK - 1)];   // e^{G_last} of this thread's key channel
        return;
      }
      const float* gc = G + ch * 64;
      // raw values only: arithmetic here would wait for every load issued so far.  The array repeats G_last past the
      // end of a short chunk.  In the K tiles every 16-byte piece belongs to one token, 32 (tile & 1) + the row of its
      // place, and this thread's pieces all sit at the same place of their tiles: the gates of two tokens cover them.
      pgl[set] = gc[63];
#pragma unroll
      for (int j = 0; j < 2; ++j) {
        pgk[set][j] = gc[32 * j + krow];
        pbk[set][j] = gate_raw<T>(beta, beta_same, (tok0 + imin(32 * j + krow, nvalid - 1)) * Hv + h);
      }
    };
    auto commit = [&](int set, int buf) {
      T* st = reinterpret_cast<T*>(gdn_smem + buf * SM::stage);
      float f1[2], f2[2];
      if constexpr (!KDA) {
#pragma unroll
        for (int j = 0; j < 2; ++j) {
          f1[j] = __expf(pgl[set] - pgk[set][j]);
          f2[j] = (32 * j + krow < pnv[set]) ? -gate_val<T>(pbk[set][j], beta_same) * __expf(pgk[set][j]) : 0.f;
        }
      }
#pragma unroll
      for (int i = 0; i < CK; ++i) {
        const int idc = imin(lt + i * NT, PK - 1), tj = (idc / (1024 / VEC)) & 1;
        if constexpr (KDA) {
          st16(st + SM::off_k + idc * VEC, pk[set][i]);
          st16(st + SM::off_k + 64 * DK + idc * VEC, pk2[set][i]);
        } else {
          st16(st + SM::off_k + idc * VEC, scale16<T>(pk[set][i], f1[tj]));
          st16(st + SM::off_k + 64 * DK + idc * VEC, scale16<T>(pk[set][i], f2[tj]));
        }
        st16(st + SM::off_q + idc * VEC, pq[set][i]);
      }
#pragma unroll
      for (int i = 0; i < CTM; ++i) {
        const int idc = imin(lt + i * NT, PTM - 1);
        st16(st + SM::off_tm + idc * VEC, ptm[set][i]);
        st16(st + SM::off_aq + idc * VEC, pa[set][i]);
      }
#pragma unroll
      for (int i = 0; i < CD; ++i) {
        const int idc = imin(lt + i * NT, PD - 1);
        const Vec16<T> x = idc / DPR < pnv[set] ? pd[set][i] : zero16<T>();
        st16(st + SM::off_do + idc * VEC, x);
        if constexpr (KDA) st16(st + SM::off_do + 64 * 32 * NW + idc * VEC, x);
        else st16(st + SM::off_do + 64 * 32 * NW + idc * VEC, scale16<T>(x, scale * __expf(pgd[set][i])));
      }
      float* row = reinterpret_cast<float*>(gdn_smem + buf * SM::stage + SM::off_row);
      if constexpr (KDA) {
        if (lt < DK) row[lt] = pgl[set];
        return;
      }
      if (lt == 0) row[0] = pgl[set];
    };
    if (nchunks == 0) return;
    if (STAGES == 2) {
      // Every path through this loop issues the same loads in the same order (steps past the end are clamped and
      // their data is never used), so that the number of loads in flight at each wait is a compile-time fact.
      issue(0, 0);
      commit(0, 0);
#pragma unroll
      for (int j = 1; j <= DEPTH; ++j) issue(imin(j, nchunks - 1), j % DEPTH);
      // The loop leaves only at the end of a whole round of register sets: an exit in the middle of the round would be
      // one more way into the code that follows it, one on which fewer loads are in flight, and the waits before the
      // LDS writes (counted by the compiler over all ways in) would then also wait for the younger set.
      int s0 = 0;
      for (; s0 + DEPTH <= nchunks; s0 += DEPTH) {
#pragma unroll
        for (int u = 0; u < DEPTH; ++u) {
          const int st = s0 + u;
          GDN_LDS_BARRIER();                // (A) step st staged; the other stage (step st-1) is free
          commit((u + 1) % DEPTH, (st + 1) & 1);
          issue(imin(st + 1 + DEPTH, nchunks - 1), (u + 1) % DEPTH);
        }
      }
#pragma unroll
      for (int u = 0; u < DEPTH - 1; ++u) {   // the steps left over: their barriers, and the stage the next one reads
        const int st = s0 + u;
        if (st < nchunks) {
          GDN_LDS_BARRIER();
          commit((u + 1) % DEPTH, (st + 1) & 1);
        }
      }
    } else {
      for (int st = 0; st < nchunks; ++st) {
        if (st > 0) GDN_LDS_BARRIER();      // (B) the single stage is free again
        issue(st, 0);
        commit(0, 0);
        GDN_LDS_BARRIER();                  // (A)
      }
    }
    return;
  }

  // ================= compute waves =================
  const int vblk = blockIdx.y * NW + wave, v0 = 32 * vblk;
  f32x16 dS[NKT];
#pragma unroll
  for (int kt = 0; kt < NKT; ++kt) {
    dS[kt] = acc_zero();
    if (dht != nullptr) {
#pragma unroll
      for (int r = 0; r < 16; ++r)
        dS[kt][r] = dht[(((int64_t)n * Hv + h) * DK + 32 * kt + acc_row(r)) * V + v0 + acc_col()];
    }
  }
  // As in the forward recurrence the vector work that does not depend on the running products (decay and packing of
  // dS) is written between the matrix instructions.
  AccB<T> dSb[NKT];
#pragma unroll
  for (int kt = 0; kt < NKT; ++kt) dSb[kt].pack(dS[kt]);
  // Two tile products into two accumulators, the matrix instructions of one alternating with those of the other: back
  // to back on one accumulator a matrix instruction costs half as much again (49 cycles against 34, measured).
  auto mma2 = [](f32x16& x0, const AccB<T>& a0, const AccB<T>& b0, f32x16& x1, const AccB<T>& a1, const AccB<T>& b1) {
#pragma unroll
    for (int kg = 0; kg < AccK<T>::kGroups; ++kg) {
      mfma_kgroup<T>(x0, a0.f[kg], b0.f[kg]);
      mfma_kgroup<T>(x1, a1.f[kg], b1.f[kg]);
    }
  };
  for (int st = 0; st < nchunks; ++st) {
    const int c = nchunks - 1 - st;
    const int buf = (STAGES == 2) ? (st & 1) : 0;
    GDN_LDS_BARRIER();                      // (A)
    const T* sm = reinterpret_cast<const T*>(gdn_smem + buf * SM::stage);
    const T* Ka = sm + SM::off_k;              // rows x e^{G_last-G}
    const T* Kn = Ka + 64 * DK;                // rows x -beta e^G
    const T* Qa = sm + SM::off_q;
    const T* Tm = sm + SM::off_tm;
    const T* Aq = sm + SM::off_aq;
    const T* dOs = sm + SM::off_do;
    const float* row = reinterpret_cast<const float*>(gdn_smem + buf * SM::stage + SM::off_row);
    // dO of this wave's 32 columns as B operand (lane <-> V column, registers <-> token), raw and scaled by scale e^G
    // of its token: the factor of the Q^T product rides on dO, so that the Q^T tiles are the same for every value head
    // of a q/k group
    AccB<T> dob[2], dos[2], aq[3];
    dob[0].load_cols(dOs + 32 * wave, 32 * NW);
    dob[1].load_cols(dOs + 32 * (32 * NW) + 32 * wave, 32 * NW);
    dos[0].load_cols(dOs + 64 * 32 * NW + 32 * wave, 32 * NW);
    dos[1].load_cols(dOs + 64 * 32 * NW + 32 * (32 * NW) + 32 * wave, 32 * NW);
    aq[0].load(Aq);                           // tiles (0,0), (1,0), (1,1)
    aq[1].load(Aq + 1024);
    aq[2].load(Aq + 2048);
    const float eg = KDA ? 1.f : __expf(row[0]);
    const int64_t tile0 = ((chunk_base + c) * Hv + h) * (V / 32) + vblk;
#pragma unroll
    for (int kt = 0; kt < NKT; ++kt) dSb[kt].store_stream(dhf + (tile0 * NKT + kt) * 1024);
    // dV' = (scale tril(Q K^T . Gam))^T dO (from the forward pass's tiles) + (e^{G_last-G} . K) dS, one accumulation
    // chain per 32-token block.  The pair of A-operand tiles of K tile kt + 1 is requested from LDS before the matrix
    // instructions of K tile kt are issued (two register buffers); the decay of dS rides in between.
    f32x16 a0 = acc_zero(), a1 = acc_zero();
    AccB<T> af[2][2];                         // [buffer][tile of the pair]
    af[0][0].load(Ka);
    af[0][1].load(Ka + 1024);
    mma2(a0, aq[0], dob[0], a1, aq[2], dob[1]);
    mma32_ff<T>(a0, aq[1], dob[1]);
    GDN_SCHED_FENCE();
#pragma unroll
    for (int kt = 0; kt < NKT; ++kt) {        // K tile kt, both 32-token blocks: one accumulator each
      if (kt + 1 < NKT) {
        af[(kt + 1) & 1][0].load(Ka + (2 * kt + 2) * 1024);
        af[(kt + 1) & 1][1].load(Ka + (2 * kt + 3) * 1024);
      }
      mma2(a0, af[kt & 1][0], dSb[kt], a1, af[kt & 1][1], dSb[kt]);
      if constexpr (KDA) {
        const f32x16 dk = rows_ld(row, 32 * kt);   // the decay of each of the tile's 32 key channels
#pragma unroll
        for (int r = 0; r < 16; ++r) dS[kt][r] *= dk[r];
      } else {
#pragma unroll
        for (int r = 0; r < 16; ++r) dS[kt][r] *= eg;
      }
      GDN_SCHED_FENCE();
    }
    AccB<T> dvb[2], rb[2], tf[3];
#pragma unroll
    for (int t = 0; t < 3; ++t) tf[t].load_t(Tm + t * 1024);   // Tm^T tiles: (lane <-> column of Tm, registers <-> row)
    dvb[0].pack(a0);
    dvb[1].pack(a1);
    dvb[0].store_stream(dvf + (tile0 * 2 + 0) * 1024);
    dvb[1].store_stream(dvf + (tile0 * 2 + 1) * 1024);
    // R = Tm^T dV' (upper triangular: R_0 = Tm00^T dV'_0 + Tm10^T dV'_1, R_1 = Tm11^T dV'_1)
    f32x16 y0 = acc_zero(), y1 = acc_zero();
    mma2(y0, tf[0], dvb[0], y1, tf[2], dvb[1]);
    mma32_ff<T>(y0, tf[1], dvb[1]);
    // A operands of the update of dS, for the pair of 32-row tiles (2 pr, 2 pr + 1) of dS and product p = 2 tj + w:
    // w = 0 the Q^T tile as it lies, w = 1 the K image read transposed
    auto load_qk = [&](int b, int pr, int p) {
#pragma unroll
      for (int j = 0; j < 2; ++j) {
        const T* tile = ((p & 1) ? Kn : Qa) + ((2 * pr + j) * 2 + (p >> 1)) * 1024;
        if (p & 1) af[b][j].load_t(tile); else af[b][j].load(tile);
      }
    };
    load_qk(0, 0, 0);
    rb[0].pack(y0);
    rb[1].pack(y1);
    GDN_SCHED_FENCE();
    // dS <- e^{G_last} dS + Q^T (scale e^G . dO) + (-beta e^G . K)^T R, two tiles of dS at a time so that consecutive
    // matrix instructions never accumulate into the same one; a finished pair is packed for the next step while the
    // matrix pipe works on the following one
    static_assert(NKT % 2 == 0, "tiles of dS are updated in pairs");
#pragma unroll
    for (int m = 0; m < 2 * NKT; ++m) {       // m = 4 pr + p
      const int pr = m >> 2, pp = m & 3;
      if (m + 1 < 2 * NKT) load_qk((m + 1) & 1, (m + 1) >> 2, (m + 1) & 3);
      const AccB<T>& bop = (pp & 1) ? rb[pp >> 1] : dos[pp >> 1];
      mma2(dS[2 * pr], af[m & 1][0], bop, dS[2 * pr + 1], af[m & 1][1], bop);
      if (pp == 1 && pr >= 1) {
        dSb[2 * pr - 2].pack(dS[2 * pr - 2]);
        dSb[2 * pr - 1].pack(dS[2 * pr - 1]);
      }
      GDN_SCHED_FENCE();
    }
    dSb[NKT - 2].pack(dS[NKT - 2]);
    dSb[NKT - 1].pack(dS[NKT - 1]);
    if (STAGES == 1 && st + 1 < nchunks) GDN_LDS_BARRIER();   // (B)
  }
  if (dh0 != nullptr) {
#pragma unroll
    for (int kt = 0; kt < NKT; ++kt)
#pragma unroll
      for (int r = 0; r < 16; ++r)
        dh0[(((int64_t)n * Hv + h) * DK + 32 * kt + acc_row(r)) * V + v0 + acc_col()] = dS[kt][r];
  }
}

// ---------------------------------------------------------------------------------------------
// chunk_bwd_local_kernel, per (chunk, head), 4 waves: everything of the backward pass that is local to a chunk once
// the reverse recurrence has left dS' and dV' behind.  Wave w owns the 32 K-columns [32w, 32w+32) of dQ, dK, dW and
// the 32x32 tile (w/2, w%2) of the 64x64 intra-chunk matrices.
//   main loop over 32-column V blocks:
//     v_new, dV', dO, S, dS' arrive in fragment order with (lane <-> V column); the contractions run over V, so each
//     tile is turned through the matrix core (mfma_transpose) into (lane <-> token / K column, registers <-> V).
//       ds += dO V'^T   a2 += dV' V^T   dQ += dO S^T   dK += V' dS'^T   dW += dV' S^T
//     and two waves per block also form R = Tm^T dV' from the tiles as they lie -> dv = beta R.
//     All operands of a V block are copied by direct global->LDS loads (no registers in between, fragment order is
//     exactly the layout such a load produces) into one of two stages, one block ahead of the arithmetic: tiles
//     shared by the four waves once per workgroup, S and dS' per wave.  During the last block the idle stage
//     receives the epilogue's operands (K in fragment order, this wave's Q columns) the same way.
//   epilogue: dQ += ds K, dK += ds^T Q, dG rows as <q,dQ> - <k,dK>; then back through W = Tm (beta e^G K) with dW
//   still in registers: P = Tm^T dW, a1 = dW K^T, dTm = strict_tril(a1 beta e^G + a2 beta), dM = -(Tm^T dTm Tm^T).Gam,
//   dK += beta e^G P + beta (dM K) + dM^T (beta K); dbeta, dg.  The 64x64 intermediates pass between the waves as
//   fragment-order tiles in LDS, in one or both of two forms of a tile X(i,j) owned as an accumulator:
//     D ("direct"):      pack(X)                  lane <-> j, registers <-> i
//     T ("transposed"):  pack(transpose(pack(X)))  lane <-> i, registers <-> j
//   dQ, dK, dv leave as 16-byte row pieces.
// ---------------------------------------------------------------------------------------------
template <typename T, int DK> struct BwdLocalSmem {
  // main loop, in elements:
  //   sh   [2 stages][v_new x2 | dV' x2]      shared fragment tiles of one 32-column V block, one block ahead
  //   raw  [2 buffers][dO [64][64] | V [64][64]]  raw rows of a PAIR of V blocks (SwizzledTile<T, 64>): 128-byte row
  //        pieces, i.e. whole lines of dO and V (32-column blocks would use half of every line they touch and fetch
  //        it twice), one pair ahead
  //   priv [4 waves][S | dS']                 per wave, single: a wave takes its tiles into registers at the top of a
  //        block and requests the next block's right behind
  static constexpr int sh = 0, raw = 2 * 4096, raw_elems = 2 * 64 * 64, priv = raw + 2 * raw_elems, main_elems = priv + 4 * 2048;
  // epilogue: K tiles [K/32][2] in the raw buffer that idles during the last block, the Q^T tiles [2] of each wave in
  // its priv slot (later the (beta dM) D-form tiles); then dW tiles [2][K/32] (later the store patches) in the other raw
  // buffer, D-form tiles [4] and T-form tiles [4] in the two shared stages
  static constexpr int off_tm = main_elems * (int)sizeof(T);                 // Tm tiles [2][2], whole kernel
  static constexpr int off_row = off_tm + 4 * 1024 * (int)sizeof(T);
  static constexpr int bytes = off_row + (8 * 64 + 5 * 256 + 8) * 4;   // 8 row vectors, 5 per-wave row-sum arrays
  static_assert(main_elems == 32 * 1024, "as large as two former stages");
  static_assert(4 * Patch<T>::kElems <= raw_elems && 2 * (DK / 32) * 1024 <= raw_elems, "epilogue tenants fit");
};

// KDA (one decay per key channel): the sums over V are the same, what follows them is not.  The kernel then stops after
// its main loop (dv is written there) and leaves the sums in kda_dump, per chunk and head
//   [dQb = dO S^T | dK2 = V' dS'^T | P = dV' S^T : 64 x DK each][dAq = dO V'^T | a2 = dV' V^T : 64 x 64 each, lower tiles]
// rounded to T like every other tensor that passes between two kernels (they are the largest of them: in fp32 they made
// up half of what the backward pass moved), and dD = sum_v dS' . S [DK] in kda_dd, in fp32,
// for kda_bwd_finish_kernel; G is not read and beta is the transformed beta in fp32.
template <typename T, int DK, bool KDA = false>
__global__ __launch_bounds__(kThreads, sizeof(T) == 2 ? 2 : 1) void chunk_bwd_local_kernel(
    const T* __restrict__ qtf, const T* __restrict__ kaf, const T* __restrict__ v, const void* __restrict__ beta, int beta_same,
    const float* __restrict__ G, const T* __restrict__ Ai, const T* __restrict__ vf, const T* __restrict__ dvf,
    const T* __restrict__ dO, const T* __restrict__ hf, const T* dhf_in, const float* __restrict__ rstd_q,
    const float* __restrict__ rstd_k, T* dq, T* dk, T* __restrict__ dv_out, void* __restrict__ dbeta,
    float* __restrict__ dg, const int64_t* __restrict__ cu, const int* __restrict__ chunk_offsets, int T_len, int N,
    int Hqk, int Hv, int V, float scale, int hh, TokenStrides ts, T* __restrict__ kda_dump, float* __restrict__ kda_dd,
    int cus) {
  using SM = BwdLocalSmem<T, DK>;
  constexpr int NKT = DK / 32, VEC = Elem<T>::kVec, KG = AccK<T>::kGroups;
  static_assert(NKT <= 4, "one 32-column block of K per wave");
  T* stage0 = reinterpret_cast<T*>(gdn_smem);
  T* TmF = reinterpret_cast<T*>(gdn_smem + SM::off_tm);
  float* Gs = reinterpret_cast<float*>(gdn_smem + SM::off_row);
  float* egs = Gs + 64;    // e^G
  float* bs = egs + 64;    // beta
  float* rsq = bs + 64;    // 1/|q_i|, 1/|k_i| of the l2 normalisation (1 without it)
  float* rsk = rsq + 64;
  // row sums, one slot of 64 rows per wave (see rows_add):
  float* rq = rsk + 64;    // <q_i, dQ_i>
  float* rk1 = rq + 256;   // <k_i, dK_i> before the terms that come back through W
  float* rbk = rk1 + 256;  // e^G <P_i,k_i> + <E_i,k_i>: dbeta without the V part; times beta it is part of dG and <k,dK>
  float* rf = rbk + 256;   // <F_i, k_i>
  float* rv = rf + 256;    // <R_i, v_i>, taken as the column sums of Tm . (dV' V^T)
  float* wsum = rv + 256;  // per wave: <S,dS'> [0..3], sum_i <k_i, dK_inter_i> [4..7]
  float* rqc = wsum + 8;   // <q_i, dQ_i> summed over the waves' slots
  float* sgs = rqc + 64;   // scale e^{G_i}: the row factor of the inter-chunk part of dQ
  float* egl = sgs + 64;   // e^{G_last - G_i}: that of dK (one exponential per row here instead of one per element there)

  stagger_second_resident<127>(KDA ? 3 : 4, 8 * cus, cus);   // about half of a workgroup's duration
  const SeqInfo s = locate_chunk(blockIdx.x, cu, chunk_offsets, N, T_len);
  if (s.nvalid <= 0) return;
  const int tid = threadIdx.x, lane = tid & 63, l32 = lane & 31;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);   // wave-uniform: branches on it are scalar
  const int hq = blockIdx.y, grp = Hv / Hqk, nvalid = s.nvalid;
  const int64_t tok0 = s.bos + (int64_t)s.chunk * kChunk;
  const int ti = wave >> 1, tj = wave & 1, cj = wave;
  const bool lower = tj <= ti, has_k = wave < NKT, l2 = rstd_q != nullptr;
  const int nblk = V / 32;
  IdentityFrag<T> id;
  id.init();

  // One launch per value head of a q/k group (hh = 0 .. Hv/Hqk-1): the first writes dq and dk, the later ones add
  // to them in place, so no per-value-head copy of dq, dk ever exists.  The l2-norm backward
  // dx = (dy - <dy,y> y) / |x| is linear in dy and is applied to each head's contribution.
  const int h = hq * grp + hh;
  const int64_t ch = (int64_t)blockIdx.x * Hv + h;

  // every load below moves 64 x 16 bytes, lane l's piece landing at +16 l
  auto issue_shared = [&](int vblk) {                // v_new and dV' tiles of V block `vblk`
    T* st = stage0 + SM::sh + (vblk & 1) * 4096;
    const int64_t t2 = (ch * nblk + vblk) * 2;
#pragma unroll
    for (int j = 0; j < 4 * KG / 4; ++j) {           // k-group pieces dealt round-robin to the waves
      const int piece = 4 * j + wave, tile = piece / KG, g = piece % KG;
      const T* src = tile < 2 ? vf + (t2 + tile) * 1024 : dvf + (t2 + tile - 2) * 1024;
      load16_to_lds(src + (g * 64 + lane) * VEC, st + tile * 1024 + g * 64 * VEC);
    }
  };
  auto issue_priv = [&](int vblk) {                  // this wave's S and dS' tiles of V block `vblk`
    if (has_k) {
      T* pv = stage0 + SM::priv + wave * 2048;
      const int64_t tile = ((ch * nblk + vblk) * NKT + cj) * 1024;
#pragma unroll
      for (int g = 0; g < KG; ++g) {
        load16_to_lds(hf + tile + (g * 64 + lane) * VEC, pv + g * 64 * VEC);
        load16_to_lds(dhf_in + tile + (g * 64 + lane) * VEC, pv + 1024 + g * 64 * VEC);
      }
    }
  };
  auto issue_raw = [&](int pair) {                   // dO and V rows of V blocks 2 pair, 2 pair + 1; rows past the end repeat the last
    T* rb = stage0 + SM::raw + (pair & 1) * SM::raw_elems;
    constexpr int LPR = 64 / VEC, RPP = 64 / LPR;    // lanes per row, rows per 64-lane piece
#pragma unroll
    for (int j = 0; j < 64 / RPP / 4; ++j) {
      const int piece = 4 * j + wave, row = piece * RPP + lane / LPR, cc = SwizzledTile<T, 64>::pos(row, lane % LPR);
      const int64_t tok = tok0 + imin(row, nvalid - 1), col = (int64_t)h * V + 64 * pair + cc * VEC;
      load16_to_lds(dO + tok * Hv * V + col, rb + piece * 64 * VEC);
      load16_to_lds(v + tok * ts.v + col, rb + 64 * 64 + piece * 64 * VEC);
    }
  };
  // epilogue operands: all K tiles of the chunk into raw buffer `rbuf`, this wave's 32 columns of Q^T into its priv slot
  auto issue_epilogue = [&](int rbuf) {
    T* kt = stage0 + SM::raw + rbuf * SM::raw_elems;
#pragma unroll
    for (int j = 0; j < 2 * NKT * KG / 4; ++j) {
      const int piece = 4 * j + wave;
      load16_to_lds(kaf + ((int64_t)blockIdx.x * Hqk + hq) * (NKT * 2048) + (piece * 64 + lane) * VEC,
                    kt + piece * 64 * VEC);
    }
    if (has_k) {
#pragma unroll
      for (int piece = 0; piece < 2 * KG; ++piece)
        load16_to_lds(qtf + (((int64_t)blockIdx.x * Hqk + hq) * NKT + cj) * 2048 + (piece * 64 + lane) * VEC,
                      stage0 + SM::priv + wave * 2048 + piece * 64 * VEC);
    }
  };
#pragma unroll
  for (int j = 0; j < KG; ++j) {                      // Tm tiles, fragment order; tile (0,1) is zero, unused and not stored
    const int piece = 4 * j + wave;
    if (piece / KG != 1) load16_to_lds(Ai + ch * 4096 + (piece * 64 + lane) * VEC, TmF + piece * 64 * VEC);
  }
  issue_shared(0);
  issue_priv(0);
  issue_raw(0);

  if (tid < 64) {   // the row vectors: all requests first, the same ones on every path
    const int tc = imin(tid, nvalid - 1);
    const float gv = KDA ? 0.f : G[ch * 64 + tc], gl = KDA ? 0.f : G[ch * 64 + nvalid - 1];
    const uint32_t braw = gate_raw<T>(beta, beta_same, (tok0 + tc) * Hv + h);
    float rq1 = 1.f, rk1v = 1.f;
    if (l2) {
      rq1 = rstd_q[((int64_t)blockIdx.x * Hqk + hq) * 64 + tc];
      rk1v = rstd_k[((int64_t)blockIdx.x * Hqk + hq) * 64 + tc];
    }
    Gs[tid] = gv;
    egs[tid] = __expf(gv);
    sgs[tid] = scale * __expf(gv);
    egl[tid] = __expf(gl - gv);
    bs[tid] = tid < nvalid ? gate_val<T>(braw, beta_same) : 0.f;
    rsq[tid] = rq1;
    rsk[tid] = rk1v;
  }
  rq[tid] = 0.f; rk1[tid] = 0.f; rbk[tid] = 0.f; rf[tid] = 0.f; rv[tid] = 0.f;   // 256 threads, 256 entries each
  GDN_WAIT_VMEM();
  GDN_LDS_BARRIER();

  // Tm^T tile (a, b) as an A operand (lane <-> column of Tm, registers <-> row): the stored tile (b, a) turned round
  auto tm_t = [&](int a, int b) {
    AccB<T> f, o;
    f.load(TmF + (2 * b + a) * 1024);
    o.pack(mfma_transpose<T>(f, id));
    return o;
  };
  f32x16 ds = acc_zero(), a2 = acc_zero(), dQi[2], dKi[2], dWa[2];
#pragma unroll
  for (int ri = 0; ri < 2; ++ri) { dQi[ri] = acc_zero(); dKi[ri] = acc_zero(); dWa[ri] = acc_zero(); }
  float sds = 0.f;

  for (int vblk = 0; vblk < nblk; ++vblk) {
    const T* st = stage0 + SM::sh + (vblk & 1) * 4096;
    const T* rb = stage0 + SM::raw + ((vblk >> 1) & 1) * SM::raw_elems;
    const int rk0 = 32 * (vblk & 1);         // this block's columns inside the raw pair
    if (vblk > 0) {
      GDN_WAIT_VMEM();       // this wave's share of the block's operands has landed ...
      GDN_LDS_BARRIER();     // ... and so has everybody else's; the other stage and raw buffer are no longer read
    }
    // Operands are taken one after the other so that few fragments are live at a time; tile indices that depend on
    // the wave are compared against loop constants (fragments indexed at run time would go to scratch).
    AccB<T> f, Sf, dSf, dOt[2];
    if (has_k) {                             // (lane <-> K column, registers <-> V)
      f.load(stage0 + SM::priv + wave * 2048);
      const f32x16 sv = mfma_transpose<T>(f, id);
      Sf.pack(sv);
      f.load(stage0 + SM::priv + wave * 2048 + 1024);
      const f32x16 dsv = mfma_transpose<T>(f, id);
      dSf.pack(dsv);
#pragma unroll
      for (int r = 0; r < 16; ++r) sds += sv[r] * dsv[r];
    }
    GDN_WAVE_LDS_SYNC();     // the wave's priv slot is in registers: the next tenant may be requested
    if (vblk + 1 < nblk) {
      issue_shared(vblk + 1);
      issue_priv(vblk + 1);
      if ((vblk & 1) == 0 && vblk + 2 < nblk) issue_raw((vblk >> 1) + 1);   // its buffer was last read in block vblk - 1
    } else if constexpr (!KDA) {
      issue_epilogue(((vblk >> 1) + 1) & 1);
    }
#pragma unroll
    for (int ri = 0; ri < 2; ++ri) {         // (lane <-> token, registers <-> V) from here on; dO rows have it already
      SwizzledTile<T, 64>::frags(dOt[ri], rb, 32 * ri + l32, rk0);
      if (32 * ri + l32 >= nvalid) {
#pragma unroll
        for (int g = 0; g < KG; ++g) dOt[ri].f[g] = u32x4{0u, 0u, 0u, 0u};
      }
      if (has_k) mma32_ff<T>(dQi[ri], dOt[ri], Sf);
    }
#pragma unroll
    for (int ri = 0; ri < 2; ++ri) {
      AccB<T> Vt;
      f.load(st + ri * 1024);
      Vt.pack(mfma_transpose<T>(f, id));
      if (has_k) mma32_ff<T>(dKi[ri], Vt, dSf);
      if (lower && ri == tj) {
        // the dO fragments of this wave's token block, picked register by register (an indexed fragment would go to
        // scratch memory, a branch per block makes the compiler copy the accumulator between two places)
        AccB<T> dsel;
#pragma unroll
        for (int g = 0; g < KG; ++g)
#pragma unroll
          for (int e = 0; e < 4; ++e) dsel.f[g][e] = ti == 0 ? dOt[0].f[g][e] : dOt[1].f[g][e];
        mma32_ff<T>(ds, dsel, Vt);
      }
    }
#pragma unroll
    for (int ri = 0; ri < 2; ++ri) {
      AccB<T> dVt;
      f.load(st + (2 + ri) * 1024);
      dVt.pack(mfma_transpose<T>(f, id));
      if (has_k) mma32_ff<T>(dWa[ri], dVt, Sf);
      if (lower && ri == ti) {
        SwizzledTile<T, 64>::frags(f, rb + 64 * 64, 32 * tj + l32, rk0);
        mma32_ff<T>(a2, dVt, f);
      }
    }
    // dv = beta (Tm^T dV') of this V block.  The dV' tiles serve as they lie in
    // the stage, as the A operand: the product is dv^T (lane <-> token, registers <-> V column), of which every lane
    // stores four adjacent columns at a time without a detour through LDS.
    const int job = (wave - 2 * vblk) & 3;   // the two token halves of a block go to two waves, rotating with the block
    if (job < 2) {
      const int rj = job;
      f32x16 Rt = acc_zero();
      if (rj == 0) {
        f.load(st + 2 * 1024);
        mma32_ff<T>(Rt, f, tm_t(0, 0));
      }
      f.load(st + 3 * 1024);
      mma32_ff<T>(Rt, f, tm_t(rj, 1));
      const float bj = bs[32 * rj + l32];
#pragma unroll
      for (int r = 0; r < 16; ++r) Rt[r] *= bj;
      // (rows past the end repeat the last valid one: the half-waves trade pieces, so every lane takes part)
      T* dvrow = dv_out + (tok0 + imin(32 * rj + l32, nvalid - 1)) * ts.dv + h * V + 32 * vblk;
      if constexpr (sizeof(T) == 2) {
        if (32 * rj < nvalid) {   // wave-uniform
          const bool live = 32 * rj + l32 < nvalid;
          acc_store_t_rows16<T>(Rt, dvrow, live);
        }
      } else {
        if (32 * rj + l32 < nvalid) acc_to_lds_t<T>(Rt, dvrow, 0, 0, 0);
      }
    }
  }
  if constexpr (KDA) {
    constexpr int64_t kDumpElems = 3 * 64 * DK + 2 * 64 * 64;
    T* dump = kda_dump + ch * kDumpElems;
    GDN_WAIT_VMEM();
    GDN_LDS_BARRIER();   // the last block's stage is consumed: its place takes the store patches
    T* patch = stage0 + SM::sh + wave * Patch<T>::kElems;
    // dQb, dK2 and the two 64x64 sums leave as tiles in fragment order (the finish kernel wants them element by
    // element in the accumulator layout): tile (token block, channel block) resp. (row block, column block); P, which
    // it feeds to the matrix cores from LDS, as rows
    if (has_k) {
#pragma unroll
      for (int ri = 0; ri < 2; ++ri) {
        AccB<T> f;
        f.pack(dQi[ri]);
        f.store_stream(dump + (ri * NKT + cj) * 1024);
        f.pack(dKi[ri]);
        f.store_stream(dump + 64 * DK + (ri * NKT + cj) * 1024);
        acc_store_rows<T, false>(dWa[ri], id, patch, dump + 2 * 64 * DK + 32 * ri * DK + 32 * cj, DK, 32);
      }
      sds += __shfl_xor(sds, 32);   // the other half of the V block's rows
      if (lane < 32) kda_dd[ch * DK + 32 * cj + lane] = sds;
    }
    if (lower) {
      AccB<T> f;
      f.pack(ds);
      f.store_stream(dump + 3 * 64 * DK + (2 * ti + tj) * 1024);
      f.pack(a2);
      f.store_stream(dump + 3 * 64 * DK + 64 * 64 + (2 * ti + tj) * 1024);
    }
    return;
  }
  sds = wave_sum(sds);
  if (lane == 0) wsum[wave] = sds;
  const int rlast = ((nblk - 1) >> 1) & 1;               // raw buffer of the last pair
  T* EA = stage0 + SM::raw + (rlast ^ 1) * SM::raw_elems;   // K tiles
  T* EQ = stage0 + SM::priv;                             // Q columns per wave; later (beta dM) D-form tiles
  T* dWF = stage0 + SM::raw + rlast * SM::raw_elems;     // dW tiles, later the store patches
  T* tileD = stage0 + SM::sh;
  T* tileT = stage0 + SM::sh + 4096;
  T* dMD = EQ;
  GDN_WAIT_VMEM();
  GDN_LDS_BARRIER();   // the epilogue operands have landed; the last block's stage is consumed

  // this wave's K and Q columns as (lane <-> column, registers <-> token): B operands and row-dot partners
  AccB<T> KTf[2], QTf[2], dWb[2];
  if (has_k) {
#pragma unroll
    for (int t = 0; t < 2; ++t) {
      AccB<T> f;
      f.load(EA + (2 * cj + t) * 1024);
      KTf[t].pack(mfma_transpose<T>(f, id));
      QTf[t].load(EQ + wave * 2048 + t * 1024);
    }
#pragma unroll
    for (int ri = 0; ri < 2; ++ri) {         // dW = -(dV' S^T): B operand of P in registers, A operand of a1 to LDS
      dWb[ri].pack(dWa[ri]);
      dWb[ri].negate();      // the sign on the packed pairs: half as many instructions as on the sixteen values
      AccB<T> a;
      a.pack(mfma_transpose<T>(dWb[ri], id));
      a.store(dWF + (ri * NKT + cj) * 1024);
    }
  }
  {
    const int j = 32 * tj + acc_col();
    const float gj = Gs[j];
    const f32x16 gi = rows_ld(Gs, 32 * ti);
    // (every exponential first, then the selection: written as one conditional expression per entry the compiler
    // branches around each exponential and the sixteen chains run one after the other)
    float eg[16];
#pragma unroll
    for (int r = 0; r < 16; ++r) {
      eg[r] = __expf(fminf(gi[r] - gj, 0.f));
      GDN_KEEP_HERE(eg[r]);
    }
#pragma unroll
    for (int r = 0; r < 16; ++r) ds[r] = (32 * ti + acc_row(r) >= j) ? scale * ds[r] * eg[r] : 0.f;
    AccB<T> d, t;
    d.pack(ds);
    d.store(tileD + wave * 1024);
    t.pack(mfma_transpose<T>(d, id));
    t.store(tileT + wave * 1024);
  }
  GDN_LDS_BARRIER();
  float ski = 0.f;
  f32x16 pb[2];
  if (has_k) {
#pragma unroll
    for (int ri = 0; ri < 2; ++ri) {
      // the dQ half and the dK half one after the other: each unpacks its own partner rows, so that the two sets of
      // sixteen values are not alive together
      {
        const f32x16 fq = rows_ld(sgs, 32 * ri);
#pragma unroll
        for (int r = 0; r < 16; ++r) dQi[ri][r] *= fq[r];
        AccB<T> a;
#pragma unroll
        for (int t = 0; t <= ri; ++t) { a.load(tileT + (2 * ri + t) * 1024); mma32_ff<T>(dQi[ri], a, KTf[t]); }
        const f32x16 qq = QTf[ri].unpack();
        f32x16 p;
#pragma unroll
        for (int r = 0; r < 16; ++r) p[r] = dQi[ri][r] * qq[r];
        rows_add(p, rq, 32 * ri);
      }
      GDN_SCHED_FENCE();
      {
        const f32x16 fk = rows_ld(egl, 32 * ri), kk = KTf[ri].unpack();
#pragma unroll
        for (int r = 0; r < 16; ++r) {
          dKi[ri][r] *= fk[r];
          ski += dKi[ri][r] * kk[r];           // still only the inter-chunk part
        }
        AccB<T> a;
#pragma unroll
        for (int t = ri; t < 2; ++t) { a.load(tileD + (2 * t + ri) * 1024); mma32_ff<T>(dKi[ri], a, QTf[t]); }
        f32x16 p;
#pragma unroll
        for (int r = 0; r < 16; ++r) p[r] = dKi[ri][r] * kk[r];
        rows_add(p, rk1, 32 * ri);
      }
      GDN_SCHED_FENCE();
    }
  }
  ski = wave_sum(ski);
  if (lane == 0) wsum[4 + wave] = ski;
  if (has_k) {       // P = Tm^T dW; dK += beta e^G P; e^G <P,k> joins the dbeta / dG row sums
#pragma unroll
    for (int rj = 0; rj < 2; ++rj) {
      f32x16 P = acc_zero();
#pragma unroll
      for (int t = rj; t < 2; ++t) mma32_ff<T>(P, tm_t(rj, t), dWb[t]);
      const f32x16 kk = KTf[rj].unpack(), er = rows_ld(egs, 32 * rj), br = rows_ld(bs, 32 * rj);
#pragma unroll
      for (int r = 0; r < 16; ++r) {
        P[r] *= er[r];
        pb[rj][r] = P[r] * kk[r];
        dKi[rj][r] += P[r] * br[r];
      }
    }
  }
  GDN_LDS_BARRIER();   // the ds tiles are consumed
  // later value heads of a group add to the dq, dk rows the earlier ones wrote: what memory holds is requested well
  // ahead, dq here (no store is in flight), dk two phases before it is needed
  // Where the state gradient of a (chunk, head) has room for them (V >= 128: V K elements against 2 x 64 K), the sums
  // travel from one head's launch to the next as fragment-order tiles in that place, which this launch has finished
  // reading (the reverse recurrence rewrites it in every backward pass): no pass through rows, and only the group's
  // last head writes dq and dk.  Tiles: dq (token block, channel block), then dk likewise.
  const bool frag_sums = V >= 128 && grp > 1, last_head = hh == grp - 1;
  T* sums_out = const_cast<T*>(dhf_in) + ch * (int64_t)(V / 32) * NKT * 1024;
  const T* sums_in = sums_out - (int64_t)(V / 32) * NKT * 1024;   // the head before this one
  RowPieces<T> held[2];   // rows, or a tile in fragment order: one set of requests either way (rows_or_tile_request)
  if (has_k && hh != 0) {
#pragma unroll
    for (int ri = 0; ri < 2; ++ri)
      rows_or_tile_request<T>(held[ri], frag_sums, sums_in + (ri * NKT + cj) * 1024,
                              dq + (tok0 + 32 * ri) * ts.dq + hq * DK + 32 * cj, ts.dq, nvalid - 32 * ri);
  }
  if (lower) {  // <R_t, v_t> = sum_i Tm[i][t] (dV' V^T)[i][t]: column sums of Tm . a2, no second pass over V needed
    const f32x16 tmv = tm_t(tj, ti).unpack();   // Tm tile (ti, tj) with lane <-> column, registers <-> row
    float sv = 0.f;
#pragma unroll
    for (int r = 0; r < 16; ++r) sv += a2[r] * tmv[r];
    sv += __shfl_xor(sv, 32);
    if (lane < 32) rv[wave * 64 + 32 * tj + lane] += sv;
  }
  {  // dTm[i][j] = beta_j (e^{G_j} a1 + a2), i > j, handed on in T form; a1 = dW K^T over all of K (the dW tiles stay
     // in place until the store patches take their buffer behind the next barrier), a2 = dV' V^T from the main loop
    f32x16 a1 = acc_zero();
    if (lower) {
#pragma unroll
      for (int kt = 0; kt < NKT; ++kt) {
        AccB<T> a, b;
        a.load(dWF + (ti * NKT + kt) * 1024);
        b.load(EA + (2 * kt + tj) * 1024);
        mma32_ff<T>(a1, a, b);
      }
    }
    const int j = 32 * tj + acc_col();
    const float bj = bs[j], ej = egs[j];
#pragma unroll
    for (int r = 0; r < 16; ++r) a1[r] = (32 * ti + acc_row(r) > j) ? bj * (ej * a1[r] + a2[r]) : 0.f;
    AccB<T> d, t;
    d.pack(a1);
    t.pack(mfma_transpose<T>(d, id));
    t.store(tileT + wave * 1024);
  }
  // <q_i, dQ_i> once per row, for the l2-norm backward of dq behind the next barrier (instead of every lane adding
  // up the four slots for each of its sixteen rows)
  if (l2 && wave == 3) rqc[lane] = (rq[lane] + rq[64 + lane]) + (rq[128 + lane] + rq[192 + lane]);
  GDN_LDS_BARRIER();
  T* patch = dWF + wave * Patch<T>::kElems;
  if (has_k) {
#pragma unroll
    for (int ri = 0; ri < 2; ++ri) {
      if (l2) {
        const f32x16 qq = QTf[ri].unpack(), dot = rows_ld(rqc, 32 * ri), rs = rows_ld(rsq, 32 * ri);
#pragma unroll
        for (int r = 0; r < 16; ++r) dQi[ri][r] = (dQi[ri][r] - dot[r] * qq[r]) * rs[r];
      }
      T* dst = dq + (tok0 + 32 * ri) * ts.dq + hq * DK + 32 * cj;
      if (frag_sums) {
        if (hh != 0) {
          const f32x16 prev = as_frag<T>(held[ri]).unpack();
#pragma unroll
          for (int r = 0; r < 16; ++r) dQi[ri][r] += prev[r];
        }
        if (last_head) {
          acc_store_rows<T, false>(dQi[ri], id, patch, dst, ts.dq, nvalid - 32 * ri);
        } else {
          AccB<T> f;
          f.pack(dQi[ri]);
          f.store_stream(sums_out + (ri * NKT + cj) * 1024);
        }
      } else if (hh == 0) {
        acc_store_rows<T, false>(dQi[ri], id, patch, dst, ts.dq, nvalid - 32 * ri);
      } else {
        acc_store_rows<T, true>(dQi[ri], id, patch, dst, ts.dq, nvalid - 32 * ri, held[ri]);
      }
    }
  }
  {  // X = dTm Tm^T, handed on in D form
    f32x16 x = acc_zero();
    AccB<T> a, b;
    for (int t = 0; t <= imin(ti, tj); ++t) {
      a.load(tileT + (2 * ti + t) * 1024);
      b.load(TmF + (2 * tj + t) * 1024);
      mma32_ff<T>(x, a, b);
    }
    a.pack(x);
    a.store(tileD + wave * 1024);
  }
  GDN_LDS_BARRIER();
  if (lower) {  // dM = -(Tm^T X) . Gam, strictly lower: T form for dM K, D form scaled by beta_i for dM^T (beta K)
    f32x16 y = acc_zero();
    AccB<T> b;
    for (int m = ti; m < 2; ++m) {
      b.load(tileD + (2 * m + tj) * 1024);
      mma32_ff<T>(y, tm_t(ti, m), b);
    }
    int j = 32 * tj + acc_col();
    GDN_KEEP_HERE(j);   // recomputed here: the address of G_j from the first use, far above, would sit in a register (or in
                        // scratch memory) through the phases between
    const float gj = Gs[j];
    const f32x16 gi = rows_ld(Gs, 32 * ti), br = rows_ld(bs, 32 * ti);
    f32x16 yb;
#pragma unroll
    for (int r = 0; r < 16; ++r) {
      y[r] = (32 * ti + acc_row(r) > j) ? -y[r] * __expf(gi[r] - gj) : 0.f;
      yb[r] = y[r] * br[r];
    }
    AccB<T> d, t;
    d.pack(y);
    t.pack(mfma_transpose<T>(d, id));
    t.store(tileT + wave * 1024);
    d.pack(yb);
    d.store(dMD + wave * 1024);
  }
  GDN_LDS_BARRIER();
  if (has_k && hh != 0) {   // the dk sums of the earlier heads, two phases before they are added to
#pragma unroll
    for (int ri = 0; ri < 2; ++ri)
      rows_or_tile_request<T>(held[ri], frag_sums, sums_in + ((2 + ri) * NKT + cj) * 1024,
                              dk + (tok0 + 32 * ri) * ts.dk + hq * DK + 32 * cj, ts.dk, nvalid - 32 * ri);
  }
  if (has_k) {       // E = dM K, F = dM^T (beta K): dK += beta E + F; <E,k> and <F,k> complete the row sums
#pragma unroll
    for (int ri = 0; ri < 2; ++ri) {
      f32x16 E = acc_zero(), Fm = acc_zero(), p;
      AccB<T> a;
#pragma unroll
      for (int t = 0; t <= ri; ++t) { a.load(tileT + (2 * ri + t) * 1024); mma32_ff<T>(E, a, KTf[t]); }
#pragma unroll
      for (int t = ri; t < 2; ++t) { a.load(dMD + (2 * t + ri) * 1024); mma32_ff<T>(Fm, a, KTf[t]); }
      const f32x16 kk = KTf[ri].unpack(), br = rows_ld(bs, 32 * ri);
#pragma unroll
      for (int r = 0; r < 16; ++r) {
        pb[ri][r] += E[r] * kk[r];
        p[r] = Fm[r] * kk[r];
        dKi[ri][r] += E[r] * br[r] + Fm[r];
      }
      rows_add(pb[ri], rbk, 32 * ri);
      rows_add(p, rf, 32 * ri);
    }
  }
  GDN_LDS_BARRIER();   // the row sums are complete
  auto slots = [&](const float* a) { return (a[lane] + a[64 + lane]) + (a[128 + lane] + a[192 + lane]); };
  if (l2) {
    // <k_i, dK_i> = <k,dK1> + beta (e^G <P,k> + <E,k>) + <F,k>, once per row (e^G has served: its place takes it) instead
    // of the four slots of three arrays being added up by every lane for each of its sixteen rows
    if (wave == 1) egs[lane] = slots(rk1) + bs[lane] * slots(rbk) + slots(rf);
    GDN_LDS_BARRIER();
  }
  if (has_k) {
#pragma unroll
    for (int ri = 0; ri < 2; ++ri) {
      if (l2) {
        const f32x16 kk = KTf[ri].unpack(), dot = rows_ld(egs, 32 * ri), rs = rows_ld(rsk, 32 * ri);
#pragma unroll
        for (int r = 0; r < 16; ++r) dKi[ri][r] = (dKi[ri][r] - dot[r] * kk[r]) * rs[r];
      }
      T* dst = dk + (tok0 + 32 * ri) * ts.dk + hq * DK + 32 * cj;
      if (frag_sums) {
        if (hh != 0) {
          const f32x16 prev = as_frag<T>(held[ri]).unpack();
#pragma unroll
          for (int r = 0; r < 16; ++r) dKi[ri][r] += prev[r];
        }
        if (last_head) {
          acc_store_rows<T, false>(dKi[ri], id, patch, dst, ts.dk, nvalid - 32 * ri);
        } else {
          AccB<T> f;
          f.pack(dKi[ri]);
          f.store_stream(sums_out + ((2 + ri) * NKT + cj) * 1024);
        }
      } else if (hh == 0) {
        acc_store_rows<T, false>(dKi[ri], id, patch, dst, ts.dk, nvalid - 32 * ri);
      } else {
        acc_store_rows<T, true>(dKi[ri], id, patch, dst, ts.dk, nvalid - 32 * ri, held[ri]);
      }
    }
  }
  if (wave == 0) {   // d(cumulative G) -> d(g): suffix sum inside the chunk
    const float sbk = slots(rbk);
    float x = slots(rq) - slots(rk1) + bs[lane] * sbk - slots(rf);
    if (lane == nvalid - 1)
      x += __expf(Gs[63]) * (wsum[0] + wsum[1] + wsum[2] + wsum[3]) + (wsum[4] + wsum[5] + wsum[6] + wsum[7]);
#pragma unroll
    for (int d = 1; d < 64; d <<= 1) {
      const float t = __shfl_down(x, d);
      if (lane + d < 64) x += t;
    }
    if (lane < nvalid) {
      dg[(tok0 + lane) * Hv + h] = x;
      gate_st<T>(dbeta, beta_same, (tok0 + lane) * Hv + h, sbk + slots(rv));
    }
  }
}

// ---------------------------------------------------------------------------------------------
template <typename K> static int set_lds_b(K kernel, int bytes) {
  return (int)hipFuncSetAttribute(reinterpret_cast<const void*>(kernel), hipFuncAttributeMaxDynamicSharedMemorySize,
                                  bytes);
}

template <typename T, int DK, int NW, int NWS, int NLS, int STAGES>
static int chunk_bwd_launch(const ChunkDims& d, const ChunkWorkspace& L, const void* q, const void* k, const void* v,
                            const void* beta, int beta_same, const int64_t* cu, const void* dO, const float* dht, void* dq,
                            void* dk, void* dv, float* dg, void* dbeta, float* dh0, unsigned char* ws, unsigned char* ws_state,
                            int phases, float scale, int l2norm, hipStream_t st) {
  // ws, ws_state: bases of the workspace's prep part and state part (see ChunkWorkspace); phases: 2 = the reverse
  // recurrence, 4 = the chunk-local kernels
  const int nc = (int)d.max_chunks();
  const int* chunk_offsets = reinterpret_cast<const int*>(ws + L.chunk_offsets);
  (void)q; (void)k;   // q and k reach the backward kernels as the forward pass's fragment tiles
  const float* G = reinterpret_cast<const float*>(ws + L.G);
  const T* Ai = reinterpret_cast<const T*>(ws + L.Ai);
  const T* AQ = reinterpret_cast<const T*>(ws + L.AQ);
  const T* VF = reinterpret_cast<const T*>(ws_state + L.VF);
  const T* HF = reinterpret_cast<const T*>(ws_state + L.HF);
  const T* QTF = reinterpret_cast<const T*>(ws + L.QTF);
  const T* KAF = reinterpret_cast<const T*>(ws + L.KAF);
  T* DVF = reinterpret_cast<T*>(ws_state + L.DVF);
  T* DHF = reinterpret_cast<T*>(ws_state + L.DHF);
  const float* rstd_q = l2norm ? reinterpret_cast<const float*>(ws + L.rstd) : nullptr;
  const float* rstd_k = l2norm ? rstd_q + (int64_t)nc * 64 * d.Hqk : nullptr;
  if (phases & 2) {
    auto kern = chunk_state_bwd_kernel<T, DK, NWS, NLS, STAGES>;
    constexpr int smem = StateBwdSmem<T, DK, NWS, STAGES>::bytes;
    if (int e = set_lds_b(kern, smem)) return e;
    GDN_LAUNCH(kKernStateBwd, st, kern, dim3(d.N * d.Hv, d.V / (32 * NWS)), dim3(64 * (NWS + NLS)), smem, st, (const T*)KAF,
               (const T*)nullptr, (const T*)QTF, Ai, AQ, (const T*)dO, G, beta, beta_same, dht, dh0, DVF, DHF, cu, chunk_offsets, d.T, d.Hqk, d.Hv, d.V,
               scale);
  }
  if (phases & 4) {
    const TokenStrides gs = d.strides();
    const int es = (int)sizeof(T), bb = beta_same ? es : 4;
    TailRows tail{{dq, dk, dv, dg, dbeta}, {gs.dq * es, gs.dk * es, gs.dv * es, (int64_t)d.Hv * 4, (int64_t)d.Hv * bb},
                  {d.Hqk * DK * es, d.Hqk * DK * es, d.Hv * d.V * es, d.Hv * 4, d.Hv * bb}};
    launch_zero_tail_rows(cu, d.N, d.tokens(), tail, st);
    auto kern = chunk_bwd_local_kernel<T, DK>;
    constexpr int smem = BwdLocalSmem<T, DK>::bytes;
    if (int e = set_lds_b(kern, smem)) return e;
    for (int hh = 0; hh < d.Hv / d.Hqk; ++hh)
      GDN_LAUNCH(kKernBwdLocal, st, kern, dim3(nc, d.Hqk), dim3(kThreads), smem, st, QTF, (const T*)KAF, (const T*)v,
                 beta, beta_same, G, Ai, VF, (const T*)DVF, (const T*)dO, HF, (const T*)DHF, rstd_q, rstd_k, (T*)dq, (T*)dk,
                 (T*)dv, dbeta, dg, cu, chunk_offsets, d.T, d.N, d.Hqk, d.Hv, d.V, scale, hh, d.strides(), (T*)nullptr, (float*)nullptr,
                 device_compute_units());
  }
  return (int)hipGetLastError();
}

}  // namespace gdn

namespace gdn {
// phases: 1 = refill the state part from the prep part (prep itself first unless prep_valid), 2 = the reverse recurrence,
// 4 = the chunk-local kernels.  workspace_state null: one buffer holds both parts.
static int chunk_bwd_entry(const void* q, const void* k, const void* v, int64_t q_stride, int64_t k_stride, int64_t v_stride,
                           const float* g, const void* beta, const float* initial_state, const int64_t* cu_seqlens,
                           const void* d_o, const float* d_final_state, void* dq, void* dk, void* dv, int64_t dq_stride,
                           int64_t dk_stride, int64_t dv_stride, float* dg, void* dbeta, float* d_initial_state,
                           void* workspace, int64_t workspace_bytes, void* workspace_state, int64_t workspace_state_bytes,
                           int phases, int prep_valid, bool share_device, int B, int T, int N, int Hqk, int Hv, int K, int V,
                           float scale, int use_qk_l2norm, int dtype, int beta_dtype, void* stream) {
  if (!q || !k || !v || !beta || !workspace) return -1;
  if ((phases & 6) && !d_o) return -1;
  if ((phases & 4) && (!dq || !dk || !dv || !dg || !dbeta)) return -1;
  if ((phases & ~7) || phases == 0) return -2;
  ChunkDims d{B, T, N, Hqk, Hv, K, V, cu_seqlens != nullptr};
  d.ts = {q_stride, k_stride, v_stride, dq_stride, dk_stride, dv_stride};
  if (int e = chunk_check_dims(d, dtype)) return e;
  if (beta_dtype != 0 && beta_dtype != dtype) return -4;
  const int beta_same = beta_dtype != 0;
  if (((uintptr_t)q | (uintptr_t)k | (uintptr_t)v | (uintptr_t)d_o | (uintptr_t)dq | (uintptr_t)dk | (uintptr_t)dv) & 15) return -6;
  ChunkDims dl = d;
  dl.varlen = true;
  const ChunkWorkspace L = chunk_workspace_layout(dl, dtype == 0 ? 4 : 2);
  unsigned char* ws = static_cast<unsigned char*>(workspace);
  unsigned char* ws_state = ws;
  if (workspace_state != nullptr) {
    if (workspace_bytes < L.prep_bytes || workspace_state_bytes < L.total_bytes - L.prep_bytes) return -5;
    if ((reinterpret_cast<uintptr_t>(workspace_state) & 255) != 0) return -5;
    ws_state = static_cast<unsigned char*>(workspace_state) - L.prep_bytes;
  } else if (workspace_bytes < L.total_bytes) {
    return -5;
  }
  if ((reinterpret_cast<uintptr_t>(workspace) & 255) != 0) return -5;
  hipStream_t st = (hipStream_t)stream;
  if (phases & 1) {
    if (!g) return -1;
    if (workspace_state == nullptr && prep_valid) return -1;   // one buffer is always refilled whole
    if (int e = chunk_fwd_entry(q, k, v, q_stride, k_stride, v_stride, g, beta, beta_dtype, initial_state, cu_seqlens, nullptr,
                                nullptr, workspace, workspace_bytes, B, T, N, Hqk, Hv, K, V, scale, use_qk_l2norm, dtype,
                                FwdNorm{}, stream, workspace_state, workspace_state_bytes, prep_valid != 0, share_device))
      return e;
    if (!(phases & 6)) return 0;
  }
#define GDN_BWD(T_, DK_, NW_, NWS_, NLS_, ST_)                                                       \
  return chunk_bwd_launch<T_, DK_, NW_, NWS_, NLS_, ST_>(d, L, q, k, v, beta, beta_same, cu_seqlens, d_o, d_final_state, dq, \
                                                          dk, dv, dg, dbeta, d_initial_state, ws, ws_state, phases, scale, \
                                                          use_qk_l2norm, st)
  const bool wide = (V % 128 == 0);
  const bool solo = one_slab_per_workgroup(d, device_compute_units()) &&
                    !(share_device && two_slabs_to_share_device(d, device_compute_units()));
  if (dtype == 1) {
    if (K == 128 && wide && solo) GDN_BWD(bf16_t, 128, 4, 1, 4, 2);
    if (K == 128 && wide) GDN_BWD(bf16_t, 128, 4, 2, 4, 2);
    if (K == 128) GDN_BWD(bf16_t, 128, 2, 2, 2, 2);
    if (wide) GDN_BWD(bf16_t, 64, 4, 2, 2, 2);
    GDN_BWD(bf16_t, 64, 2, 2, 2, 2);
  } else {
    if (K == 128) GDN_BWD(float, 128, 2, 2, 2, 1);
    GDN_BWD(float, 64, 2, 2, 2, 1);
  }
#undef GDN_BWD
}
}  // namespace gdn

extern "C" int gdn_chunk_bwd_strided(const void* q, const void* k, const void* v, int64_t q_stride, int64_t k_stride,
                                     int64_t v_stride, const float* g, const void* beta, const float* initial_state,
                                     const int64_t* cu_seqlens, const void* d_o, const float* d_final_state, void* dq,
                                     void* dk, void* dv, int64_t dq_stride, int64_t dk_stride, int64_t dv_stride,
                                     float* dg, void* dbeta, float* d_initial_state, void* workspace,
                                     int64_t workspace_bytes, int B, int T, int N, int Hqk, int Hv, int K, int V,
                                     float scale, int use_qk_l2norm, int dtype, int beta_dtype, void* stream) {
  (void)g; (void)initial_state;   // their effect is already in the workspace (G, per-chunk states)
  return gdn::chunk_bwd_entry(q, k, v, q_stride, k_stride, v_stride, g, beta, initial_state, cu_seqlens, d_o, d_final_state,
                              dq, dk, dv, dq_stride, dk_stride, dv_stride, dg, dbeta, d_initial_state, workspace,
                              workspace_bytes, nullptr, 0, 6, 1, false, B, T, N, Hqk, Hv, K, V, scale, use_qk_l2norm, dtype,
                              beta_dtype, stream);
}

extern "C" int gdn_chunk_bwd_parts(const void* q, const void* k, const void* v, int64_t q_stride, int64_t k_stride,
                                   int64_t v_stride, const float* g, const void* beta, const float* initial_state,
                                   const int64_t* cu_seqlens, const void* d_o, const float* d_final_state, void* dq,
                                   void* dk, void* dv, int64_t dq_stride, int64_t dk_stride, int64_t dv_stride, float* dg,
                                   void* dbeta, float* d_initial_state, void* workspace_prep, int64_t workspace_prep_bytes,
                                   void* workspace_state, int64_t workspace_state_bytes, int phases, int prep_valid, int B,
                                   int T, int N, int Hqk, int Hv, int K, int V, float scale, int use_qk_l2norm, int dtype,
                                   int beta_dtype, void* stream) {
  if (!workspace_state) return -1;
  return gdn::chunk_bwd_entry(q, k, v, q_stride, k_stride, v_stride, g, beta, initial_state, cu_seqlens, d_o, d_final_state,
                              dq, dk, dv, dq_stride, dk_stride, dv_stride, dg, dbeta, d_initial_state, workspace_prep,
                              workspace_prep_bytes, workspace_state, workspace_state_bytes, phases, prep_valid, true, B, T, N,
                              Hqk, Hv, K, V, scale, use_qk_l2norm, dtype, beta_dtype, stream);
}

extern "C" int gdn_chunk_bwd(const void* q, const void* k, const void* v, const float* g, const float* beta,
                             const float* initial_state, const int64_t* cu_seqlens, const void* d_o,
                             const float* d_final_state, void* dq, void* dk, void* dv, float* dg, float* dbeta,
                             float* d_initial_state, void* workspace, int64_t workspace_bytes, int B, int T, int N,
                             int Hqk, int Hv, int K, int V, float scale, int use_qk_l2norm, int dtype, void* stream) {
  return gdn_chunk_bwd_strided(q, k, v, 0, 0, 0, g, beta, initial_state, cu_seqlens, d_o, d_final_state, dq, dk, dv, 0, 0,
                               0, dg, dbeta, d_initial_state, workspace, workspace_bytes, B, T, N, Hqk, Hv, K, V, scale,
                               use_qk_l2norm, dtype, 0, stream);
}

#include "gdn_kda_bwd.h"
