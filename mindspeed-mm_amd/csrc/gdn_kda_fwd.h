// KDA (Kimi delta attention) forward: the gated delta rule with one decay per key channel,
//     S <- diag(e^{g_t}) S;  S <- S + beta_t k_t (v_t - S^T k_t)^T;  o_t = scale S^T q_t
// (reference: mindspeed_mm/fsdp/ops/kda/chunk_kda_naive.py:106-221, operator entry :223-381, gate :76-104).
// Included at the end of gdn_chunk_fwd.hip: the recurrence and the output product are that file's kernels
// (chunk_state_kernel in its KDA mode, whose output waves form O from an image of q that already carries scale and
// decay; where a workgroup serves two slabs of the state, or in fp32, chunk_out_kernel forms O from the stored states
// instead); this file adds the chunk-local preparation, which is where the per-channel decay changes the algebra, and
// the entry points.
//
// Per chunk, with G the chunk-local cumulative log decay [64, K]:
//     L_ij  = beta_i sum_d k_id k_jd e^{G_id - G_jd}   (i > j)       Tm = (I + L)^-1
//     Aq_ij = scale sum_d q_id k_jd e^{G_id - G_jd}    (i >= j)
//     V' = Tm beta (v - (k . e^G) S)      O = (scale q . e^G) S + Aq V'      S <- e^{G_last} . S + (k . e^{G_last-G})^T V'
// e^{G_i - G_j} does not factor over a whole chunk without overflow (e^{-G_j} is unbounded).  It does factor safely
// for a pair (i, j) that straddles a point m, j < m <= i: e^{G_i-G_m} e^{G_m-G_j}, both factors at most 1.  Halving the
// chunk recursively (blocks of 64, 32, ..., 2 tokens, m the middle of the block) puts every pair i > j into exactly one
// such block at one level, where i lies in the second half and j in the first.  So per level every row is rescaled
// once, x_r e^{-|G_r - G_m|} with m the middle of its block, the 32x32 tile products run on the matrix cores, and of
// each product only the entries of that level are kept; the diagonal i = j needs no decay at all.  The rescaled rows
// are built in registers, straight into the operand layout, so nothing but k, q and G occupies LDS.
#pragma once
#include "gdn_kda_common.h"

namespace gdn {

template <typename T, int DK> struct KdaPrepSmem {
  static constexpr int LDK = lds_ld<T>(DK), LDG = DK + 4, L64 = lds_ld<T>(64);
  static constexpr int tile = 64 * LDK * (int)sizeof(T), gmat = 64 * LDG * 4, amat = 64 * kLF * 4;
  static constexpr int off_ks = 0, off_qs = off_ks + tile, off_gs = off_qs + tile;   // k, q rows (T), G rows (fp32)
  static constexpr int off_misc = off_gs + gmat;         // beta [64], partial totals of the cumulative sum [4][DK]
  static constexpr int off_tm = off_misc + (64 + 4 * DK) * 4;   // the inverse in operand precision, row-major
  static constexpr int end0 = off_tm + 64 * L64 * (int)sizeof(T);
  // L, Aq and the inverse (fp32 64 x kLF each) take the place of k, q and G once those are dead; where a region is too
  // small for its tenant the tenant moves behind everything else
  static constexpr bool wide = tile >= amat;             // K = 128
  static constexpr int off_as = off_ks;                                  // K = 64: spans the k and q rows
  static constexpr int off_aq = wide ? off_qs : off_gs;
  static constexpr int off_ti = wide ? off_gs : end0;
  static constexpr int bytes = wide ? end0 : end0 + amat;
  static_assert(wide ? gmat >= amat : (2 * tile >= amat && gmat >= amat), "tenants fit");
  static_assert(bytes <= 160 * 1024, "one CU's LDS");
};

template <typename T, int DK>
__global__ __launch_bounds__(kThreads) GDN_WAVES_PER_SIMD(2) void kda_prep_kernel(
    const T* __restrict__ q, const T* __restrict__ k, const void* __restrict__ g, const void* __restrict__ beta,
    const float* __restrict__ A_log, const float* __restrict__ dt_bias, const int64_t* __restrict__ cu,
    const int* __restrict__ chunk_offsets, float* __restrict__ bhat_out, float* __restrict__ dec_out,
    T* __restrict__ Ai_out, T* __restrict__ Aq_out, T* __restrict__ K1_out,
    T* __restrict__ K2_out, T* __restrict__ QB_out, T* __restrict__ QBT_out, T* __restrict__ TMR_out,
    float* __restrict__ rstd_q_out, float* __restrict__ rstd_k_out,
    int T_len, int N, int H, float scale, KdaFlags fl) {
  using SM = KdaPrepSmem<T, DK>;
  constexpr int LDK = SM::LDK, LDG = SM::LDG, VEC = Elem<T>::kVec, CPR = DK / VEC;
  T* Ks = reinterpret_cast<T*>(gdn_smem + SM::off_ks);
  T* Qs = reinterpret_cast<T*>(gdn_smem + SM::off_qs);
  float* Gs = reinterpret_cast<float*>(gdn_smem + SM::off_gs);
  float* bs = reinterpret_cast<float*>(gdn_smem + SM::off_misc);
  float* tot = bs + 64;
  float* As = reinterpret_cast<float*>(gdn_smem + SM::off_as);
  float* Aqs = reinterpret_cast<float*>(gdn_smem + SM::off_aq);
  float* Ti = reinterpret_cast<float*>(gdn_smem + SM::off_ti);
  T* Tms = reinterpret_cast<T*>(gdn_smem + SM::off_tm);

  const SeqInfo s = locate_chunk(blockIdx.x, cu, chunk_offsets, N, T_len);
  if (s.nvalid <= 0) return;
  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);   // wave-uniform: branches and offsets from it are scalar
  const int h = blockIdx.y, nvalid = s.nvalid;
  const int64_t tok0 = s.bos + (int64_t)s.chunk * kChunk, hk = (int64_t)H * DK;
  const int64_t ch = (int64_t)blockIdx.x * H + h;

  // ---- phase 0: requests first: the gate input (4 channels per piece; loads arrive in the order of their requests
  //      and the gate is what the workgroup computes first), then k and q rows, beta ----
  TileQK<T, DK> kt, qt;
  constexpr int GP = 64 * (DK / 4) / kThreads;
  const bool g32 = sizeof(T) == 4 || fl.g_f32;
  // as bits, and with one branch around each whole round of requests: a conversion or a test between two loads would
  // make each of them wait for the one before
  u32x4 gw[GP];
  f32x4 bv[GP];
  if (g32) {
#pragma unroll
    for (int i = 0; i < GP; ++i) {
      const int c = tid + i * kThreads, row = imin(c / (DK / 4), nvalid - 1), c4 = c % (DK / 4);
      gw[i] = *reinterpret_cast<const u32x4*>(reinterpret_cast<const uint32_t*>(g) + (tok0 + row) * hk + h * DK + 4 * c4);
    }
  } else {
#pragma unroll
    for (int i = 0; i < GP; ++i) {
      const int c = tid + i * kThreads, row = imin(c / (DK / 4), nvalid - 1), c4 = c % (DK / 4);
      const u32x2 x = *reinterpret_cast<const u32x2*>(reinterpret_cast<const uint16_t*>(g) + (tok0 + row) * hk + h * DK + 4 * c4);
      gw[i][0] = x[0]; gw[i][1] = x[1];   // the other two stay unset: unread on this path, and zeros here made the
                                          // fp32 path wait at the join for its requests
    }
  }
  if (fl.use_gate && dt_bias != nullptr) {
#pragma unroll
    for (int i = 0; i < GP; ++i) bv[i] = *reinterpret_cast<const f32x4*>(dt_bias + h * DK + 4 * ((tid + i * kThreads) % (DK / 4)));
  } else {
#pragma unroll
    for (int i = 0; i < GP; ++i) { bv[i][0] = 0.f; bv[i][1] = 0.f; bv[i][2] = 0.f; bv[i][3] = 0.f; }
  }
  tile_qk_request<T, DK>(kt, k + tok0 * hk + h * DK, hk, nvalid, tid);
  tile_qk_request<T, DK>(qt, q + tok0 * hk + h * DK, hk, nvalid, tid);
  // beta: requested by every wave alike (a branch around the request would make its wave wait at the join for all of
  // the requests above), as bits; used behind the gate
  const int64_t beta_at = (tok0 + imin(lane, nvalid - 1)) * H + h;
  uint32_t beta_bits;
  if (sizeof(T) == 4 || fl.beta_f32) beta_bits = reinterpret_cast<const uint32_t*>(beta)[beta_at];
  else beta_bits = reinterpret_cast<const uint16_t*>(beta)[beta_at];
  // the gate: log decay of every token and channel, 0 on the rows past the end (they leave the cumulative sum alone)
  {
    const float a = fl.use_gate ? __expf(A_log[h]) : 0.f;
    const float au = a * KdaDecay<T>::kUnit, lbu = fl.lower_bound * KdaDecay<T>::kUnit;   // in the units G is kept in
    // MODE 0: g is the log decay itself; 1: -e^{A_log} softplus(g + bias); 2: lower_bound sigmoid(e^{A_log} (g + bias)).
    // One copy of the loop per mode: a test of the options per element would cost as much as the gate.
    auto gate_rows = [&](auto mode) {
      constexpr int MODE = decltype(mode)::value;
#pragma unroll
      for (int i = 0; i < GP; ++i) {
        const int c = tid + i * kThreads, row = c / (DK / 4), c4 = c % (DK / 4);
        f32x4 y;
#pragma unroll
        for (int e = 0; e < 4; ++e) {
          const float x = __uint_as_float(g32 ? gw[i][e] : (gw[i][e >> 1] >> (16 * (e & 1))) << 16);
          y[e] = row < nvalid ? kda_gate<T, MODE>(x, bv[i][e], a, au, lbu) : 0.f;
        }
        *reinterpret_cast<f32x4*>(Gs + row * LDG + 4 * c4) = y;
      }
    };
    if (!fl.use_gate) gate_rows(IntConst<0>());
    else if (!fl.has_lower_bound) gate_rows(IntConst<1>());
    else gate_rows(IntConst<2>());
  }
  if (wave == 0) {
    float b = __uint_as_float(beta_bits);
    if constexpr (sizeof(T) == 2) {
      if (!fl.beta_f32) { T t; t.bits = (uint16_t)beta_bits; b = Elem<T>::to_f(t); }
    }
    if (fl.beta_sigmoid) b = kda_sigmoid(b) * (fl.beta_x2 ? 2.f : 1.f);
    bs[lane] = lane < nvalid ? b : 0.f;
    if (lane < nvalid) bhat_out[beta_at] = b;
  }
  {
    const int64_t roff = ch * 64;
    tile_qk_finish<T, DK>(kt, Ks, LDK, nvalid, tid, fl.l2norm != 0, nullptr, 0, rstd_k_out ? rstd_k_out + roff : nullptr, 1);
    tile_qk_finish<T, DK>(qt, Qs, LDK, nvalid, tid, fl.l2norm != 0, nullptr, 0, rstd_q_out ? rstd_q_out + roff : nullptr, 1);
  }
  GDN_LDS_BARRIER();
  // cumulative sum down the tokens, a thread per channel and part of the chunk, then the totals of the parts before it
  {
    constexpr int PARTS = kThreads / DK, RPP = 64 / PARTS;
    const int d = tid % DK, part = tid / DK;
    kda_cumsum_part<DK, LDG, PARTS>(Gs, tot, tid);
    GDN_LDS_BARRIER();
    const float off = kda_cumsum_before<DK, PARTS>(tot, part, d);
    if (part > 0) {
#pragma unroll
      for (int r = 0; r < RPP; ++r) Gs[(part * RPP + r) * LDG + d] += off;
    }
  }
  GDN_LDS_BARRIER();

  // ---- phase 1: L and Aq level by level on the matrix cores.  Wave w: diagonal tile w >> 1 of both matrices (k k^T and
  //      q k^T share every rescaling factor, the costly part) over half w & 1 of the channel groups; the tile below
  //      the diagonal (level 64) goes to waves 0 and 1.  The halves are added in phase 1d. ----
  const int kh = wave & 1, td = wave >> 1, l32 = lane & 31, half = lane >> 5;
  constexpr int KGL = KGroup<T>::kLen, NKG = DK / KGL, NKH = NKG / 2;
  static_assert(NKG % 2 == 0, "two halves of the channel groups");
  const int R = 32 * td + l32;
  // the levels' entries, each kept where its level owns the pair: tile (td, td) of k k^T and of q k^T, and the tile below
  f32x16 dgk = acc_zero(), dgq = acc_zero(), lowk = acc_zero(), lowq = acc_zero();
  // One pass over this wave's channel groups for the levels [I0, I0 + NI) (blocks of 2 << level tokens), all of them
  // advancing together: the rows of k, q and G are read once per group and only the reference row of G differs from
  // level to level; the products of the levels are independent chains.  Two passes (three levels and the undecayed
  // diagonal of q k^T, then two levels and level 64): the accumulators of all levels of both matrices at once would
  // not fit the registers that two workgroups per CU leave a wave.
  auto level_pass = [&](auto i0_c, auto ni_c, auto diag_c, auto low_c) {
    constexpr int I0 = decltype(i0_c)::value, NI = decltype(ni_c)::value;
    constexpr bool DIAG = decltype(diag_c)::value != 0, LOW = decltype(low_c)::value != 0;
    f32x16 ak[NI], aq[NI], adg = acc_zero();
#pragma unroll
    for (int i = 0; i < NI; ++i) { ak[i] = acc_zero(); aq[i] = acc_zero(); }
#pragma unroll 1
    for (int kg = kh * NKH; kg < (kh + 1) * NKH; ++kg) {
      const int c0 = kg * KGL + half * VEC;
      float fk[VEC], fq[VEC], gR[VEC];
      unpack16<T>(ld16(Ks + R * LDK + c0), fk);
      unpack16<T>(ld16(Qs + R * LDK + c0), fq);
      ld_f32<VEC>(Gs + R * LDG + c0, gR);
      if (DIAG) mfma_kgroup<T>(adg, pack16<T>(fq).raw, pack16<T>(fk).raw);   // the diagonal of q k^T: no decay
#pragma unroll
      for (int i = 0; i < NI; ++i) {   // rows of the second half of a block against rows of its first half
        const int n = 2 << (I0 + i), m = (R / n) * n + n / 2;
        float gm[VEC], xq[VEC], xk[VEC];
        ld_f32<VEC>(Gs + m * LDG + c0, gm);
#pragma unroll
        for (int e = 0; e < VEC; ++e) {
          const float f = KdaDecay<T>::exp(-fabsf(gR[e] - gm[e]));
          xq[e] = fq[e] * f;
          xk[e] = fk[e] * f;
        }
        const u32x4 bK = pack16<T>(xk).raw;
        mfma_kgroup<T>(ak[i], bK, bK);
        mfma_kgroup<T>(aq[i], pack16<T>(xq).raw, bK);
      }
      if (LOW && wave < 2) {   // level 64: tokens 32..63 against 0..31 (these waves' rows R), all entries kept
        float gm[VEC], ga[VEC], xk2[VEC], xq2[VEC], xb[VEC];
        ld_f32<VEC>(Gs + 32 * LDG + c0, gm);
        ld_f32<VEC>(Gs + (32 + l32) * LDG + c0, ga);
        unpack16<T>(ld16(Ks + (32 + l32) * LDK + c0), xk2);
        unpack16<T>(ld16(Qs + (32 + l32) * LDK + c0), xq2);
#pragma unroll
        for (int e = 0; e < VEC; ++e) {
          const float fa = KdaDecay<T>::exp(-fabsf(ga[e] - gm[e]));
          xk2[e] *= fa;
          xq2[e] *= fa;
          xb[e] = fk[e] * KdaDecay<T>::exp(-fabsf(gR[e] - gm[e]));
        }
        const u32x4 bK = pack16<T>(xb).raw;
        mfma_kgroup<T>(lowk, pack16<T>(xk2).raw, bK);
        mfma_kgroup<T>(lowq, pack16<T>(xq2).raw, bK);
      }
    }
#pragma unroll
    for (int r = 0; r < 16; ++r) {
      const int i = acc_row(r), j = l32;
#pragma unroll
      for (int q2 = 0; q2 < NI; ++q2) {
        const int n = 2 << (I0 + q2);
        const bool keep = (i / n == j / n) && (i % n >= n / 2) && (j % n < n / 2);
        dgk[r] += keep ? ak[q2][r] : 0.f;
        dgq[r] += keep ? aq[q2][r] : 0.f;
      }
      if (DIAG) dgq[r] += i == j ? adg[r] : 0.f;
    }
  };
  level_pass(IntConst<0>(), IntConst<3>(), IntConst<1>(), IntConst<0>());
  level_pass(IntConst<3>(), IntConst<2>(), IntConst<0>(), IntConst<1>());
  GDN_LDS_BARRIER();   // every wave is done with q as it lies: its place becomes the staging tile

  // ---- phase 1c: what the recurrence reads, in fragment order: the two K images and (scale q . e^{G})^T ----
  if (QB_out == nullptr) {
    // Straight from the rows in LDS into the registers of an A operand (lane <-> token, 4 consecutive channels per
    // piece, frag_a_split's order): e^{G} serves q and the first K image, nothing is staged and no barrier is needed.
    // The q tiles are turned by a pass through the matrix core (exact) into (lane <-> channel, registers <-> token).
    constexpr int KG = AccK<T>::kGroups, GL = KGroup<T>::kLen, NP = sizeof(T) == 2 ? 2 : 1;
    IdentityFrag<T> id;
    id.init();
    for (int tt = wave; tt < 2 * (DK / 32); tt += 4) {
      const int tj = tt & 1, kt2 = tt >> 1, row = 32 * tj + l32;
      const float nb = -bs[row];
      AccB<T> f1, f2, fq;
#pragma unroll
      for (int kg = 0; kg < KG; ++kg) {
        float x1[4 * NP], x2[4 * NP], xq[4 * NP];
#pragma unroll
        for (int pc = 0; pc < NP; ++pc) {
          const int c = 32 * kt2 + GL * kg + 4 * half + 8 * pc;
          float k4[4], q4[4];
          if constexpr (sizeof(T) == 2) {
            const u32x2 kw = *reinterpret_cast<const u32x2*>(Ks + row * LDK + c), qw = *reinterpret_cast<const u32x2*>(Qs + row * LDK + c);
#pragma unroll
            for (int e = 0; e < 2; ++e) {
              k4[2 * e] = __uint_as_float(kw[e] << 16); k4[2 * e + 1] = __uint_as_float(kw[e] & 0xffff0000u);
              q4[2 * e] = __uint_as_float(qw[e] << 16); q4[2 * e + 1] = __uint_as_float(qw[e] & 0xffff0000u);
            }
          } else {
            const f32x4 kw = *reinterpret_cast<const f32x4*>(Ks + row * LDK + c), qw = *reinterpret_cast<const f32x4*>(Qs + row * LDK + c);
#pragma unroll
            for (int e = 0; e < 4; ++e) { k4[e] = kw[e]; q4[e] = qw[e]; }
          }
          const f32x4 g4 = *reinterpret_cast<const f32x4*>(Gs + row * LDG + c), gl4 = *reinterpret_cast<const f32x4*>(Gs + 63 * LDG + c);
#pragma unroll
          for (int e = 0; e < 4; ++e) {
            const float eg = KdaDecay<T>::exp(g4[e]);
            x1[4 * pc + e] = k4[e] * (nb * eg);      // the products in the order of the staged path below: same bits
            x2[4 * pc + e] = k4[e] * KdaDecay<T>::exp(gl4[e] - g4[e]);
            xq[4 * pc + e] = q4[e] * (scale * eg);
          }
        }
        if constexpr (sizeof(T) == 2) {
#pragma unroll
          for (int e = 0; e < 4; ++e) {
            f1.f[kg][e] = f32x2_to_bf16x2(x1[2 * e], x1[2 * e + 1]);
            f2.f[kg][e] = f32x2_to_bf16x2(x2[2 * e], x2[2 * e + 1]);
            fq.f[kg][e] = f32x2_to_bf16x2(xq[2 * e], xq[2 * e + 1]);
          }
        } else {
#pragma unroll
          for (int e = 0; e < 4; ++e) {
            f1.f[kg][e] = __float_as_uint(x1[e]); f2.f[kg][e] = __float_as_uint(x2[e]); fq.f[kg][e] = __float_as_uint(xq[e]);
          }
        }
      }
      const int64_t tile = ((ch * (DK / 32) + kt2) * 2 + tj) * 1024;
      f1.store_stream(K1_out + tile);
      f2.store_stream(K2_out + tile);
      if (QBT_out != nullptr) {
        AccB<T> qt2;
        qt2.pack(mfma_transpose<T>(fq, id));
        qt2.store_stream(QBT_out + tile);
      }
    }
  } else {
    // with the rows of q also wanted as rows (the stand-alone output kernel): through a row-major staging tile (the q
    // rows' place): rows of q with scale and decay first (in place), then the two K images
    for (int c = tid; c < 64 * CPR; c += kThreads) {
      const int row = c / CPR, cc = c % CPR;
      float f[VEC], gi[VEC];
      unpack16<T>(ld16(Qs + row * LDK + cc * VEC), f);
      ld_f32<VEC>(Gs + row * LDG + cc * VEC, gi);
#pragma unroll
      for (int e = 0; e < VEC; ++e) f[e] *= scale * KdaDecay<T>::exp(gi[e]);
      const Vec16<T> x = pack16<T>(f);
      if (row < nvalid) st16(QB_out + (tok0 + row) * hk + h * DK + cc * VEC, x);   // row-major for the output kernel
      st16(Qs + row * LDK + cc * VEC, x);
    }
    if (QBT_out != nullptr) {   // transposed tiles for a backward pass
      GDN_LDS_BARRIER();
      for (int tt = wave; tt < 2 * (DK / 32); tt += 4) {
        const int tj = tt & 1, kt2 = tt >> 1;
        AccB<T> kf;
        kf.load_cols(Qs + 32 * tj * LDK + 32 * kt2, LDK);
        kf.store_stream(QBT_out + ((ch * (DK / 32) + kt2) * 2 + tj) * 1024);
      }
    }
    auto stage_k = [&](bool first) {
      for (int c = tid; c < 64 * CPR; c += kThreads) {
        const int row = c / CPR, cc = c % CPR;
        float f[VEC], gi[VEC], gl[VEC];
        unpack16<T>(ld16(Ks + row * LDK + cc * VEC), f);
        ld_f32<VEC>(Gs + row * LDG + cc * VEC, gi);
        ld_f32<VEC>(Gs + 63 * LDG + cc * VEC, gl);
        const float nb = -bs[row];
#pragma unroll
        for (int e = 0; e < VEC; ++e) f[e] *= first ? nb * KdaDecay<T>::exp(gi[e]) : KdaDecay<T>::exp(gl[e] - gi[e]);
        st16(Qs + row * LDK + cc * VEC, pack16<T>(f));
      }
    };
    auto store_k = [&](T* out) {
      for (int tt = wave; tt < 2 * (DK / 32); tt += 4) {
        const int tj = tt & 1, kt2 = tt >> 1;
        AccB<T> kf;
        frags_from_lds<T>(kf, Qs + (32 * tj + (lane & 31)) * LDK + 32 * kt2);
        kf.store_stream(out + ((ch * (DK / 32) + kt2) * 2 + tj) * 1024);
      }
    };
    GDN_LDS_BARRIER();
    stage_k(true);
    GDN_LDS_BARRIER();
    store_k(K1_out);
    GDN_LDS_BARRIER();
    stage_k(false);
    GDN_LDS_BARRIER();
    store_k(K2_out);
  }
  // the decay of the whole chunk per channel (the cumulative decay itself is not kept: the backward pass rebuilds it
  // from the gate input, which it reads anyway)
  if (tid < DK) dec_out[ch * DK + tid] = KdaDecay<T>::exp(Gs[63 * LDG + tid]);
  GDN_LDS_BARRIER();   // k, the staging tile and G are dead

  // ---- phase 1d: L and Aq as 64x64 fp32 matrices ----
  // Zeroed: the place of the inverse, and the tile above the diagonal of both matrices; every other entry is written by
  // the first of the two waves that share a tile (one per half of the channels), then the second adds its half.  A wave
  // reads all of its entries, then adds, then writes: entry by entry each read would wait for the write before it (the
  // compiler must assume that the two matrices overlap).
  static_assert(kLF % 4 == 0, "rows of the fp32 matrices are whole 16-byte pieces");
  for (int i = tid; i < 64 * kLF / 4; i += kThreads) reinterpret_cast<f32x4*>(Ti)[i] = f32x4{0.f, 0.f, 0.f, 0.f};
  for (int i = tid; i < 32 * 8; i += kThreads) {
    const int at = (i >> 3) * kLF + 32 + 4 * (i & 7);
    *reinterpret_cast<f32x4*>(As + at) = f32x4{0.f, 0.f, 0.f, 0.f};
    *reinterpret_cast<f32x4*>(Aqs + at) = f32x4{0.f, 0.f, 0.f, 0.f};
  }
  if (kh == 0) {
    const f32x16 bi = rows_ld(bs, 32 * td);
#pragma unroll
    for (int r = 0; r < 16; ++r) {
      const int i = 32 * td + acc_row(r), j = 32 * td + l32;
      As[i * kLF + j] = i > j ? bi[r] * dgk[r] : 0.f;
      Aqs[i * kLF + j] = i >= j ? scale * dgq[r] : 0.f;
    }
    if (wave < 2) {   // the tile below the diagonal
      const f32x16 bl = rows_ld(bs, 32);
#pragma unroll
      for (int r = 0; r < 16; ++r) {
        const int i2 = 32 + acc_row(r);
        As[i2 * kLF + l32] = bl[r] * lowk[r];
        Aqs[i2 * kLF + l32] = scale * lowq[r];
      }
    }
  }
  GDN_LDS_BARRIER();
  if (kh == 1) {
    float ca[16], cq[16];
    const f32x16 bi = rows_ld(bs, 32 * td);
#pragma unroll
    for (int r = 0; r < 16; ++r) {
      const int i = 32 * td + acc_row(r), j = 32 * td + l32;
      ca[r] = As[i * kLF + j];
      cq[r] = Aqs[i * kLF + j];
    }
    GDN_SCHED_FENCE();
#pragma unroll
    for (int r = 0; r < 16; ++r) {
      const int i = 32 * td + acc_row(r), j = 32 * td + l32;
      As[i * kLF + j] = ca[r] + (i > j ? bi[r] * dgk[r] : 0.f);
      Aqs[i * kLF + j] = cq[r] + (i >= j ? scale * dgq[r] : 0.f);
    }
    if (wave < 2) {   // the tile below the diagonal
      const f32x16 bl = rows_ld(bs, 32);
#pragma unroll
      for (int r = 0; r < 16; ++r) {
        const int i2 = 32 + acc_row(r);
        ca[r] = As[i2 * kLF + l32];
        cq[r] = Aqs[i2 * kLF + l32];
      }
      GDN_SCHED_FENCE();
#pragma unroll
      for (int r = 0; r < 16; ++r) {
        const int i2 = 32 + acc_row(r);
        As[i2 * kLF + l32] = ca[r] + bl[r] * lowk[r];
        Aqs[i2 * kLF + l32] = cq[r] + scale * lowq[r];
      }
    }
  }
  GDN_LDS_BARRIER();
  if (wave != 1) {  // Aq leaves as tiles packed as they sit in an accumulator (lane <-> column j, registers <-> row i);
                    // tile (0,1) is zero, is read by no kernel and is not written
    const int ti = wave >> 1, tj = wave & 1;
    f32x16 aq;
#pragma unroll
    for (int r = 0; r < 16; ++r) aq[r] = Aqs[(32 * ti + acc_row(r)) * kLF + 32 * tj + acc_col()];
    AccB<T> af;
    af.pack(aq);
    af.store_stream(Aq_out + (ch * 4 + wave) * 1024);
  }
  tril_inverse_64(As, Ti, wave, lane);
  store_tm_tiles<T>(Ti, Tms, Ai_out + ch * 4096, tid, wave, lane);
  if (TMR_out != nullptr) {   // the staging tile holds Tm row-major in operand precision
    constexpr int C64 = 64 / VEC;
    for (int c = tid; c < 64 * C64; c += kThreads)
      st16(TMR_out + ch * 4096 + (c / C64) * 64 + (c % C64) * VEC, ld16(Tms + (c / C64) * SM::L64 + (c % C64) * VEC));
  }
}

// NWO: waves of the output kernel's workgroup; NWS, NLS, STAGES: slabs, loader waves and LDS stages of the recurrence
template <typename T, int DK, int NWO, int NWS, int NLS, int STAGES>
static int kda_fwd_launch(const ChunkDims& d, const KdaWorkspace& L, const void* q, const void* k, const void* v,
                          const void* g, const void* beta, const float* A_log, const float* dt_bias, const float* h0,
                          const int64_t* cu, void* o, float* ht, unsigned char* ws, float scale, const KdaFlags& fl,
                          bool with_backward, hipStream_t st) {
  const int H = d.Hv;
  const int nc = (int)d.max_chunks();
  int* chunk_offsets = reinterpret_cast<int*>(ws + L.chunk_offsets);
  float* rstd = reinterpret_cast<float*>(ws + L.rstd);
  float* bhat = reinterpret_cast<float*>(ws + L.bhat);
  float* dec = reinterpret_cast<float*>(ws + L.dec);
  T* Ai = reinterpret_cast<T*>(ws + L.Ai);
  T* AQ = reinterpret_cast<T*>(ws + L.AQ);
  T* K1F = reinterpret_cast<T*>(ws + L.K1F);
  T* K2F = reinterpret_cast<T*>(ws + L.K2F);
  // Where one slab per workgroup is the choice and the K, Q and Aq images of two stages fit the LDS beside the slab's
  // state, the recurrence kernel's own output waves write O and the stand-alone output kernel is not launched.
  constexpr bool FUSE = NWS == 1 && STAGES == 2 && sizeof(T) == 2;
  T* QB = FUSE ? nullptr : reinterpret_cast<T*>(ws + L.QB);
  T* VF = reinterpret_cast<T*>(ws + L.VF);
  T* HF = reinterpret_cast<T*>(ws + L.HF);
  T* QBT = (with_backward || FUSE) ? reinterpret_cast<T*>(ws + L.QBT) : nullptr;
  T* TMR = with_backward ? reinterpret_cast<T*>(ws + L.TMR) : nullptr;
  if (cu != nullptr) GDN_LAUNCH(kKernChunkTable, st, chunk_table_kernel, dim3(1), dim3(kThreads), 0, st, cu, chunk_offsets, d.N);
  {
    const int64_t ob = (int64_t)H * d.V * (int)sizeof(T);
    TailRows tail{{o}, {ob}, {(int)ob}};
    launch_zero_tail_rows(cu, d.N, d.tokens(), tail, st);
  }
  {
    auto kern = kda_prep_kernel<T, DK>;
    constexpr int smem = KdaPrepSmem<T, DK>::bytes;
    if (int e = set_lds(kern, smem)) return e;
    const bool keep = with_backward && fl.l2norm;
    GDN_LAUNCH(kKernKdaPrep, st, kern, dim3(nc, H), dim3(kThreads), smem, st, (const T*)q, (const T*)k, g, beta, A_log,
               dt_bias, cu, (const int*)chunk_offsets, bhat, dec, Ai, AQ, K1F, K2F, QB, QBT, TMR, keep ? rstd : nullptr,
               keep ? rstd + (int64_t)nc * 64 * H : nullptr, d.T, d.N, H, scale, fl);
  }
  if constexpr (FUSE) {
    auto kern = chunk_state_kernel<T, DK, NWS, NLS, STAGES, true, true, true>;
    constexpr int smem = StateSmem<T, DK, NWS, STAGES, true, true, true>::bytes;
    if (int e = set_lds(kern, smem)) return e;
    // the per-chunk states and v_new leave the kernel only for a backward pass
    GDN_LAUNCH(kKernStateFwd, st, kern, dim3(d.N * H, d.V / (32 * NWS)), dim3(64 * (NWS * (1 + StateOutWaves<NWS>::value) + NLS)),
               smem, st, (const T*)K1F, (const T*)K2F, (const T*)Ai, (const T*)AQ, (const T*)v, (const float*)dec,
               (const void*)bhat, 0, h0, ht, with_backward ? VF : (T*)nullptr, with_backward ? HF : (T*)nullptr, (T*)o, cu,
               (const int*)chunk_offsets, d.T, H, H, d.V, scale, (int64_t)H * d.V, (const T*)QBT);
    return (int)hipGetLastError();
  }
  {
    auto kern = chunk_state_kernel<T, DK, NWS, NLS, STAGES, false, true, true>;
    constexpr int smem = StateSmem<T, DK, NWS, STAGES, false, true, true>::bytes;
    if (int e = set_lds(kern, smem)) return e;
    GDN_LAUNCH(kKernStateFwd, st, kern, dim3(d.N * H, d.V / (32 * NWS)), dim3(64 * (NWS + NLS)), smem, st, (const T*)K1F,
               (const T*)K2F, (const T*)Ai, (const T*)AQ, (const T*)v, (const float*)dec, (const void*)bhat, 0, h0, ht, VF, HF,
               (T*)nullptr, cu, (const int*)chunk_offsets, d.T, H, H, d.V, scale, (int64_t)H * d.V, (const T*)nullptr);
  }
  {
    auto kern = chunk_out_kernel<T, DK, NWO, false, T>;
    constexpr int smem = OutSmem<T, DK, NWO>::bytes;
    if (int e = set_lds(kern, smem)) return e;
    GDN_LAUNCH(kKernOut, st, kern, dim3(nc, H, d.V / (32 * NWO)), dim3(64 * NWO), smem, st, (const T*)QB, (const T*)AQ,
               (const T*)VF, (const T*)HF, (const float*)nullptr, (T*)o, cu, (const int*)chunk_offsets, d.T, d.N, H, H, d.V,
               scale, (int64_t)H * DK, (const float*)nullptr, OutNorm<T, T>{});
  }
  return (int)hipGetLastError();
}

}  // namespace gdn

namespace gdn {
// chunk_kda(..., return_intermediate_states=True) (chunk_kda_naive.py:287-303, :375-380): the state at the entry of
// every chunk.  The recurrence left it in the workspace as fragment-order tiles (lane <-> V column, registers <-> K
// row, tile (V block, K block) of chunk and head at ((ch * V/32 + vb) * K/32 + kt) * 1024); here it is written out as
// [chunks, H, K, V] or, transposed, [chunks, H, V, K] in the operand type.  One workgroup per (chunk, head), the tiles
// dealt to its four waves.
template <typename T>
__global__ __launch_bounds__(kThreads) void kda_states_out_kernel(const T* __restrict__ hf, T* __restrict__ out,
                                                                 const int64_t* __restrict__ cu,
                                                                 const int* __restrict__ chunk_offsets, int N, int T_len,
                                                                 int H, int K, int V, int transposed, int64_t out_chunks) {
  const SeqInfo s = locate_chunk(blockIdx.x, cu, chunk_offsets, N, T_len);
  if (s.nvalid <= 0 || (int64_t)blockIdx.x >= out_chunks) return;
  const int wave = threadIdx.x >> 6, nkt = K / 32, nvb = V / 32;
  const int64_t ch = (int64_t)blockIdx.x * H + blockIdx.y;
  T* dst = out + ch * K * V;
  IdentityFrag<T> id;
  id.init();
  T* patch = reinterpret_cast<T*>(gdn_smem) + wave * Patch<T>::kElems;
  for (int t = wave; t < nkt * nvb; t += kThreads / 64) {
    const int vb = t / nkt, kt = t % nkt;
    AccB<T> f;
    f.load(hf + (ch * nvb * nkt + t) * 1024);
    const f32x16 c = f.unpack();
    if (transposed) acc_to_lds_t<T>(c, dst, K, 32 * kt, 32 * vb);
    else acc_store_rows<T, false>(c, id, patch, dst + (int64_t)32 * kt * V + 32 * vb, V, 32);
  }
}

template <typename T>
static int kda_states_out_launch(const ChunkDims& d, const KdaWorkspace& L, const unsigned char* ws, const int64_t* cu,
                                 void* out, int64_t out_chunks, int transposed, hipStream_t st) {
  const int smem = 4 * Patch<T>::kElems * (int)sizeof(T);
  hipLaunchKernelGGL(kda_states_out_kernel<T>, dim3((unsigned)d.max_chunks(), d.Hv), dim3(kThreads), smem, st,
                     reinterpret_cast<const T*>(ws + L.HF), static_cast<T*>(out), cu,
                     reinterpret_cast<const int*>(ws + L.chunk_offsets), d.N, d.T, d.Hv, d.K, d.V, transposed, out_chunks);
  return (int)hipGetLastError();
}
}  // namespace gdn

extern "C" int gdn_kda_intermediate_states(const void* workspace, int64_t workspace_bytes, const int64_t* cu_seqlens,
                                           void* h_out, int64_t h_chunks, int B, int T, int N, int H, int K, int V,
                                           int transpose_state_layout, int dtype, void* stream) {
  using namespace gdn;
  if (!workspace || !h_out) return -1;
  ChunkDims d{B, T, N, H, H, K, V, cu_seqlens != nullptr};
  if (int e = chunk_check_dims(d, dtype)) return e;
  if (h_chunks < 0) return -2;
  if ((uintptr_t)h_out & 15) return -6;
  ChunkDims dl = d;
  dl.varlen = true;
  const KdaWorkspace L = kda_workspace_layout(dl, dtype == 0 ? 4 : 2);
  // the recurrence keeps the per-chunk states only in a workspace of the size that serves a backward pass
  if (workspace_bytes < L.total_bytes || (reinterpret_cast<uintptr_t>(workspace) & 255) != 0) return -5;
  if (h_chunks == 0) return 0;
  const unsigned char* ws = static_cast<const unsigned char*>(workspace);
  hipStream_t st = (hipStream_t)stream;
  if (dtype == 1) return kda_states_out_launch<bf16_t>(d, L, ws, cu_seqlens, h_out, h_chunks, transpose_state_layout, st);
  return kda_states_out_launch<float>(d, L, ws, cu_seqlens, h_out, h_chunks, transpose_state_layout, st);
}

extern "C" int64_t gdn_kda_workspace_bytes(int B, int T, int N, int H, int K, int V, int with_backward, int dtype) {
  gdn::ChunkDims d{B, T, N, H, H, K, V, true};   // the packed bound is the larger
  const gdn::KdaWorkspace w = gdn::kda_workspace_layout(d, dtype == 0 ? 4 : 2);
  return with_backward ? w.total_bytes : w.fwd_bytes;
}

extern "C" int gdn_kda_fwd(const void* q, const void* k, const void* v, const void* g, const void* beta,
                           const float* A_log, const float* dt_bias, const float* initial_state,
                           const int64_t* cu_seqlens, void* o, float* final_state, void* workspace,
                           int64_t workspace_bytes, int B, int T, int N, int H, int K, int V, float scale,
                           int use_qk_l2norm, int use_gate, int has_lower_bound, float lower_bound, int beta_sigmoid,
                           int allow_neg_eigval, int dtype, int g_dtype, int beta_dtype, void* stream) {
  using namespace gdn;
  if (!q || !k || !v || !g || !beta || !o || !workspace) return -1;
  if (use_gate && !A_log) return -1;
  ChunkDims d{B, T, N, H, H, K, V, cu_seqlens != nullptr};
  if (int e = chunk_check_dims(d, dtype)) return e;
  if ((g_dtype != 0 && g_dtype != dtype) || (beta_dtype != 0 && beta_dtype != dtype)) return -4;
  if (((uintptr_t)q | (uintptr_t)k | (uintptr_t)v | (uintptr_t)g | (uintptr_t)o) & 15) return -6;
  ChunkDims dl = d;
  dl.varlen = true;
  const KdaWorkspace L = kda_workspace_layout(dl, dtype == 0 ? 4 : 2);
  if (workspace_bytes < L.fwd_bytes || (reinterpret_cast<uintptr_t>(workspace) & 255) != 0) return -5;
  const bool with_bwd = workspace_bytes >= L.total_bytes;
  KdaFlags fl{use_qk_l2norm, use_gate, has_lower_bound, beta_sigmoid, allow_neg_eigval, g_dtype == 0, beta_dtype == 0, lower_bound};
  unsigned char* ws = static_cast<unsigned char*>(workspace);
  hipStream_t st = (hipStream_t)stream;
#define GDN_KDA(T_, DK_, NWO_, NWS_, NLS_, ST_)                                                                          \
  return kda_fwd_launch<T_, DK_, NWO_, NWS_, NLS_, ST_>(d, L, q, k, v, g, beta, A_log, dt_bias, initial_state, cu_seqlens, o, \
                                                        final_state, ws, scale, fl, with_bwd, st)
  // a CU per 32-column slab of the state while there are no more slabs than CUs (see one_slab_per_workgroup)
  const bool one_slab = one_slab_per_workgroup(d, device_compute_units());
  if (dtype == 1) {
    if (K == 128) {
      if (one_slab) GDN_KDA(bf16_t, 128, 2, 1, 4, 2);
      GDN_KDA(bf16_t, 128, 2, 2, 4, 2);
    }
    GDN_KDA(bf16_t, 64, 2, 2, 4, 2);
  } else {
    if (K == 128) GDN_KDA(float, 128, 2, 2, 2, 1);
    GDN_KDA(float, 64, 2, 2, 2, 2);
  }
#undef GDN_KDA
}
