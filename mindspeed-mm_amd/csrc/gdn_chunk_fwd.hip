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

// (I + A)^-1 of a strictly lower triangular 64x64 matrix.  A arrives in As (fp32, leading dimension kLF; its upper
// triangle is used as scratch), the inverse is left in Ti, which must arrive zeroed.  All four waves; the last thing
// it does is a barrier.
__device__ __forceinline__ void tril_inverse_64(float* As, float* Ti, int wave, int lane) {
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

}

// The inverse as four 32x32 A-operand tiles in operand precision (lane <-> row, registers <-> column), through the
// row-major staging tile Tms [64][lds_ld<T>(64)].
template <typename T>
__device__ __forceinline__ void store_tm_tiles(const float* Ti, T* Tms, T* tiles_out, int tid, int wave, int lane) {
  constexpr int L64 = lds_ld<T>(64), VEC = Elem<T>::kVec;
  // ---- phase 3: Tm in operand precision, as four 32x32 A-operand tiles (lane <-> row, registers <-> column) ----
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
  {
    // tile (0,1) of a lower triangular matrix is zero: no kernel reads it, and it is not written
    if (wave != 1) {
      AccB<T> tf;
      frags_from_lds<T>(tf, Tms + (32 * (wave >> 1) + (lane & 31)) * L64 + 32 * (wave & 1));
      tf.store_stream(tiles_out + wave * 1024);
    }
  }
}

// ---------------------------------------------------------------------------------------------
// chunk_prep_kernel: what is independent across chunks and does not involve v.
//   G (cumulative decay), Tm = (I+L)^-1, Aq = scale tril(Q K^T . Gam), and per q/k group the K and Q^T tiles, all in
//   fragment order (AccB<>): 16 bytes per lane per k-group, copied straight to LDS by the recurrence kernels.
// W = Tm (beta e^G K) and U = Tm (beta V) are never formed: the recurrence applies Tm to beta (v - e^G K S) itself.
// One workgroup per (chunk, q/k group): q and k are loaded and normalised, and the products k.k and q.k formed, once
// for the group; its value heads, which differ in decay and beta only, follow one after the other (mask, Aq tiles,
// the 64x64 inverse).
// Its barriers order LDS traffic only (GDN_LDS_BARRIER): a __syncthreads() would also wait until every store issued
// so far has been acknowledged.
// ---------------------------------------------------------------------------------------------
template <typename T, int DK> struct PrepSmem {
  static constexpr int LDK = lds_ld<T>(DK), L64 = lds_ld<T>(64);
  static constexpr int cmax(int a, int b) { return a > b ? a : b; }
  // Two regions, each reused once its tenant is dead, so that four workgroups (bf16) fit a CU's LDS:
  //   region 1: K tile -> Tm (fp32, solve output)
  //   region 2: Q tile -> A (fp32, solve input) -> Tm in T
  static constexpr int off_ks = 0;
  static constexpr int r1_bytes = cmax(64 * LDK * (int)sizeof(T), 64 * kLF * 4);
  static constexpr int off_qs = off_ks + r1_bytes;
  static constexpr int qs_bytes = cmax(cmax(64 * LDK * (int)sizeof(T), 64 * kLF * 4), 64 * L64 * (int)sizeof(T));
  static constexpr int off_ti = off_ks;
  static constexpr int off_misc = off_qs + qs_bytes;
  static constexpr int bytes = off_misc + 2 * 64 * 4;            // plus as much per further value head of the group
  static int launch_bytes(int heads_per_group) { return bytes + (heads_per_group - 1) * 2 * 64 * 4; }
};

template <typename T, int DK>
__global__ __launch_bounds__(kThreads) GDN_WAVES_PER_SIMD(sizeof(T) == 2 ? 4 : 3) void chunk_prep_kernel(
    const T* __restrict__ q, const T* __restrict__ k, const float* __restrict__ g, const void* __restrict__ beta,
    int beta_same, const int64_t* __restrict__ cu, const int* __restrict__ chunk_offsets, float* __restrict__ G_out,
    T* __restrict__ Ai_out, T* __restrict__ Aq_out, T* __restrict__ KA_out, T* __restrict__ QT_out,
    float* __restrict__ rstd_q_out, float* __restrict__ rstd_k_out, int T_len, int N, int Hqk, int Hv, float scale,
    int l2norm, TokenStrides ts) {
  using SM = PrepSmem<T, DK>;
  constexpr int LDK = SM::LDK, L64 = SM::L64, VEC = Elem<T>::kVec;
  T* Ks = reinterpret_cast<T*>(gdn_smem + SM::off_ks);
  T* Qs = reinterpret_cast<T*>(gdn_smem + SM::off_qs);
  float* As = reinterpret_cast<float*>(gdn_smem + SM::off_qs);    // after Q
  T* Tms = reinterpret_cast<T*>(gdn_smem + SM::off_qs);          // after A
  float* Ti = reinterpret_cast<float*>(gdn_smem + SM::off_ti);   // after K
  float* Gs = reinterpret_cast<float*>(gdn_smem + SM::off_misc);   // per value head of the group: G [64], beta [64]

  const SeqInfo s = locate_chunk(blockIdx.x, cu, chunk_offsets, N, T_len);
  if (s.nvalid <= 0) return;
  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);   // wave-uniform: branches and offsets from it are scalar
  const int hq = blockIdx.y, grp = Hv / Hqk, nvalid = s.nvalid;
  const int64_t tok0 = s.bos + (int64_t)s.chunk * kChunk;

  // ---- phase 0: K and Q tiles of the q/k group; cumulative decay (one lane per token) and beta of each of its value
  //      heads, a wave per head.  All requests first: the gate values of the wave's first head (every wave and lane
  //      asks alike, for a place that exists; inside the loop over heads the request would come behind a wait for the
  //      tiles), then the tiles. ----
  const int64_t tokl = tok0 + imin(lane, nvalid - 1);
  const int64_t at0 = tokl * Hv + hq * grp + imin(wave, grp - 1);
  const float g_first = g[at0];
  const uint32_t b_first = gate_raw<T>(beta, beta_same, at0);
  TileQK<T, DK> kt, qt;
  tile_qk_request<T, DK>(kt, k + tok0 * ts.k + hq * DK, ts.k, nvalid, tid);
  tile_qk_request<T, DK>(qt, q + tok0 * ts.q + hq * DK, ts.q, nvalid, tid);
  auto head_gates = [&](int hh, float graw, uint32_t braw) {
    const int h = hq * grp + hh;
    float x = lane < nvalid ? graw : 0.f;
    const float b = lane < nvalid ? gate_val<T>(braw, beta_same) : 0.f;
#pragma unroll
    for (int d = 1; d < 64; d <<= 1) {
      const float t = __shfl_up(x, d);
      if (lane >= d) x += t;
    }
    Gs[hh * 128 + lane] = x;
    Gs[hh * 128 + 64 + lane] = b;
    G_out[((int64_t)blockIdx.x * Hv + h) * 64 + lane] = x;   // 64 contiguous values per chunk and head
  };
  if (wave < grp) head_gates(wave, g_first, b_first);
  for (int hh = wave + 4; hh < grp; hh += 4) {
    const int64_t at = tokl * Hv + hq * grp + hh;
    const float graw = g[at];
    head_gates(hh, graw, gate_raw<T>(beta, beta_same, at));
  }
  {
    // q and k arrive raw; with the in-kernel l2 norm they are normalised on the way into LDS, and 1/|q|, 1/|k| are left
    // for the output kernel, which scales q itself, and the backward pass
    const int64_t roff = ((int64_t)blockIdx.x * Hqk + hq) * 64;   // 64 contiguous values per chunk and q/k head
    tile_qk_finish<T, DK>(kt, Ks, LDK, nvalid, tid, l2norm != 0, nullptr, 0, l2norm ? rstd_k_out + roff : nullptr, 1);
    tile_qk_finish<T, DK>(qt, Qs, LDK, nvalid, tid, l2norm != 0, nullptr, 0, l2norm ? rstd_q_out + roff : nullptr, 1);
  }
  GDN_LDS_BARRIER();

  // ---- phase 1: the products k_i.k_j and q_i.k_j, one 32x32 tile per wave, once for the group: the value heads
  //      differ in decay and beta only ----
  const int ti = wave >> 1, tj = wave & 1;
  f32x16 kk_raw = acc_zero(), qk_raw = acc_zero();
  if (tj <= ti) {
    mma32<T, DK, true, true>(kk_raw, Ks + 32 * ti * LDK, LDK, Ks + 32 * tj * LDK, LDK);
    mma32<T, DK, true, true>(qk_raw, Qs + 32 * ti * LDK, LDK, Ks + 32 * tj * LDK, LDK);
  }
  // K (lane <-> token, registers <-> K column) and Q^T (lane <-> K column, registers <-> token) as A-operand fragments,
  // once per q/k group; the recurrence kernels read each of them both as it lies and transposed
  for (int tt = wave; tt < 2 * (DK / 32); tt += 4) {
    const int tjj = tt & 1, ktt = tt >> 1;
    const int64_t gtile = ((((int64_t)blockIdx.x * Hqk + hq) * (DK / 32) + ktt) * 2 + tjj) * 1024;
    AccB<T> kf;
    frags_from_lds<T>(kf, Ks + (32 * tjj + (lane & 31)) * LDK + 32 * ktt);
    kf.store_stream(KA_out + gtile);
    kf.load_cols(Qs + 32 * tjj * LDK + 32 * ktt, LDK);
    kf.store_stream(QT_out + gtile);
  }
  GDN_LDS_BARRIER();   // Q and K are consumed: their space takes A and Tm

  // ---- per value head: A = strict_tril(beta_i k_i.k_j Gam_ij), Aq = scale tril(q_i.k_j Gam_ij), Tm = (I + A)^-1 ----
#pragma clang loop unroll(disable)
  for (int hh = 0; hh < grp; ++hh) {
    const int h = hq * grp + hh;
    const float* Gh = Gs + hh * 128;
    const float* bh = Gh + 64;
    {
      const int j = 32 * tj + acc_col();
      const float gj = Gh[j];
      const f32x16 gi = rows_ld(Gh, 32 * ti), bi = rows_ld(bh, 32 * ti);
      f32x16 aq;
#pragma unroll
      for (int r = 0; r < 16; ++r) {   // branch-free: where the mask discards the value the exponent is set to 0 first
        const int i = 32 * ti + acc_row(r);
        const float e = __expf(i >= j ? gi[r] - gj : 0.f);
        const float gam = i >= j ? e : 0.f;
        As[i * kLF + j] = i > j ? bi[r] * kk_raw[r] * gam : 0.f;
        aq[r] = qk_raw[r] * (gam * scale);
      }
      // scale tril(Q K^T . Gam) leaves as 32x32 tiles in fragment order, packed as they sit in the accumulator
      // (lane <-> column j, registers <-> row i): the A operand of Aq^T dO as is, of Aq V' read transposed
      // (tile (0,1) is zero, is read by no kernel and is not written)
      if (wave != 1) {
        AccB<T> af;
        af.pack(aq);
        af.store_stream(Aq_out + (((int64_t)blockIdx.x * Hv + h) * 4 + wave) * 1024);
      }
    }
    static_assert(kLF % 4 == 0, "rows of the fp32 matrices are whole 16-byte pieces");
    for (int i = tid; i < 64 * kLF / 4; i += kThreads) reinterpret_cast<f32x4*>(Ti)[i] = f32x4{0.f, 0.f, 0.f, 0.f};
    GDN_LDS_BARRIER();

    tril_inverse_64(As, Ti, wave, lane);
    store_tm_tiles<T>(Ti, Tms, Ai_out + ((int64_t)blockIdx.x * Hv + h) * 4096, tid, wave, lane);
    GDN_LDS_BARRIER();   // the staging tile (where the next head's A goes) and Tm are consumed
  }
}

// ---------------------------------------------------------------------------------------------
// chunk_state_kernel: the inter-chunk recurrence, the only part of the forward pass that is sequential in the
// chunks.  One compute wave owns a 32-column slab of the state S[K, 32] in fp32 registers for the whole sequence
// and per chunk does
//     y = K S     z = beta (v - e^G . y)     V' = Tm z     S <- e^{G_last} S + K^T (e^{G_last-G} . V')
// which is V' = U - W S with W = Tm (beta e^G K), U = Tm (beta V) never materialised.  Every B operand (S, z, V')
// comes straight from accumulator registers (frag_b_from_acc), so the chain never touches LDS.  The A operands are
// fragment-order tiles prepared by chunk_prep_kernel (K per q/k group, Tm per value head), one contiguous block per
// chunk; K^T is the same K image read with the transposing LDS read, and the slab's raw v rows are read the same way
// into the accumulator layout.  NL loader waves of the workgroup copy the next chunks' operands global -> registers ->
// LDS two chunks ahead (two LDS stages); the roles meet at one barrier per chunk.  Where LDS allows (PRE) the loaders
// write K twice, rows scaled by -beta e^G and by e^{G_last-G}, and v scaled by beta, so that the per-token factors
// never enter the compute wave's dependent chain: z is the accumulator of (-beta e^G K) S started from beta v.
// OUT: a second wave per slab forms the output O = scale e^G . (Q S) + Aq V' of the same 32 columns from the state and
// V' the compute wave leaves in LDS (Q read transposed from the Q^T image, Aq likewise), one step behind it, so that
// neither S nor V' has to be re-read from memory; both are still stored when a backward pass will need them.
// ---------------------------------------------------------------------------------------------
// PRE: two images of K, rows scaled by -beta e^G and by e^{G_last-G} on their way into LDS.  Whether they fit is
// decided for the variant with output waves (FUSE) and two slabs per workgroup, and every other variant of the same
// element type and key width follows, so that all of them round alike.
// output waves per slab: a workgroup with a single slab has room for two, one per 32-token block of the chunk
template <int NW> struct StateOutWaves { static constexpr int value = NW == 1 ? 2 : 1; };
template <typename T, int DK, int NW, int STAGES, bool FUSE> struct StatePre {
  static constexpr int x_elems = 2 * DK * 32 + 2 * 2048 + StateOutWaves<NW>::value * Patch<T>::kElems;
  static constexpr bool value = STAGES * ((2 * 64 * DK + 3 * 1024 + 64 * 32 * NW + (FUSE ? 64 * DK + 3 * 1024 : 0)) * (int)sizeof(T) + 68 * 4) +
                                    (FUSE ? NW * x_elems * (int)sizeof(T) : 0) <= 160 * 1024;
};
template <typename T, int DK, int NW, int STAGES, bool OUT, bool PRE_, bool KDA = false> struct StateSmem {
  static constexpr int x_elems = 2 * DK * 32 + 2 * 2048 + StateOutWaves<NW>::value * Patch<T>::kElems;
  static constexpr bool PRE = PRE_;
  // one stage, in elements of T
  static constexpr int off_k = 0;                                   // K image(s) [K/32][2] tiles
  static constexpr int off_tm = off_k + (PRE ? 2 : 1) * 64 * DK;    // Tm tiles (0,0), (1,0), (1,1)
  static constexpr int off_v = off_tm + 3 * 1024;                   // raw v rows of the slabs [64][32 NW]
  static constexpr int off_q = off_v + 64 * 32 * NW;                // OUT: Q^T image
  static constexpr int off_aq = off_q + (OUT ? 64 * DK : 0);        // OUT: Aq tiles (0,0), (1,0), (1,1)
  static constexpr int off_row = (off_aq + (OUT ? 3 * 1024 : 0)) * (int)sizeof(T);   // bytes: float rows
  // rows: scale e^G [64], G_last; without PRE also e^{G_last-G} [64], beta e^G [64], beta [64]; KDA: e^{G_last} per key
  // channel [DK] at 68
  static constexpr int stage = off_row + (PRE && !KDA ? 68 : 260) * 4;   // a multiple of 16 bytes, like the offset of every row vector
  static_assert(!KDA || (PRE && DK <= 128), "KDA: both K images arrive ready-made");
  static_assert(stage % 16 == 0, "stages keep 16-byte alignment");
  static constexpr int off_x = STAGES * stage;                      // OUT: per slab S [2][DK*32], V' [2][2048], a store patch per output wave
  static constexpr int bytes = off_x + (OUT ? NW * x_elems * (int)sizeof(T) : 0);
  static_assert(bytes <= 160 * 1024, "one CU's LDS");
};

// pieces [0, PIECES) of 16 bytes dealt to NT threads, the same number to each: indices past the end repeat the last
// piece (the same loads on every path; the duplicate lands on the same LDS address with the same data)
template <int PIECES, int NT> struct Deal { static constexpr int kPer = (PIECES + NT - 1) / NT; };

// KDA (one decay per key channel): kaf and qtf hold the two K images ready-made, rows scaled by -beta e^{G} and by
// e^{G_last-G} channel by channel, G holds e^{G_last} [chunks,Hv,DK] and beta the transformed beta in fp32; the state's
// rows decay each by their own factor.  With OUT the output waves take (scale q . e^{G})^T from a third image, qim,
// whose rows carry every factor of the output's first term (the other modes read their Q^T image through qtf).
template <typename T, int DK, int NW, int NL, int STAGES, bool OUT, bool PRE_, bool KDA = false>
__global__ __launch_bounds__(64 * (NW + (OUT ? NW * StateOutWaves<NW>::value : 0) + NL)) GDN_WAVES_PER_SIMD(sizeof(T) == 2 ? 2 : 1)
void chunk_state_kernel(const T* __restrict__ kaf, const T* __restrict__ qtf, const T* __restrict__ ai,
                        const T* __restrict__ aqf, const T* __restrict__ v, const float* __restrict__ G,
                        const void* __restrict__ beta, int beta_same, const float* __restrict__ h0, float* __restrict__ ht,
                        T* __restrict__ vf, T* __restrict__ hf, T* __restrict__ o, const int64_t* __restrict__ cu,
                        const int* __restrict__ chunk_offsets, int T_len, int Hqk, int Hv, int V, float scale,
                        int64_t v_stride, const T* __restrict__ qim) {
  using SM = StateSmem<T, DK, NW, STAGES, OUT, PRE_, KDA>;
  static_assert(!KDA || 64 * NL >= DK, "a loader thread per key channel");
  constexpr int NT = 64 * NL, VEC = Elem<T>::kVec, NKT = DK / 32, OS = StateOutWaves<NW>::value, NWO = OUT ? NW * OS : 0;
  constexpr int PK = 64 * DK / VEC, PTM = 3 * 1024 / VEC, PV = 64 * 32 * NW / VEC, VPR = 32 * NW / VEC;
  constexpr int CK = Deal<PK, NT>::kPer, CTM = Deal<PTM, NT>::kPer, CV = Deal<PV, NT>::kPer;
  static_assert(STAGES == 1 || STAGES == 2, "one or two LDS stages");
  static_assert(!OUT || STAGES == 2, "the output waves read a stage while the next one is filled");

  const int tid = threadIdx.x;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);   // wave-uniform: the roles branch on a scalar
  const int nh = xcd_grouped_head(blockIdx.x, gridDim.x, Hv / Hqk), n = nh / Hv, h = nh % Hv;
  const int64_t bos = cu ? cu[n] : (int64_t)n * T_len;
  const int len = cu ? (int)(cu[n + 1] - bos) : T_len;
  const int nchunks = (len + kChunk - 1) / kChunk;
  const int64_t chunk_base = cu ? chunk_offsets[n] : (int64_t)n * ((T_len + kChunk - 1) / kChunk);
  // number of barriers every wave passes: one per chunk, plus one that hands the last V' to the output waves
  const int nsteps = nchunks + (OUT ? 1 : 0);
  if (nchunks == 0) {   // an empty sequence: its final state is its initial state
    if (wave < NW && ht != nullptr) {
      const int v0 = 32 * (blockIdx.y * NW + wave);
      for (int kt = 0; kt < NKT; ++kt)
        for (int r = 0; r < 16; ++r) {
          const int64_t at = (((int64_t)n * Hv + h) * DK + 32 * kt + acc_row(r)) * V + v0 + acc_col();
          ht[at] = h0 != nullptr ? h0[at] : 0.f;
        }
    }
    return;
  }

  if (wave >= NW + NWO) {
    // ================= loader waves: 16-byte copies =================
    const int lt = tid - 64 * (NW + NWO);
    // DEPTH register sets: chunk j sits in set j % DEPTH from the iteration that requests it (j - DEPTH - 1) to the
    // one that copies it to LDS (j - 1), so global loads have DEPTH chunk periods to arrive
    constexpr int DEPTH = (STAGES == 2) ? 2 : 1;
    Vec16<T> pk[DEPTH][CK], ptm[DEPTH][CTM], pv[DEPTH][CV], pq[DEPTH][OUT || KDA ? CK : 1], pa[DEPTH][OUT ? CTM : 1];   // KDA: pq = second K image
    Vec16<T> pq2[DEPTH][OUT && KDA ? CK : 1];   // KDA with output waves: the Q^T image
    float pgl[DEPTH], pg[DEPTH], pgk[DEPTH][2];
    uint32_t pb[DEPTH], pbk[DEPTH][2], pbv[DEPTH][CV];   // beta as fetched
    int pnv[DEPTH];
    constexpr bool PRE = SM::PRE;
    static_assert(NT % (sizeof(T) == 2 ? 128 : 32) == 0, "a thread's pieces sit at one place of their tiles");
    const int krow = frag_piece_row<T>(lt & 127);
    auto tm_src = [&](int idc) {   // piece of the three kept tiles -> its place among the four stored ones
      const int t = idc / (1024 / VEC);
      return (t == 0 ? 0 : t + 1) * (1024 / VEC) + idc % (1024 / VEC);
    };
    auto issue = [&](int c, int set) {      // global -> registers
      const int nvalid = imin(kChunk, len - c * kChunk);
      const int64_t ch = (chunk_base + c) * Hv + h, chq = (chunk_base + c) * Hqk + h / (Hv / Hqk);
      const int64_t tok0 = bos + (int64_t)c * kChunk;
#pragma unroll
      for (int i = 0; i < CK; ++i) {
        const int idc = imin(lt + i * NT, PK - 1);
        pk[set][i] = ld16(kaf + chq * (64 * DK) + idc * VEC);   // shared by the value heads of the group
        if constexpr (OUT || KDA) pq[set][i] = ld16(qtf + chq * (64 * DK) + idc * VEC);
        if constexpr (OUT && KDA) pq2[set][i] = ld16(qim + chq * (64 * DK) + idc * VEC);
      }
#pragma unroll
      for (int i = 0; i < CTM; ++i) {
        const int src = tm_src(imin(lt + i * NT, PTM - 1));
        ptm[set][i] = ld16(ai + ch * 4096 + src * VEC);
        if constexpr (OUT) pa[set][i] = ld16(aqf + ch * 4096 + src * VEC);
      }
#pragma unroll
      for (int i = 0; i < CV; ++i) {   // rows past the end of the sequence repeat the last one (their beta is 0)
        const int idc = imin(lt + i * NT, PV - 1), row = imin(idc / VPR, nvalid - 1), cc = idc % VPR;
        pv[set][i] = ld16(v + (tok0 + row) * v_stride + (int64_t)h * V + blockIdx.y * (32 * NW) + cc * VEC);
        if constexpr (PRE) pbv[set][i] = gate_raw<T>(beta, beta_same, (tok0 + row) * Hv + h);
      }
      pnv[set] = nvalid;
      if constexpr (KDA) {
        pgl[set] = G[ch * DK + imin(lt, DK - 1)];   // e^{G_last} of this thread's key channel
        return;
      }
      const float* gc = G + ch * 64;
      const int t = lt & 63;
      // raw values only: arithmetic here would wait for every load issued so far.  G repeats G_last past the end of a
      // short chunk.
      pgl[set] = gc[63];
      pg[set] = gc[t];
      pb[set] = gate_raw<T>(beta, beta_same, (tok0 + imin(t, nvalid - 1)) * Hv + h);
      if constexpr (PRE) {
        // In the K tiles every 16-byte piece belongs to one token, 32 (tile & 1) + the row of its place, and this
        // thread's pieces all sit at the same place of their tiles: the gates of two tokens cover them.
#pragma unroll
        for (int j = 0; j < 2; ++j) {
          pgk[set][j] = gc[32 * j + krow];
          pbk[set][j] = gate_raw<T>(beta, beta_same, (tok0 + imin(32 * j + krow, nvalid - 1)) * Hv + h);
        }
      }
    };
    auto commit = [&](int set, int buf) {   // registers -> LDS stage
      T* st = reinterpret_cast<T*>(gdn_smem + buf * SM::stage);
      float f1[2], f2[2];
      if constexpr (PRE && !KDA) {
#pragma unroll
        for (int j = 0; j < 2; ++j) {
          f1[j] = (32 * j + krow < pnv[set]) ? -gate_val<T>(pbk[set][j], beta_same) * __expf(pgk[set][j]) : 0.f;
          f2[j] = __expf(pgl[set] - pgk[set][j]);
        }
      }
#pragma unroll
      for (int i = 0; i < CK; ++i) {
        const int idc = imin(lt + i * NT, PK - 1);
        if constexpr (KDA) {
          st16(st + SM::off_k + idc * VEC, pk[set][i]);
          st16(st + SM::off_k + 64 * DK + idc * VEC, pq[set][i]);
        } else if constexpr (PRE) {
          const int tj = (idc / (1024 / VEC)) & 1;
          st16(st + SM::off_k + idc * VEC, scale16<T>(pk[set][i], f1[tj]));
          st16(st + SM::off_k + 64 * DK + idc * VEC, scale16<T>(pk[set][i], f2[tj]));
        } else {
          st16(st + SM::off_k + idc * VEC, pk[set][i]);
        }
        if constexpr (OUT) st16(st + SM::off_q + idc * VEC, KDA ? pq2[set][i] : pq[set][i]);
      }
#pragma unroll
      for (int i = 0; i < CTM; ++i) {
        const int idc = imin(lt + i * NT, PTM - 1);
        st16(st + SM::off_tm + idc * VEC, ptm[set][i]);
        if constexpr (OUT) st16(st + SM::off_aq + idc * VEC, pa[set][i]);
      }
#pragma unroll
      for (int i = 0; i < CV; ++i) {
        const int idc = imin(lt + i * NT, PV - 1);
        if constexpr (PRE) st16(st + SM::off_v + idc * VEC, scale16<T>(pv[set][i], idc / VPR < pnv[set] ? gate_val<T>(pbv[set][i], beta_same) : 0.f));
        else st16(st + SM::off_v + idc * VEC, pv[set][i]);
      }
      float* row = reinterpret_cast<float*>(gdn_smem + buf * SM::stage + SM::off_row);
      if constexpr (KDA) {
        if (lt < DK) row[68 + lt] = pgl[set];
        return;
      }
      if (lt < 64) {
        const float b = lt < pnv[set] ? gate_val<T>(pb[set], beta_same) : 0.f, eg = __expf(pg[set]);
        row[lt] = scale * eg;
        if constexpr (!PRE) {
          row[68 + lt] = __expf(pgl[set] - pg[set]);
          row[132 + lt] = b * eg;
          row[196 + lt] = b;
        }
      }
      if (lt == 0) row[64] = pgl[set];
    };
    if (STAGES == 2) {
      // Every path through this loop issues the same loads in the same order (chunk indices past the end are clamped
      // and their data is never used), so that the number of loads in flight at each wait is a compile-time fact and
      // the waits before the LDS writes of one register set leave the younger sets in flight.
      issue(0, 0);
      commit(0, 0);
#pragma unroll
      for (int j = 1; j <= DEPTH; ++j) issue(imin(j, nchunks - 1), j % DEPTH);
      // The loop leaves only at the end of a whole round of register sets: an exit in the middle of the round would be
      // one more way into the code that follows it, one on which fewer loads are in flight, and the waits before the
      // LDS writes (counted by the compiler over all ways in) would then also wait for the younger set.
      int c0 = 0;
      for (; c0 + DEPTH <= nsteps; c0 += DEPTH) {
#pragma unroll
        for (int u = 0; u < DEPTH; ++u) {
          const int c = c0 + u;
          GDN_LDS_BARRIER();                // (A) chunk c staged; the other stage (chunk c-1) is free
          commit((u + 1) % DEPTH, (c + 1) & 1);
          issue(imin(c + 1 + DEPTH, nchunks - 1), (u + 1) % DEPTH);
        }
      }
#pragma unroll
      for (int u = 0; u < DEPTH - 1; ++u) {   // the steps left over: their barriers, and the stage the next one reads
        const int c = c0 + u;
        if (c < nsteps) {
          GDN_LDS_BARRIER();
          commit((u + 1) % DEPTH, (c + 1) & 1);
        }
      }
    } else {
      for (int c = 0; c < nsteps; ++c) {
        if (c > 0) GDN_LDS_BARRIER();       // (B) the single stage is free again
        issue(imin(c, nchunks - 1), 0);
        commit(0, 0);
        GDN_LDS_BARRIER();                  // (A)
      }
    }
    return;
  }

  if constexpr (OUT) {
    if (wave >= NW) {
      // ================= output waves: O of the slab's 32 columns, one step behind the compute wave =================
      // OS == 2: wave `hw` of the slab's two owns the chunk's 32-token block hw (and that share of the stores for the
      // backward pass); OS == 1: one wave does both blocks.  Either way every row is accumulated by the same
      // instructions in the same order.
      const int w = (wave - NW) / OS, hw = (wave - NW) % OS;
      const int vblk = blockIdx.y * NW + w, v0 = 32 * vblk;
      T* xs = reinterpret_cast<T*>(gdn_smem + SM::off_x) + w * SM::x_elems;
      T* patch = xs + 2 * DK * 32 + 2 * 2048 + hw * Patch<T>::kElems;
      IdentityFrag<T> id;
      id.init();
      f32x16 oa[2];
      AccB<T> Af[3];
      for (int c = 0; c < nsteps; ++c) {
        const int buf = (STAGES == 2) ? (c & 1) : 0;
        GDN_LDS_BARRIER();                    // (A)
        if (c > 0) {                          // finish chunk c-1: + Aq V', rows out
          const T* vx = xs + 2 * DK * 32 + ((c - 1) & 1) * 2048;
          const int64_t tile0 = ((chunk_base + c - 1) * Hv + h) * (V / 32) + vblk;
          const int64_t tok0 = bos + (int64_t)(c - 1) * kChunk;
          const int nvalid = imin(kChunk, len - (c - 1) * kChunk);
          T* og = o + (tok0 * Hv + h) * V + v0;
          AccB<T> Vb[2];
          Vb[0].load(vx);
          if (OS == 1 || hw == 1) Vb[1].load(vx + 1024);
          if constexpr (OS == 2) {
            if (vf != nullptr) {                          // v_new of chunk c-1, for the backward pass
              if (hw == 0) Vb[0].store_stream(vf + (tile0 * 2 + 0) * 1024);
              else Vb[1].store_stream(vf + (tile0 * 2 + 1) * 1024);
            }
            mma32_ff<T>(oa[0], Af[0], Vb[0]);            // hw == 0: Aq tile (0,0); hw == 1: tile (1,0) ...
            if (hw == 1) mma32_ff<T>(oa[0], Af[1], Vb[1]);   // ... and (1,1)
            acc_store_rows<T, false>(oa[0], id, patch, og + (int64_t)32 * hw * Hv * V, (int64_t)Hv * V, nvalid - 32 * hw);
          } else {
            if (vf != nullptr) {
              Vb[0].store_stream(vf + (tile0 * 2 + 0) * 1024);
              Vb[1].store_stream(vf + (tile0 * 2 + 1) * 1024);
            }
            mma32_ff<T>(oa[0], Af[0], Vb[0]);
            mma32_ff<T>(oa[1], Af[1], Vb[0]);
            mma32_ff<T>(oa[1], Af[2], Vb[1]);
#pragma unroll
            for (int ri = 0; ri < 2; ++ri)
              acc_store_rows<T, false>(oa[ri], id, patch, og + (int64_t)32 * ri * Hv * V, (int64_t)Hv * V, nvalid - 32 * ri);
          }
        }
        if (c < nchunks) {                    // start chunk c: scale e^G . (Q S), and its Aq tiles into registers
          const T* st = reinterpret_cast<const T*>(gdn_smem + buf * SM::stage);
          const float* row = reinterpret_cast<const float*>(gdn_smem + buf * SM::stage + SM::off_row);
          const T* sx = xs + (c & 1) * (DK * 32);
          oa[0] = acc_zero();
          oa[1] = acc_zero();
#pragma unroll
          for (int kt = 0; kt < NKT; ++kt) {
            AccB<T> Sb, Qf;
            Sb.load(sx + kt * 1024);
            if (hf != nullptr && (OS == 1 || (kt & 1) == hw))   // the state before chunk c, for the backward pass
              Sb.store_stream(hf + ((((chunk_base + c) * Hv + h) * (V / 32) + vblk) * NKT + kt) * 1024);
            if constexpr (OS == 2) {
              Qf.load_t(st + SM::off_q + (kt * 2 + hw) * 1024);   // Q tile (token block hw, K block kt)
              mma32_ff<T>(oa[0], Qf, Sb);
            } else {
#pragma unroll
              for (int ri = 0; ri < 2; ++ri) {
                Qf.load_t(st + SM::off_q + (kt * 2 + ri) * 1024);   // Q tile (token block ri, K block kt)
                mma32_ff<T>(oa[ri], Qf, Sb);
              }
            }
          }
          if constexpr (OS == 2) {
            if constexpr (!KDA) {   // KDA: the rows of the Q image carry scale and decay
              const f32x16 e0 = rows_ld(row, 32 * hw);
#pragma unroll
              for (int r = 0; r < 16; ++r) oa[0][r] *= e0[r];
            }
            Af[0].load_t(st + SM::off_aq + hw * 1024);   // (lane <-> row i, registers <-> column j)
            if (hw == 1) Af[1].load_t(st + SM::off_aq + 2 * 1024);
          } else {
            if constexpr (!KDA) {
              const f32x16 e0 = rows_ld(row, 0), e1 = rows_ld(row, 32);
#pragma unroll
              for (int r = 0; r < 16; ++r) { oa[0][r] *= e0[r]; oa[1][r] *= e1[r]; }
            }
#pragma unroll
            for (int t = 0; t < 3; ++t) Af[t].load_t(st + SM::off_aq + t * 1024);   // (lane <-> row i, registers <-> column j)
          }
          if (STAGES == 1 && c + 1 < nsteps) GDN_LDS_BARRIER();   // (B)
        }
      }
      return;
    }
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
  // depend on the running product (decay of S, packing S for the next chunk) sits between the matrix instructions
  // instead of before or after them.
  AccB<T> Sb[NKT];
  T* xs = reinterpret_cast<T*>(gdn_smem + SM::off_x) + wave * SM::x_elems;   // OUT only
  // Two tile products into two accumulators, the matrix instructions of one alternating with those of the other: back
  // to back on one accumulator a matrix instruction costs half as much again (49 cycles against 34, measured).
  auto mma2 = [](f32x16& x0, const AccB<T>& a0, const AccB<T>& b0, f32x16& x1, const AccB<T>& a1, const AccB<T>& b1) {
#pragma unroll
    for (int kg = 0; kg < AccK<T>::kGroups; ++kg) {
      mfma_kgroup<T>(x0, a0.f[kg], b0.f[kg]);
      mfma_kgroup<T>(x1, a1.f[kg], b1.f[kg]);
    }
  };
#pragma unroll
  for (int kt = 0; kt < NKT; ++kt) {
    Sb[kt].pack(S[kt]);
    if constexpr (OUT) Sb[kt].store(xs + kt * 1024);
  }
  for (int c = 0; c < nchunks; ++c) {
    const int buf = (STAGES == 2) ? (c & 1) : 0;
    GDN_LDS_BARRIER();                        // (A) stage `buf` holds chunk c
    const T* st = reinterpret_cast<const T*>(gdn_smem + buf * SM::stage);
    constexpr bool PRE = SM::PRE;
    const T* Ka = st + SM::off_k;                        // PRE: rows scaled by -beta e^G
    const T* Kb = Ka + (PRE ? 64 * DK : 0);              // PRE: rows scaled by e^{G_last-G}
    const T* Tm = st + SM::off_tm;
    const T* Vs = st + SM::off_v;
    const float* row = reinterpret_cast<const float*>(gdn_smem + buf * SM::stage + SM::off_row);
    const int64_t tile0 = ((chunk_base + c) * Hv + h) * (V / 32) + vblk;

    constexpr int NP = NKT / 2;             // K tiles are processed two at a time
    AccB<T> Kf[2][2][2];                    // [buffer][32-token block][K tile of the pair]; later [buffer][K tile][token block]
    auto load_k = [&](int b, int kp) {      // K as it lies: (lane <-> token, registers <-> K column)
#pragma unroll
      for (int ri = 0; ri < 2; ++ri)
#pragma unroll
        for (int j = 0; j < 2; ++j) Kf[b][ri][j].load(Ka + ((2 * kp + j) * 2 + ri) * 1024);
    };
    auto load_kt = [&](int b, int kp) {     // K^T: (lane <-> K column, registers <-> token)
#pragma unroll
      for (int j = 0; j < 2; ++j)
#pragma unroll
        for (int tj = 0; tj < 2; ++tj) Kf[b][j][tj].load_t(Kb + ((2 * kp + j) * 2 + tj) * 1024);
    };
    AccB<T> Vb[2], Tf[3];
    Vb[0].load_cols(Vs + 32 * wave, 32 * NW);                     // raw v, (lane <-> V column, registers <-> token)
    Vb[1].load_cols(Vs + 32 * (32 * NW) + 32 * wave, 32 * NW);
    load_k(0, 0);
    if (NP > 1) load_k(1, 1);
    const float eg = KDA ? 1.f : __expf(row[64]);
    if (!OUT && hf != nullptr) {   // with output waves the stores are theirs: they hold S and V' too and have the time
#pragma unroll
      for (int kt = 0; kt < NKT; ++kt) Sb[kt].store_stream(hf + (tile0 * NKT + kt) * 1024);
    }
    // y = K S (PRE: z = beta v - beta e^G . (K S) at once), the two 32-token blocks are independent accumulation
    // chains.  The decay of S rides between the matrix instructions.
    f32x16 p0 = PRE ? Vb[0].unpack() : acc_zero(), p1 = PRE ? Vb[1].unpack() : acc_zero();
    GDN_SCHED_FENCE();
#pragma unroll
    for (int kp = 0; kp < NP; ++kp) {
#pragma unroll
      for (int j = 0; j < 2; ++j) {
        mma2(p0, Kf[kp & 1][0][j], Sb[2 * kp + j], p1, Kf[kp & 1][1][j], Sb[2 * kp + j]);
        if constexpr (KDA) {
          const f32x16 dk = rows_ld(row + 68, 32 * (2 * kp + j));   // the decay of each of the tile's 32 key channels
#pragma unroll
          for (int r = 0; r < 16; ++r) S[2 * kp + j][r] *= dk[r];
        } else {
#pragma unroll
          for (int r = 0; r < 16; ++r) S[2 * kp + j][r] *= eg;
        }
        GDN_INTERLEAVE_MFMA_VALU(2 * AccK<T>::kGroups, 16 / (2 * AccK<T>::kGroups));
      }
      GDN_SCHED_FENCE();
      if (kp + 2 < NP) load_k(kp & 1, kp + 2);
      GDN_SCHED_FENCE();
    }
#pragma unroll
    for (int t = 0; t < 3; ++t) Tf[t].load(Tm + t * 1024);
    if constexpr (!PRE) {
      // z = beta (v - e^G . y), the B operand of Tm z
      const f32x16 b0 = rows_ld(row + 196, 0), b1 = rows_ld(row + 196, 32);
      const f32x16 e0 = rows_ld(row + 132, 0), e1 = rows_ld(row + 132, 32);
      const f32x16 x0 = Vb[0].unpack(), x1 = Vb[1].unpack();
#pragma unroll
      for (int r = 0; r < 16; ++r) { p0[r] = b0[r] * x0[r] - e0[r] * p0[r]; p1[r] = b1[r] * x1[r] - e1[r] * p1[r]; }
    }
    Vb[0].pack(p0);
    Vb[1].pack(p1);
    load_kt(0, 0);
    // V' = Tm z (Tm lower triangular: tiles (0,0), (1,0), (1,1))
    p0 = acc_zero();
    p1 = acc_zero();
    mma2(p0, Tf[0], Vb[0], p1, Tf[1], Vb[0]);
    mma32_ff<T>(p1, Tf[2], Vb[1]);
    if (NP > 1) load_kt(1, 1);
    Vb[0].pack(p0);
    Vb[1].pack(p1);
    if (!OUT && vf != nullptr) {
      Vb[0].store_stream(vf + (tile0 * 2 + 0) * 1024);
      Vb[1].store_stream(vf + (tile0 * 2 + 1) * 1024);
    }
    if constexpr (OUT) {
      T* vx = xs + 2 * DK * 32 + (c & 1) * 2048;
      Vb[0].store(vx);
      Vb[1].store(vx + 1024);
    }
    if constexpr (!PRE) {
      // the decay of the state update rides on V': (e^{G_last - G} . K)^T V' = K^T (e^{G_last - G} . V')
      const f32x16 d0 = rows_ld(row + 68, 0), d1 = rows_ld(row + 68, 32);
#pragma unroll
      for (int r = 0; r < 16; ++r) { p0[r] *= d0[r]; p1[r] *= d1[r]; }
      Vb[0].pack(p0);
      Vb[1].pack(p1);
    }
    GDN_SCHED_FENCE();
    // S <- e^{G_last} S + K^T (e^{G_last - G} . V'); a finished tile of S is packed for the next chunk while the
    // matrix pipe works on the following ones
#pragma unroll
    for (int kp = 0; kp < NP; ++kp) {
#pragma unroll
      for (int tj = 0; tj < 2; ++tj) {   // the pair's two tiles of S take turns
        mma2(S[2 * kp], Kf[kp & 1][0][tj], Vb[tj], S[2 * kp + 1], Kf[kp & 1][1][tj], Vb[tj]);
        if (kp >= 1) Sb[2 * kp - 2 + tj].pack(S[2 * kp - 2 + tj]);
      }
      GDN_SCHED_FENCE();
      if (kp + 2 < NP) { load_kt(kp & 1, kp + 2); GDN_SCHED_FENCE(); }
    }
#pragma unroll
    for (int kt = (NKT >= 2 ? NKT - 2 : 0); kt < NKT; ++kt) Sb[kt].pack(S[kt]);
    if constexpr (OUT) {   // the state before chunk c+1, for the output wave's next step
#pragma unroll
      for (int kt = 0; kt < NKT; ++kt) Sb[kt].store(xs + ((c + 1) & 1) * (DK * 32) + kt * 1024);
    }
    if (STAGES == 1 && c + 1 < nsteps) GDN_LDS_BARRIER();      // (B) done with the single stage
  }
  if constexpr (OUT) GDN_LDS_BARRIER();       // (A) of the extra step: the last V' is in LDS for the output wave
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
  // G null: the rows of q arrive with scale and decay already applied (KDA, one decay per key channel)
  const float gval = G != nullptr ? G[ch * 64 + imin(tid & 63, nvalid - 1)] : 0.f;
#pragma unroll
  for (int i = 0; i < QPT; ++i) {
    const int c = tid + i * NT, row = c / (DK / VEC), cc = c % (DK / VEC);
    Vec16<T> x = zero16<T>();
    if (row < nvalid) x = rstd_q != nullptr ? scale16<T>(qreg[i], qs[i]) : qreg[i];
    st16(Qs + row * LDK + cc * VEC, x);
  }
  if (tid < 64) Eg[tid] = G != nullptr ? scale * __expf(gval) : 1.f;
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

// NW: waves (32-column blocks) per workgroup of the stand-alone output kernel; NWS, NLS, STAGES: slabs, loader waves
// and LDS stages of the recurrence kernel; FUSE: the recurrence kernel's own output waves write O (no norm, bf16)
template <typename T, int DK, int NW, int NWS, int NLS, int STAGES, bool FUSE>
static int chunk_fwd_launch(const ChunkDims& d, const ChunkWorkspace& L, const void* q, const void* k, const void* v,
                            const float* g, const void* beta, int beta_same, const float* h0, const int64_t* cu, void* o,
                            float* ht, unsigned char* ws, unsigned char* ws_state, bool skip_prep, float scale, int l2norm,
                            bool with_backward, const FwdNorm& fn, hipStream_t st) {
  // ws: base of the workspace's prep part; ws_state: base such that ws_state + L.VF, + L.HF are the state part (equal to
  // ws when the workspace is one buffer).  skip_prep: the prep part already holds this input's tiles.
  const int nc = (int)d.max_chunks();
  int* chunk_offsets = reinterpret_cast<int*>(ws + L.chunk_offsets);
  const T* qq = (const T*)q;
  const T* kk = (const T*)k;
  if (cu != nullptr && !skip_prep) GDN_LAUNCH(kKernChunkTable, st, chunk_table_kernel, dim3(1), dim3(kThreads), 0, st, cu, chunk_offsets, d.N);
  float* rstd = reinterpret_cast<float*>(ws + L.rstd);
  float* G = reinterpret_cast<float*>(ws + L.G);
  T* Ai = reinterpret_cast<T*>(ws + L.Ai);
  T* AQ = reinterpret_cast<T*>(ws + L.AQ);
  T* KAF = reinterpret_cast<T*>(ws + L.KAF);
  T* QTF = reinterpret_cast<T*>(ws + L.QTF);
  const bool fill_only = o == nullptr && fn.y == nullptr;   // refill the workspace for a backward pass, no output
  const bool fuse = FUSE && fn.y == nullptr && !fill_only;
  // the per-chunk states and v_new leave the recurrence kernel only for a later reader: the backward pass or the
  // stand-alone output kernel
  const bool keep = with_backward || !fuse;
  T* VF = keep ? reinterpret_cast<T*>(ws_state + L.VF) : nullptr;
  T* HF = keep ? reinterpret_cast<T*>(ws_state + L.HF) : nullptr;
  const TokenStrides ts = d.strides();
  {
    const int64_t ob = (int64_t)d.Hv * d.V * (int)sizeof(T);
    TailRows tail{{o, fn.y, fn.y != nullptr ? (void*)fn.rstd : nullptr}, {ob, ob, (int64_t)d.Hv * 4}, {(int)ob, (int)ob, d.Hv * 4}};
    launch_zero_tail_rows(cu, d.N, d.tokens(), tail, st);
  }
  if (!skip_prep) {
    auto kern = chunk_prep_kernel<T, DK>;
    const int smem = PrepSmem<T, DK>::launch_bytes(d.Hv / d.Hqk);
    if (int e = set_lds(kern, smem)) return e;
    GDN_LAUNCH(kKernPrep, st, kern, dim3(nc, d.Hqk), dim3(kThreads), smem, st, qq, kk, g, beta, beta_same, cu,
               (const int*)chunk_offsets, G, Ai, AQ, KAF, QTF, rstd, rstd + (int64_t)nc * 64 * d.Hqk, d.T, d.N, d.Hqk,
               d.Hv, scale, l2norm, ts);
  }
  // decided for the two-slab variant, the largest one: results must not depend on how many slabs a launch happens
  // to give a workgroup (a sequence computes the same bits alone and inside a packed batch)
  constexpr bool PRE = StatePre<T, DK, 2, STAGES, FUSE>::value && StatePre<T, DK, NWS, STAGES, FUSE>::value;
  auto launch_state = [&](auto kern, int smem, int waves, T* op) -> int {
    if (int e = set_lds(kern, smem)) return e;
    GDN_LAUNCH(kKernStateFwd, st, kern, dim3(d.N * d.Hv, d.V / (32 * NWS)), dim3(64 * waves), smem, st, (const T*)KAF,
               (const T*)QTF, (const T*)Ai, (const T*)AQ, (const T*)v, (const float*)G, beta, beta_same, h0, ht, VF, HF, op, cu,
               (const int*)chunk_offsets, d.T, d.Hqk, d.Hv, d.V, scale, ts.v, (const T*)nullptr);
    return 0;
  };
  if constexpr (FUSE) {
    if (fuse) {
      if (int e = launch_state(chunk_state_kernel<T, DK, NWS, NLS, STAGES, true, PRE>,
                               StateSmem<T, DK, NWS, STAGES, true, PRE>::bytes, NWS * (1 + StateOutWaves<NWS>::value) + NLS, (T*)o))
        return e;
      return (int)hipGetLastError();
    }
  }
  if (int e = launch_state(chunk_state_kernel<T, DK, NWS, NLS, STAGES, false, PRE>,
                           StateSmem<T, DK, NWS, STAGES, false, PRE>::bytes, NWS + NLS, (T*)nullptr))
    return e;
  if (fill_only) return (int)hipGetLastError();
  auto launch_out = [&](auto kern, auto nm) -> int {
    constexpr int smem = OutSmem<T, DK, NW>::bytes;
    if (int e = set_lds(kern, smem)) return e;
    GDN_LAUNCH(kKernOut, st, kern, dim3(nc, d.Hv, d.V / (32 * NW)), dim3(64 * NW), smem, st, qq,
               (const T*)AQ, (const T*)VF, (const T*)HF, (const float*)G, (T*)o, cu, (const int*)chunk_offsets, d.T, d.N, d.Hqk,
               d.Hv, d.V, scale, ts.q, l2norm ? (const float*)rstd : (const float*)nullptr, nm);
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
  if (with_backward == 2) return w.prep_bytes;                    // the prep part alone
  if (with_backward == 3) return w.total_bytes - w.prep_bytes;    // the state part alone
  return with_backward ? w.total_bytes : w.fwd_bytes;
}

namespace gdn {
int chunk_fwd_entry(const void* q, const void* k, const void* v, int64_t q_stride, int64_t k_stride,
                           int64_t v_stride, const float* g, const void* beta, int beta_dtype, const float* initial_state,
                           const int64_t* cu_seqlens, void* o, float* final_state, void* workspace,
                           int64_t workspace_bytes, int B, int T, int N, int Hqk, int Hv, int K, int V, float scale,
                           int use_qk_l2norm, int dtype, const FwdNorm& fn, void* stream, void* workspace_state,
                           int64_t workspace_state_bytes, bool skip_prep, bool share_device) {
  if (!q || !k || !v || !g || !beta || !workspace) return -1;
  if (fn.y != nullptr && (!fn.gate || !fn.weight)) return -1;
  ChunkDims d{B, T, N, Hqk, Hv, K, V, cu_seqlens != nullptr};
  d.ts = {q_stride, k_stride, v_stride, 0, 0, 0};
  if (int e = chunk_check_dims(d, dtype)) return e;
  if (beta_dtype != 0 && beta_dtype != dtype) return -4;
  const int beta_same = beta_dtype != 0;
  if (((uintptr_t)q | (uintptr_t)k | (uintptr_t)v | (uintptr_t)o | (uintptr_t)fn.y | (uintptr_t)fn.gate |
       (uintptr_t)fn.weight) & 15)
    return -6;
  ChunkDims dl = d;
  dl.varlen = true;  // one layout for both modes (the packed bound is the larger)
  const ChunkWorkspace L = chunk_workspace_layout(dl, dtype == 0 ? 4 : 2);
  // One buffer: sized for backward (states and v_new are kept), for forward only, or -- where the recurrence writes the
  // output itself and nothing reads states or v_new from memory (16-bit types, no fused norm) -- just the prep part.
  // Two buffers: the prep part and the state part (forward states, v_new, and room for their gradients).
  const bool fused_out = dtype == 1 && fn.y == nullptr && o != nullptr;
  bool with_bwd;
  unsigned char* ws = static_cast<unsigned char*>(workspace);
  unsigned char* ws_state = ws;
  if (workspace_state != nullptr) {
    if (workspace_bytes < L.prep_bytes || workspace_state_bytes < L.total_bytes - L.prep_bytes) return -5;
    if ((reinterpret_cast<uintptr_t>(workspace_state) & 255) != 0) return -5;
    ws_state = static_cast<unsigned char*>(workspace_state) - L.prep_bytes;
    with_bwd = true;
  } else {
    if (workspace_bytes < (fused_out ? L.prep_bytes : L.fwd_bytes)) return -5;
    with_bwd = workspace_bytes >= L.total_bytes;
    if (skip_prep) return -1;
  }
  if (!o && !fn.y && !with_bwd) return -1;   // without an output the call only makes sense as a refill
  if ((reinterpret_cast<uintptr_t>(workspace) & 255) != 0) return -5;
  hipStream_t st = (hipStream_t)stream;
#define GDN_FWD(T_, DK_, NW_, NWS_, NLS_, ST_, FUSE_)                                                                       \
  return chunk_fwd_launch<T_, DK_, NW_, NWS_, NLS_, ST_, FUSE_>(d, L, q, k, v, g, beta, beta_same, initial_state, cu_seqlens, o, final_state, \
                                                   ws, ws_state, skip_prep, scale, use_qk_l2norm, with_bwd, fn, st)
  const bool wide = (V % 128 == 0);
  const bool solo = one_slab_per_workgroup(d, device_compute_units()) &&
                    !(share_device && two_slabs_to_share_device(d, device_compute_units()));
  if (dtype == 1) {
    if (K == 128 && wide && solo) GDN_FWD(bf16_t, 128, 4, 1, 4, 2, true);
    if (K == 128 && wide) GDN_FWD(bf16_t, 128, 4, 2, 4, 2, true);
    if (K == 128) GDN_FWD(bf16_t, 128, 2, 2, 4, 2, true);
    if (K == 64 && wide) GDN_FWD(bf16_t, 64, 4, 2, 4, 2, true);
    GDN_FWD(bf16_t, 64, 2, 2, 4, 2, true);
  } else {
    if (K == 128 && wide) GDN_FWD(float, 128, 4, 4, 4, 1, false);
    if (K == 128) GDN_FWD(float, 128, 2, 2, 2, 1, false);
    if (wide) GDN_FWD(float, 64, 4, 4, 4, 2, false);
    GDN_FWD(float, 64, 2, 2, 2, 2, false);
  }
#undef GDN_FWD
}
}  // namespace gdn

extern "C" int gdn_chunk_fwd_strided(const void* q, const void* k, const void* v, int64_t q_stride, int64_t k_stride,
                                     int64_t v_stride, const float* g, const void* beta, const float* initial_state,
                                     const int64_t* cu_seqlens, void* o, float* final_state, void* workspace,
                                     int64_t workspace_bytes, int B, int T, int N, int Hqk, int Hv, int K, int V,
                                     float scale, int use_qk_l2norm, int dtype, int beta_dtype, void* stream) {
  return gdn::chunk_fwd_entry(q, k, v, q_stride, k_stride, v_stride, g, beta, beta_dtype, initial_state, cu_seqlens, o, final_state,
                              workspace, workspace_bytes, B, T, N, Hqk, Hv, K, V, scale, use_qk_l2norm, dtype,
                              gdn::FwdNorm{}, stream);
}

extern "C" int gdn_chunk_fwd_norm_strided(const void* q, const void* k, const void* v, int64_t q_stride,
                                          int64_t k_stride, int64_t v_stride, const float* g, const void* beta,
                                          const float* initial_state, const int64_t* cu_seqlens, const void* gate,
                                          const void* norm_weight, void* o, void* y, float* rstd, float* final_state,
                                          void* workspace, int64_t workspace_bytes, int B, int T, int N, int Hqk,
                                          int Hv, int K, int V, float scale, float eps, int use_qk_l2norm, int dtype,
                                          int weight_dtype, int beta_dtype, void* stream) {
  if (!y) return -1;
  if (weight_dtype != 0 && weight_dtype != dtype) return -4;
  if (V != 64 && V != 128) return -3;
  return gdn::chunk_fwd_entry(q, k, v, q_stride, k_stride, v_stride, g, beta, beta_dtype, initial_state, cu_seqlens, o, final_state,
                              workspace, workspace_bytes, B, T, N, Hqk, Hv, K, V, scale, use_qk_l2norm, dtype,
                              gdn::FwdNorm{gate, norm_weight, y, rstd, eps, weight_dtype == 0}, stream);
}

extern "C" int gdn_chunk_fwd(const void* q, const void* k, const void* v, const float* g, const float* beta,
                             const float* initial_state, const int64_t* cu_seqlens, void* o, float* final_state,
                             void* workspace, int64_t workspace_bytes, int B, int T, int N, int Hqk, int Hv, int K,
                             int V, float scale, int use_qk_l2norm, int dtype, void* stream) {
  return gdn_chunk_fwd_strided(q, k, v, 0, 0, 0, g, beta, initial_state, cu_seqlens, o, final_state, workspace,
                               workspace_bytes, B, T, N, Hqk, Hv, K, V, scale, use_qk_l2norm, dtype, 0, stream);
}

#include "gdn_kda_fwd.h"
