// Host-side description of the workspace shared by the chunked forward and backward passes.
#pragma once
#include <stdint.h>

namespace gdn {

// Distance between consecutive tokens, in elements, of the token-major tensors the caller hands over.  The heads of a
// token are contiguous ([Hqk,K] / [Hv,V]); a stride larger than that lets q, k, v (and dq, dk, dv) be slices of one
// wider [tokens, D] tensor, e.g. the output of the convolution in front of the operator.
struct TokenStrides {
  int64_t q, k, v, dq, dk, dv;
};

struct ChunkDims {
  int B, T, N, Hqk, Hv, K, V;
  bool varlen;
  TokenStrides ts = {0, 0, 0, 0, 0, 0};   // 0 = contiguous heads
  TokenStrides strides() const {
    const int64_t nq = (int64_t)Hqk * K, nv = (int64_t)Hv * V;
    return {ts.q ? ts.q : nq, ts.k ? ts.k : nq, ts.v ? ts.v : nv, ts.dq ? ts.dq : nq, ts.dk ? ts.dk : nq, ts.dv ? ts.dv : nv};
  }
  int64_t tokens() const { return (int64_t)B * T; }
  // upper bound on the number of 64-token chunks; exact without cu_seqlens.  Packed sequences add at
  // most one partial chunk each, so the bound needs no look at the (device-resident) lengths.
  int64_t max_chunks() const {
    if (!varlen) return (int64_t)B * ((T + 63) / 64);
    return tokens() / 64 + N;
  }
};

// Byte offsets into the workspace.  Everything the backward pass re-reads is written by the forward.
// Tiles exchanged between kernels are in fragment order (see AccB<>): 1024 elements per 32x32 tile.
struct ChunkWorkspace {
  int64_t chunk_offsets;  // int32 [N+1]      chunks before each packed sequence
  int64_t rstd;           // f32 [2][chunks,Hqk,64] 1/|q|, 1/|k| of the in-kernel l2 norm, 64 contiguous values per chunk
  int64_t G;              // f32 [chunks,Hv,64]      chunk-local cumulative log decay
  int64_t Ai;             // T [chunks,Hv,2,2]       Tm = (I + L)^-1 as A operand: tile = (32 rows) x (32 columns)
  int64_t AQ;             // T [chunks,Hv,2,2]       scale tril(Q K^T . Gam), accumulator tiles: lane <-> column, registers <-> row
  int64_t KAF;            // T [chunks,Hqk,K/32,2]   K as A operand: tile = (32 tokens) x (32 columns of K)
  int64_t QTF;            // T [chunks,Hqk,K/32,2]   Q^T as A operand: tile = (32 columns of K) x (32 tokens)
  int64_t prep_bytes;     // everything above: what chunk_prep_kernel leaves (no v, no state in it).  What follows, the "state
                          // part", may live in a second buffer: the kernels take a base pointer for each part.
  int64_t VF;             // T [chunks,Hv,V/32,2]    v_new = Tm (beta v - beta e^G K S), tile = (32-column block) x (32-token block)
  int64_t HF;             // T [chunks,Hv,V/32,K/32] state BEFORE each chunk, tile = (32 rows of K) x (32 columns of V)
  int64_t fwd_bytes;
  int64_t DVF;            // T [chunks,Hv,V/32,2]    d(v_new)
  int64_t DHF;            // T [chunks,Hv,V/32,K/32] gradient of the state AFTER each chunk; once the chunk-local kernel of a
                          //   head has read its part it may leave the group's dq, dk sums there for the next head's launch
  int64_t total_bytes;
};

inline int64_t align256(int64_t x) { return (x + 255) / 256 * 256; }

inline ChunkWorkspace chunk_workspace_layout(const ChunkDims& d, int elem_bytes) {
  ChunkWorkspace w;
  int64_t off = 0;
  auto take = [&](int64_t bytes) { int64_t o = off; off += align256(bytes); return o; };
  const int64_t nc = d.max_chunks();
  w.chunk_offsets = take((int64_t)(d.N + 1) * 4);
  w.rstd = take(2 * nc * 64 * d.Hqk * 4);
  w.G = take(nc * 64 * d.Hv * 4);
  w.Ai = take(nc * 64 * d.Hv * 64 * elem_bytes);
  w.AQ = take(nc * 64 * d.Hv * 64 * elem_bytes);
  w.KAF = take(nc * 64 * d.Hqk * d.K * elem_bytes);
  w.QTF = take(nc * 64 * d.Hqk * d.K * elem_bytes);
  w.prep_bytes = off;
  w.VF = take(nc * 64 * d.Hv * d.V * elem_bytes);
  w.HF = take(nc * d.Hv * d.V * d.K * elem_bytes);
  w.fwd_bytes = off;
  w.DVF = take(nc * 64 * d.Hv * d.V * elem_bytes);
  w.DHF = take(nc * d.Hv * d.V * d.K * elem_bytes);
  w.total_bytes = off;
  return w;
}

// KDA (one decay per key channel; q, k, v heads in equal number H): what its prep kernel leaves for the recurrence and
// the output kernel.  The two K images carry the per-channel factors, so the recurrence itself only decays the rows
// of the state by e^{G_last}.
struct KdaWorkspace {
  int64_t chunk_offsets;  // int32 [N+1]
  int64_t rstd;           // f32 [2][chunks,H,64]   1/|q|, 1/|k| of the in-kernel l2 norm
  int64_t bhat;           // f32 [tokens,H]         beta as the recurrence uses it (after the optional sigmoid)
  int64_t dec;            // f32 [chunks,H,K]       e^{G_last}: decay of each key channel over the whole chunk
  int64_t Ai;             // T [chunks,H,2,2]       Tm = (I + L)^-1 tiles
  int64_t AQ;             // T [chunks,H,2,2]       scale tril(sum_d q_i k_j e^{G_i-G_j}) tiles
  int64_t K1F;            // T [chunks,H,K/32,2]    rows -beta k . e^{G}
  int64_t K2F;            // T [chunks,H,K/32,2]    rows k . e^{G_last-G}
  int64_t QB;             // T [tokens,H,K]         rows scale q . e^{G}, row-major: written for the stand-alone output kernel only
  int64_t QBT;            // T [chunks,H,K/32,2]    (scale q . e^{G})^T as A operand: tile = (32 columns of K) x (32 tokens);
                          //                        written when the recurrence forms the output itself or a backward pass follows
  int64_t VF;             // T [chunks,H,V/32,2]    v_new
  int64_t HF;             // T [chunks,H,V/32,K/32] state before each chunk
  int64_t fwd_bytes;
  // kept for a backward pass
  int64_t TMR;            // T [chunks,H,64,64]     Tm row-major, as rounded for the tiles
  int64_t DVF;            // T [chunks,H,V/32,2]    d(v_new)
  int64_t DHF;            // T [chunks,H,V/32,K/32] gradient of the state AFTER each chunk
  int64_t DUMP;           // T [chunks,H][dQb | dK2 | P : 64,K each][dAq | a2 : 64,64 each]  sums over V of the chunk-local pass;
                          //   P as rows, the others as 32x32 tiles in fragment order: (token block, channel block), (row block, column block)
  int64_t DD;             // f32 [chunks,H,K]       sum over V of dS' . S: the gradient of the chunk's decay per channel
  int64_t PART;           // f32 [chunks,H][1 + K]  partial sums of dA_log and d(dt_bias)
  int64_t total_bytes;
  static int64_t dump_elems(int K) { return 3 * 64 * (int64_t)K + 2 * 64 * 64; }
};

inline KdaWorkspace kda_workspace_layout(const ChunkDims& d, int elem_bytes) {
  KdaWorkspace w;
  int64_t off = 0;
  auto take = [&](int64_t bytes) { int64_t o = off; off += align256(bytes); return o; };
  const int64_t nc = d.max_chunks(), H = d.Hv;
  w.chunk_offsets = take((int64_t)(d.N + 1) * 4);
  w.rstd = take(2 * nc * 64 * H * 4);
  w.bhat = take(d.tokens() * H * 4);
  w.dec = take(nc * H * d.K * 4);
  w.Ai = take(nc * 64 * H * 64 * elem_bytes);
  w.AQ = take(nc * 64 * H * 64 * elem_bytes);
  w.K1F = take(nc * 64 * H * d.K * elem_bytes);
  w.K2F = take(nc * 64 * H * d.K * elem_bytes);
  w.QB = take(d.tokens() * H * d.K * elem_bytes);
  w.QBT = take(nc * 64 * H * d.K * elem_bytes);
  w.VF = take(nc * 64 * H * d.V * elem_bytes);
  w.HF = take(nc * H * d.V * d.K * elem_bytes);
  w.fwd_bytes = off;
  w.TMR = take(nc * H * 64 * 64 * elem_bytes);
  w.DVF = take(nc * 64 * H * d.V * elem_bytes);
  w.DHF = take(nc * H * d.V * d.K * elem_bytes);
  w.DUMP = take(nc * H * KdaWorkspace::dump_elems(d.K) * elem_bytes);
  w.DD = take(nc * H * d.K * 4);
  w.PART = take(nc * H * (1 + d.K) * 4);
  w.total_bytes = off;
  return w;
}

// The two sequential kernels give one compute wave a 32-column slab of the state.  What limits them is the rate at
// which one CU gets its requests served (about 35 GB/s measured, loads and stores together), whatever the number of
// slabs the workgroup serves, so when the whole problem has no more slabs than the device has CUs every slab gets a
// workgroup (and a CU) of its own; larger problems put two slabs in a workgroup, which share the tiles.
int device_compute_units();   // defined with the forward launcher

inline bool one_slab_per_workgroup(const ChunkDims& d, int compute_units) {
  return (int64_t)d.N * d.Hv * (d.V / 32) <= compute_units;
}
// Two recurrences at once (a backward pass that refills the forward states on a second stream while the reverse
// recurrence runs): with two slabs per workgroup each of them is as fast as with one and needs half of the compute
// units, so both fit the device side by side.  Only needed where one slab per workgroup would take more than half.
inline bool two_slabs_to_share_device(const ChunkDims& d, int compute_units) {
  const int64_t slabs = (int64_t)d.N * d.Hv * (d.V / 32);
  return slabs <= compute_units && 2 * slabs > compute_units;
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

// The forward pass behind gdn_chunk_fwd_strided / gdn_chunk_fwd_norm_strided (defined with the forward kernels).
// workspace_state non-null: the workspace comes in two buffers, `workspace` holding the prep part and workspace_state
// the state part; skip_prep: the prep part already holds this input's tiles and is not computed again; share_device:
// the recurrence leaves half of the compute units to another one that runs beside it (two_slabs_to_share_device).
int chunk_fwd_entry(const void* q, const void* k, const void* v, int64_t q_stride, int64_t k_stride, int64_t v_stride,
                    const float* g, const void* beta, int beta_dtype, const float* initial_state,
                    const int64_t* cu_seqlens, void* o, float* final_state, void* workspace, int64_t workspace_bytes,
                    int B, int T, int N, int Hqk, int Hv, int K, int V, float scale, int use_qk_l2norm, int dtype,
                    const FwdNorm& fn, void* stream, void* workspace_state = nullptr, int64_t workspace_state_bytes = 0,
                    bool skip_prep = false, bool share_device = false);

inline int chunk_check_dims(const ChunkDims& d, int dtype) {
  if (d.B <= 0 || d.T <= 0 || d.N <= 0 || d.Hqk <= 0 || d.Hv <= 0 || d.Hv % d.Hqk != 0) return -2;
  if (d.varlen && d.B != 1) return -2;
  if (!d.varlen && d.N != d.B) return -2;
  if (d.K != 64 && d.K != 128) return -3;
  if (d.V <= 0 || d.V % 64 != 0) return -3;
  if (dtype != 0 && dtype != 1) return -4;
  // rows are moved in 16-byte pieces: strides must keep them aligned and cannot be shorter than a token's heads
  const int64_t vec = dtype == 0 ? 4 : 8, nq = (int64_t)d.Hqk * d.K, nv = (int64_t)d.Hv * d.V;
  const TokenStrides s = d.strides();
  if (s.q % vec || s.k % vec || s.v % vec || s.dq % vec || s.dk % vec || s.dv % vec) return -6;
  if (s.q < nq || s.k < nq || s.dq < nq || s.dk < nq || s.v < nv || s.dv < nv) return -6;
  return 0;
}

}  // namespace gdn
