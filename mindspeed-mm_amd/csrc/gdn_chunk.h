// Host-side description of the workspace shared by the chunked forward and backward passes.
#pragma once
#include <stdint.h>

namespace gdn {

struct ChunkDims {
  int B, T, N, Hqk, Hv, K, V;
  bool varlen;
  int64_t tokens() const { return (int64_t)B * T; }
  // upper bound on the number of 64-token chunks; exact without cu_seqlens.  Packed sequences add at
  // most one partial chunk each, so the bound needs no look at the (device-resident) lengths.
  int64_t max_chunks() const {
    if (!varlen) return (int64_t)B * ((T + 63) / 64);
    return tokens() / 64 + N;
  }
};

// Byte offsets into the workspace.  Everything the backward pass re-reads is written by the forward.
struct ChunkWorkspace {
  int64_t chunk_offsets;  // int32 [N+1]      chunks before each packed sequence
  int64_t qn, kn;         // T [tokens,Hqk,K] l2-normalised q,k (only with use_qk_l2norm)
  int64_t G;              // f32 [tokens,Hv]  chunk-local cumulative log decay
  int64_t Ai;             // T [tokens,Hv,64] rows of (I + A)^-1
  int64_t W;              // T [tokens,Hv,K]
  int64_t AQ;             // T [tokens,Hv,64] rows of tril(Q K^T . Gam) (unscaled)
  int64_t U;              // T [chunks,Hv,V/32,2,64,16] U in accumulator-fragment order (see chunk_prep_kernel)
  int64_t VN;             // T [tokens,Hv,V]  v_new = U - W S (kept for the backward pass)
  int64_t H;              // T [chunks,Hv,K,V] state BEFORE each chunk
  int64_t fwd_bytes;
  int64_t DV;             // T [tokens,Hv,V]  d(v_new)
  int64_t DH;             // T [chunks,Hv,K,V] gradient of the state AFTER each chunk
  int64_t DW;             // T [tokens,Hv,K]
  int64_t DQH, DKH;       // T [tokens,Hv,K]  per-value-head dq, dk before the group sum
  int64_t DG;             // f32 [tokens,Hv]  gradient w.r.t. the cumulative decay (two partial terms)
  int64_t DB;             // f32 [tokens,Hv]
  int64_t total_bytes;
};

inline int64_t align256(int64_t x) { return (x + 255) / 256 * 256; }

inline ChunkWorkspace chunk_workspace_layout(const ChunkDims& d, int elem_bytes) {
  ChunkWorkspace w;
  int64_t off = 0;
  auto take = [&](int64_t bytes) { int64_t o = off; off += align256(bytes); return o; };
  const int64_t tok = d.tokens(), nc = d.max_chunks();
  w.chunk_offsets = take((int64_t)(d.N + 1) * 4);
  w.qn = take(tok * d.Hqk * d.K * elem_bytes);
  w.kn = take(tok * d.Hqk * d.K * elem_bytes);
  w.G = take(tok * d.Hv * 4);
  w.Ai = take(tok * d.Hv * 64 * elem_bytes);
  w.W = take(tok * d.Hv * d.K * elem_bytes);
  w.AQ = take(tok * d.Hv * 64 * elem_bytes);
  w.U = take(nc * 64 * d.Hv * d.V * elem_bytes);
  w.VN = take(tok * d.Hv * d.V * elem_bytes);
  w.H = take(nc * d.Hv * d.V * d.K * elem_bytes);
  w.fwd_bytes = off;
  w.DV = take(tok * d.Hv * d.V * elem_bytes);
  w.DH = take(nc * d.Hv * d.V * d.K * elem_bytes);
  w.DW = take(tok * d.Hv * d.K * elem_bytes);
  w.DQH = take(tok * d.Hv * d.K * elem_bytes);
  w.DKH = take(tok * d.Hv * d.K * elem_bytes);
  w.DG = take(tok * d.Hv * 4);
  w.DB = take(tok * d.Hv * 4);
  w.total_bytes = off;
  return w;
}

inline int chunk_check_dims(const ChunkDims& d, int dtype) {
  if (d.B <= 0 || d.T <= 0 || d.N <= 0 || d.Hqk <= 0 || d.Hv <= 0 || d.Hv % d.Hqk != 0) return -2;
  if (d.varlen && d.B != 1) return -2;
  if (!d.varlen && d.N != d.B) return -2;
  if (d.K != 64 && d.K != 128) return -3;
  if (d.V <= 0 || d.V % 64 != 0) return -3;
  if (dtype != 0 && dtype != 1) return -4;
  return 0;
}

}  // namespace gdn
