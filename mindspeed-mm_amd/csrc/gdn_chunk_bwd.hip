#include "gdn_chunk.h"
#include "gdn_common.h"
extern "C" int gdn_chunk_bwd(const void* q, const void* k, const void* v, const float* g, const float* beta,
                  const float* initial_state, const int64_t* cu_seqlens, const void* d_o,
                  const float* d_final_state, void* dq, void* dk, void* dv, float* dg, float* dbeta,
                  float* d_initial_state, void* workspace, int64_t workspace_bytes, int B, int T, int N, int Hqk,
                  int Hv, int K, int V, float scale, int use_qk_l2norm, int dtype, void* stream) { return -100; }
