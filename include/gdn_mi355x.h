/* C ABI of libgdn_mi355x.so -- MI355X (gfx950) kernels for the Gated DeltaNet operator path.
 *
 * The reference binds this path as Python callables chosen by a config string
 * (mindspeed_mm/fsdp/models/qwen3_5/modeling_qwen3_5.py:569-633); it has no FFI of its own.  The
 * entry points below are what a binding for that plugin slot calls: one launcher per operator,
 * raw device pointers and sizes only.
 *
 * Common rules
 *   - every pointer is device memory, tensors are dense (contiguous) in the stated layout unless an entry
 *     point takes strides;
 *   - dtype: 0 = fp32, 1 = bf16 (conv1d also 2 = fp16) and applies to q/k/v/o and their gradients;
 *     g, states and their gradients are always fp32; beta and its gradient are fp32 unless an entry point takes
 *     beta_dtype (0 = fp32, or equal to dtype: the layer's beta = sigmoid(b) is bf16, modeling_qwen3_5.py:833);
 *   - `stream` is a hipStream_t; launches are asynchronous, nothing allocates or synchronises;
 *   - return 0 on success, <0 for an invalid argument (-1 null pointer, -2 bad shape, -3 unsupported
 *     size, -4 bad dtype, -5 workspace too small, -6 bad stride or a pointer not 16-byte aligned), >0 is a
 *     hipError_t from the launch;
 *   - layouts: q,k [B,T,Hqk,K]; v,o [B,T,Hv,V]; g,beta [B,T,Hv]; states [N,Hv,K,V]; Hv % Hqk == 0
 *     (grouped heads are read in place, no expansion); with cu_seqlens (int64 [N+1], device) B == 1.
 */
#ifndef GDN_MI355X_H
#define GDN_MI355X_H
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* -------- chunked gated delta rule, forward + backward --------------------------------------
 * replaces chunk_gated_delta_rule_fwd / _bwd, mindspeed_mm/fsdp/ops/gdn/chunk_gated_delta_rule.py:30-174
 * (semantics of torch_chunk_gated_delta_rule, modeling_qwen3_5.py:398-475). K in {64,128}, V % 64 == 0.
 *
 * The workspace keeps what the backward pass needs (cumulative decay, Tm, per-chunk states, v_new);
 * gdn_chunk_bwd must be given a workspace a forward call on the same inputs filled, unchanged, sized with
 * with_backward = 1.  The workspace must be 256-byte aligned.  A forward call with o = NULL (and such a workspace)
 * only fills the workspace and writes no output: it is the recomputation step of a backward pass whose forward pass
 * kept nothing (chunk_gated_delta_rule.py:102-119 recomputes w, u, h, v_new the same way).  A forward call with a
 * workspace sized with with_backward = 0 writes neither per-chunk states nor v_new to memory.
 *
 * The workspace has two parts.  The prep part (with_backward = 2) holds what depends on q, k, g, beta only: the
 * cumulative decay, Tm, the intra-chunk Q K^T tiles and the K / Q^T tile images; the state part (with_backward = 3)
 * holds the per-chunk states, v_new and room for their gradients.  with_backward = 1 is both, contiguous.  A forward
 * call in a 16-bit dtype that writes o (and no fused norm) needs the prep part only.  gdn_chunk_bwd_parts takes the
 * two parts as separate buffers, so that a caller can keep the prep part of its forward call (0.28 GB at B=2, T=8192,
 * Hqk=16, Hv=32, d=128 in bf16, against 1.2 GB for both) and have the backward pass rebuild the state part.
 */
int64_t gdn_chunk_workspace_bytes(int B, int T, int N, int Hqk, int Hv, int K, int V, int dtype, int with_backward);

int gdn_chunk_fwd(const void* q, const void* k, const void* v, const float* g, const float* beta,
                  const float* initial_state, const int64_t* cu_seqlens, void* o, float* final_state,
                  void* workspace, int64_t workspace_bytes, int B, int T, int N, int Hqk, int Hv, int K, int V,
                  float scale, int use_qk_l2norm, int dtype, void* stream);

int gdn_chunk_bwd(const void* q, const void* k, const void* v, const float* g, const float* beta,
                  const float* initial_state, const int64_t* cu_seqlens, const void* d_o,
                  const float* d_final_state, void* dq, void* dk, void* dv, float* dg, float* dbeta,
                  float* d_initial_state, void* workspace, int64_t workspace_bytes, int B, int T, int N, int Hqk,
                  int Hv, int K, int V, float scale, int use_qk_l2norm, int dtype, void* stream);

/* The same pair for q, k, v (and dq, dk, dv) that are column slices of a wider token-major tensor, as the layer has
 * them after `torch.split(mixed_qkv, [key_dim, key_dim, value_dim], dim=-1)` of the convolution's output
 * (modeling_qwen3_5.py:818-831): x_stride is the distance between consecutive tokens in elements, the heads of a
 * token stay contiguous; 0 means dense.  Strides must be multiples of 16 bytes and the pointers 16-byte aligned.
 * The reference's Triton entry makes such views contiguous first (input_guard, triton/utils.py:210-239); reading
 * and writing them in place saves those copies and the concatenation of dq, dk, dv in the backward pass. */
int gdn_chunk_fwd_strided(const void* q, const void* k, const void* v, int64_t q_stride, int64_t k_stride,
                          int64_t v_stride, const float* g, const void* beta, const float* initial_state,
                          const int64_t* cu_seqlens, void* o, float* final_state, void* workspace,
                          int64_t workspace_bytes, int B, int T, int N, int Hqk, int Hv, int K, int V, float scale,
                          int use_qk_l2norm, int dtype, int beta_dtype, void* stream);

/* gdn_chunk_fwd_strided followed, inside its output kernel, by the layer's gated RMSNorm over head_v_dim
 * (Qwen3_5RMSNormGated.forward, modeling_qwen3_5.py:330-349, applied to the rule's output at :897-900):
 * y = (norm_weight * rmsnorm(o, eps)) * silu(gate), with the arithmetic and the bits of gdn_rmsnorm_gated_fwd below.
 * gate, y [tokens, Hv, V] dense in `dtype`; norm_weight [V] in `dtype` or fp32 (weight_dtype = 0).  o (the rule's
 * output) and rstd [tokens * Hv] fp32 are written only if non-null: a caller without a backward pass saves one write
 * and one read of o.  V must be 64 or 128 (a workgroup of the output kernel then holds whole rows), else -3. */
int gdn_chunk_fwd_norm_strided(const void* q, const void* k, const void* v, int64_t q_stride, int64_t k_stride,
                               int64_t v_stride, const float* g, const void* beta, const float* initial_state,
                               const int64_t* cu_seqlens, const void* gate, const void* norm_weight, void* o, void* y,
                               float* rstd, float* final_state, void* workspace, int64_t workspace_bytes, int B,
                               int T, int N, int Hqk, int Hv, int K, int V, float scale, float eps,
                               int use_qk_l2norm, int dtype, int weight_dtype, int beta_dtype, void* stream);

int gdn_chunk_bwd_strided(const void* q, const void* k, const void* v, int64_t q_stride, int64_t k_stride,
                          int64_t v_stride, const float* g, const void* beta, const float* initial_state,
                          const int64_t* cu_seqlens, const void* d_o, const float* d_final_state, void* dq, void* dk,
                          void* dv, int64_t dq_stride, int64_t dk_stride, int64_t dv_stride, float* dg, void* dbeta,
                          float* d_initial_state, void* workspace, int64_t workspace_bytes, int B, int T, int N,
                          int Hqk, int Hv, int K, int V, float scale, int use_qk_l2norm, int dtype, int beta_dtype,
                          void* stream);

/* The backward pass in phases, on a workspace given in two buffers (see gdn_chunk_workspace_bytes): any combination of
 *   1  refill the state part (forward recurrence without output; chunk_prep_kernel first unless prep_valid != 0,
 *      i.e. unless workspace_prep still holds what a forward call on the same inputs left there)
 *   2  the reverse recurrence
 *   4  the chunk-local kernels (dq, dk, dv, dg, dbeta); needs phases 1 and 2 of the same inputs done, and uses up what
 *      phase 2 left: with several value heads per q/k head it reuses the place of the state gradients it has read, so a
 *      second run of phase 4 needs phase 2 again
 * Phases 1 and 2 do not depend on each other: a caller may launch them on two streams and join both before phase 4.
 * Each of them is a latency-bound kernel with one workgroup per compute unit at most; for shapes whose slabs would fill
 * more than half of the device they are launched with two slabs per workgroup here, so that the two fit side by side
 * (same results, bit for bit).  Counterpart in the reference: the recomputation inside chunk_gated_delta_rule_bwd,
 * chunk_gated_delta_rule.py:102-119, followed by its stages :120-174.  Arguments a phase does not use may be NULL
 * (g for 2 and 4; d_o for 1; the gradient outputs for 1 and 2). */
int gdn_chunk_bwd_parts(const void* q, const void* k, const void* v, int64_t q_stride, int64_t k_stride,
                        int64_t v_stride, const float* g, const void* beta, const float* initial_state,
                        const int64_t* cu_seqlens, const void* d_o, const float* d_final_state, void* dq, void* dk,
                        void* dv, int64_t dq_stride, int64_t dk_stride, int64_t dv_stride, float* dg, void* dbeta,
                        float* d_initial_state, void* workspace_prep, int64_t workspace_prep_bytes,
                        void* workspace_state, int64_t workspace_state_bytes, int phases, int prep_valid, int B, int T,
                        int N, int Hqk, int Hv, int K, int V, float scale, int use_qk_l2norm, int dtype, int beta_dtype,
                        void* stream);

/* -------- fused recurrent gated delta rule (decode) ------------------------------------------
 * replaces the `recurrent_gated_delta_rule` slot (third-party fla kernel or
 * torch_recurrent_gated_delta_rule, modeling_qwen3_5.py:478-517, bound at :633, called at :877-886).
 * state_in may be NULL (zeros); state_out may be NULL or equal to state_in (updated in place).
 * K in {64,128,256}, V % 64 == 0.
 */
int gdn_recurrent_fwd(const void* q, const void* k, const void* v, const float* g, const float* beta,
                      const float* state_in, float* state_out, void* o, int B, int T, int Hqk, int Hv, int K,
                      int V, float scale, int use_qk_l2norm, int dtype, void* stream);

/* The same rule on packed sequences: q, k, v, g, beta, o hold one batch row of T tokens, cu_seqlens int64 [N+1] on the
 * device lists the N sequences, state_in / state_out are [N,Hv,K,V]; every sequence runs on its own from its own
 * state.  Counterpart: the `cu_seqlens` argument of the kernel bound in the same slot (third-party fla, un-vendored;
 * the in-tree torch fallback has none), with the meaning packed input has at the chunk entry
 * (chunk_gated_delta_rule.py:297-311).  Tokens outside every listed sequence are not written. */
int gdn_recurrent_fwd_packed(const void* q, const void* k, const void* v, const float* g, const float* beta,
                             const float* state_in, float* state_out, void* o, const int64_t* cu_seqlens, int N, int T,
                             int Hqk, int Hv, int K, int V, float scale, int use_qk_l2norm, int dtype, void* stream);

/* The same step reading q, k, v in place from the [tokens, D] output of the convolution (column ranges [0, Hqk K),
 * [Hqk K, 2 Hqk K), [2 Hqk K, 2 Hqk K + Hv V); token_stride >= that width, in elements, a multiple of 16 bytes) and
 * forming the gates from the layer's projections a, b [tokens, Hv] and parameters A_log, dt_bias [Hv] (in `dtype`
 * when param_dtype = dtype, fp32 when param_dtype = 0) as modeling_qwen3_5.py:833-841 does: the decode branch of
 * Qwen3_5GatedDeltaNet.forward (:738-744, :808-848, :877-886) is gdn_conv1d_update followed by this call. */
int gdn_recurrent_fwd_qkv(const void* qkv, int64_t token_stride, const void* a, const void* b, const void* A_log,
                          const void* dt_bias, const float* state_in, float* state_out, void* o, int B, int T,
                          int Hqk, int Hv, int K, int V, float scale, int use_qk_l2norm, int dtype, int param_dtype,
                          void* stream);

/* -------- causal short depthwise conv1d --------------------------------------------------------
 * replaces causal_conv1d_fwd_impl / causal_conv1d_bwd_impl / causal_conv1d_update_states,
 * mindspeed_mm/fsdp/ops/gdn/triton/convolution.py:517-588, 591-714, 762-787.
 * x,y,residual,dy,dx [B,T,D]; weight [W,D]; bias [D]; states [N,D,W]; activation 0 = none, 1 = SiLU.
 * W in 1..8; D % 8 == 0 (D % 4 for fp32).  dw [W,D] and db [D] are fp32.
 */
int gdn_conv1d_fwd(const void* x, const void* weight, const void* bias, const void* residual,
                   const void* initial_state, const int64_t* cu_seqlens, void* y, void* final_state, int B, int T,
                   int N, int D, int W, int activation, int dtype, void* stream);

int64_t gdn_conv1d_bwd_workspace_bytes(int B, int T, int D, int W);

int gdn_conv1d_bwd(const void* x, const void* dy, const void* weight, const void* bias, const void* initial_state,
                   const void* d_final_state, const int64_t* cu_seqlens, void* dx, float* dw, float* db,
                   void* d_initial_state, void* workspace, int64_t workspace_bytes, int B, int T, int N, int D,
                   int W, int activation, int dtype, void* stream);

/* decode-time update, replaces the `causal_conv1d_update` slot (torch_causal_conv1d_update,
 * modeling_qwen3_5.py:373-389, called at :738-744): hidden,out [B,T,D]; conv_state [B,D,state_len]
 * rolled in place; weight [D,W]; state_len >= W-1. */
int gdn_conv1d_update(const void* hidden, void* conv_state, const void* weight, const void* bias, void* out, int B,
                      int T, int D, int W, int state_len, int activation, int dtype, void* stream);

/* -------- gated RMSNorm (the step after the gated delta rule in the layer) -----------------------------
 * replaces Qwen3_5RMSNormGated.forward, modeling_qwen3_5.py:330-349 (called on [tokens*Hv, head_v_dim] rows at
 * :897-900): y = (weight * (x * rsqrt(mean(x^2) + eps))) * silu(gate), intermediate casts to the input dtype as
 * in the reference.  x, gate, y, dy, dx, dgate [rows, N]; weight [N] in the input dtype (weight_dtype = dtype) or
 * fp32 (weight_dtype = 0); rstd [rows] fp32 is written by the forward and read by the backward; dweight [N] fp32.
 * N * element size / 16 must be 4, 8, 16, 32 or 64 (bf16: N = 32 ... 512; fp32: N = 16 ... 256).
 * gate_activation = 1 replaces KimiK_3_MoeRMSNormGated.forward of the KDA layer instead,
 * mindspeed_mm/fsdp/models/kimi_k3/modeling_kimi_linear.py:75-96 (called at :741 on rows of head_dim elements):
 * y = (weight * (x * rsqrt(mean(x^2) + eps))) * sigmoid(gate), the sigmoid cast to the input dtype before the
 * product; the result is in the input dtype. */
int gdn_rmsnorm_gated_fwd(const void* x, const void* gate, const void* weight, void* y, float* rstd, int64_t rows,
                          int N, float eps, int dtype, int weight_dtype, int gate_activation, void* stream);

int64_t gdn_rmsnorm_gated_bwd_workspace_bytes(int64_t rows, int N);

int gdn_rmsnorm_gated_bwd(const void* x, const void* gate, const void* weight, const float* rstd, const void* dy,
                          void* dx, void* dgate, float* dweight, void* workspace, int64_t workspace_bytes,
                          int64_t rows, int N, int dtype, int weight_dtype, int gate_activation, void* stream);

/* -------- gates of the rule from the layer's projections -------------------------------------------------
 * replaces the elementwise chain in Qwen3_5GatedDeltaNet.forward, modeling_qwen3_5.py:833-841:
 * beta = sigmoid(b) (in b's dtype), g = -exp(A_log) * softplus(a + dt_bias) (fp32).  a, b, beta, da, db, dbeta
 * [tokens, Hv] in `dtype`; A_log, dt_bias [Hv] in `dtype` (param_dtype = dtype) or fp32 (param_dtype = 0); g, dg
 * [tokens, Hv] fp32; dA_log, ddt_bias [Hv] fp32.  Hv <= 256. */
int gdn_gate_fwd(const void* a, const void* b, const void* A_log, const void* dt_bias, float* g, void* beta,
                 int64_t tokens, int Hv, int dtype, int param_dtype, void* stream);

int64_t gdn_gate_bwd_workspace_bytes(int64_t tokens, int Hv);

int gdn_gate_bwd(const void* a, const void* b, const void* A_log, const void* dt_bias, const float* dg,
                 const void* dbeta, void* da, void* db, float* dA_log, float* ddt_bias, void* workspace,
                 int64_t workspace_bytes, int64_t tokens, int Hv, int dtype, int param_dtype, void* stream);

/* gdn_gate_bwd without the workspace argument.  No counterpart in the reference: it exists for callers that cannot
 * allocate device memory around the call (a step under HIP graph capture, a loop whose harness forbids hipMalloc).
 * The per-workgroup partial sums live in a 1 MiB buffer inside the library (one per device, held until the process
 * ends), which limits Hv to 128 (-3 beyond); any number of tokens is accepted.  Same kernels and same order of
 * additions as gdn_gate_bwd: identical results.  Calls that overlap on one device (two streams) share that buffer and
 * race; calls on one stream are ordered.  Nothing is allocated, freed or synchronised.  The first call on each device
 * looks the buffer's address up (hipGetSymbolAddress, which may load the code object): make that one call, with any
 * small input, before a capture begins or a no-allocation region is entered; every later call only launches kernels. */
int gdn_gate_bwd_noalloc(const void* a, const void* b, const void* A_log, const void* dt_bias, const float* dg,
                         const void* dbeta, void* da, void* db, float* dA_log, float* ddt_bias, int64_t tokens, int Hv,
                         int dtype, int param_dtype, void* stream);

/* -------- KDA (Kimi delta attention): the delta rule with one decay per key channel ------------------
 * replaces: chunk_kda (mindspeed_mm/fsdp/ops/kda/triton_ascend/chunk.py:215-407, the fused operator the layer calls at
 * mindspeed_mm/fsdp/models/kimi_k3/modeling_kimi_linear.py:681-699) and its pure-PyTorch statement chunk_kda_naive
 * (mindspeed_mm/fsdp/ops/kda/chunk_kda_naive.py:223-381; gate :76-104, chunk algebra :106-221).
 * q, k, g [B,T,H,K], v, o [B,T,H,V], beta [B,T,H] (token-major, contiguous); q, k, v, o in `dtype` (0 fp32, 1 bf16),
 * g in g_dtype and beta in beta_dtype (each 0 = fp32 or equal to dtype); A_log [H] and dt_bias [H*K] (or null) in fp32;
 * initial_state, final_state [N,H,K,V] fp32 or null; cu_seqlens int64 [N+1] on the device or null (then N = B).
 * use_gate: g is the raw gate input and the log decay is -e^{A_log} softplus(g + dt_bias), or, with has_lower_bound,
 * lower_bound * sigmoid(e^{A_log} (g + dt_bias)); otherwise g is the log decay itself (<= 0).
 * beta_sigmoid: beta <- sigmoid(beta), times 2 with allow_neg_eigval.  K in {64, 128}, V a multiple of 64.
 * A workspace of gdn_kda_workspace_bytes(..., with_backward = 1, ...) bytes also keeps Tm as rows, 1/|q|, 1/|k| and
 * the places of the backward pass's intermediates (the cumulative decay is not kept: gdn_kda_bwd rebuilds it from g,
 * A_log and dt_bias).  Returns 0, or -1 null argument, -2 shape, -3 unsupported K / V, -4 dtype, -5 workspace,
 * -6 alignment. */
int64_t gdn_kda_workspace_bytes(int B, int T, int N, int H, int K, int V, int with_backward, int dtype);

int gdn_kda_fwd(const void* q, const void* k, const void* v, const void* g, const void* beta, const float* A_log,
                const float* dt_bias, const float* initial_state, const int64_t* cu_seqlens, void* o,
                float* final_state, void* workspace, int64_t workspace_bytes, int B, int T, int N, int H, int K, int V,
                float scale, int use_qk_l2norm, int use_gate, int has_lower_bound, float lower_bound, int beta_sigmoid,
                int allow_neg_eigval, int dtype, int g_dtype, int beta_dtype, void* stream);

/* chunk_kda(..., return_intermediate_states=True) (chunk_kda_naive.py:287-303, :375-380; triton_ascend/chunk.py:149-151,
 * an inference-time option): the state at the entry of every chunk of 64 tokens, from the workspace a gdn_kda_fwd call
 * with the same B, T, N, H, K, V, dtype and cu_seqlens filled; that workspace must have the size
 * gdn_kda_workspace_bytes gives with with_backward = 1 (a forward-only workspace does not keep the states: -5).  h_out [h_chunks, H, K, V], or [h_chunks, H, V, K] with
 * transpose_state_layout, in `dtype`; chunk c of batch row b is row b * ceil(T/64) + c, packed input lists the chunks
 * of its sequences in order (h_chunks = sum of ceil(len/64); chunks past h_chunks are not written). */
int gdn_kda_intermediate_states(const void* workspace, int64_t workspace_bytes, const int64_t* cu_seqlens, void* h_out,
                                int64_t h_chunks, int B, int T, int N, int H, int K, int V, int transpose_state_layout,
                                int dtype, void* stream);

/* Backward pass of gdn_kda_fwd: needs the workspace that call filled when it was sized with with_backward = 1, and the
 * same q, k, v, g, A_log, dt_bias, cu_seqlens and options.  The reference has no hand-written counterpart in its tree
 * (it differentiates chunk_kda_naive.py:106-221 with autograd; the fused operator's backward,
 * triton_ascend/chunk.py:172-213, calls kernels of a package that is not part of it).  d_o [B,T,H,V] in `dtype`;
 * d_final_state [N,H,K,V] fp32 or null.  Written: dq, dk [B,T,H,K] and dv [B,T,H,V] in `dtype`, dg [B,T,H,K] in g_dtype
 * (gradient of the raw gate input when use_gate is set, of the log decay otherwise), dbeta [B,T,H] in beta_dtype
 * (gradient of beta as handed in, i.e. before the sigmoid when beta_sigmoid is set), dA_log [H] and ddt_bias [H*K]
 * fp32 (each may be null; written only with use_gate), d_initial_state [N,H,K,V] fp32 or null. */
int gdn_kda_bwd(const void* q, const void* k, const void* v, const void* g, const float* A_log, const float* dt_bias,
                const int64_t* cu_seqlens, const void* d_o, const float* d_final_state, void* dq, void* dk, void* dv,
                void* dg, void* dbeta, float* dA_log, float* ddt_bias, float* d_initial_state, void* workspace,
                int64_t workspace_bytes, int B, int T, int N, int H, int K, int V, float scale, int use_qk_l2norm,
                int use_gate, int has_lower_bound, float lower_bound, int beta_sigmoid, int allow_neg_eigval, int dtype,
                int g_dtype, int beta_dtype, void* stream);

/* -------- per-kernel timing ------------------------------------------------------------------------
 * op-level counterpart of the reference's step profiler (mindspeed_mm/fsdp/tools/profiler.py:32-147).
 * While enabled, every kernel launch of this library is bracketed by HIP events on its stream (this mode
 * creates events, i.e. it allocates); gdn_profile_collect waits for them and ADDS, per kernel id
 * (0 .. gdn_profile_kernel_count()-1), the elapsed milliseconds to total_ms[id] and 1 to launches[id]. */
int gdn_profile_enable(int on);
int gdn_profile_kernel_count(void);
const char* gdn_profile_kernel_name(int id);
int gdn_profile_collect(double* total_ms, int64_t* launches);

#ifdef __cplusplus
}
#endif
#endif
