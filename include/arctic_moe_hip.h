/*
 * C ABI of libarctic_moe_hip.so -- the MI355X (gfx950) expert-layer kernels that stand where
 * the reference binds its pybind11 module `ragged_ops`
 * (arctic_training/kernels/moe_ops/ragged_ops.cpp:12-26) and where its default path calls
 * torch ops (arctic_training/model/moe/moe.py:54-60, 176-193, 340-411, 450-461).
 *
 * Conventions (all entry points):
 *   - plain pointers and sizes only; every pointer is DEVICE memory owned by the caller
 *     (the reference's functions likewise fill caller-allocated tensors in place,
 *     top_k_gating.h:15-35, moe_scatter.h:16-29);
 *   - the library never allocates, frees or keeps a pointer past return;
 *   - `stream` is a hipStream_t passed as void*; work is stream-ordered, no host sync;
 *   - return 0 on success or a negative AMOE_ERR_* code; arguments are validated before
 *     the first HIP call, so argument errors can be exercised without a GPU;
 *     amoe_last_error() returns the calling thread's last message;
 *   - dtype: AMOE_F32, AMOE_BF16 or AMOE_F16 for activations / weights (the three types the
 *     reference's kernels dispatch, top_k_gating.cpp:56-59; the two 16-bit types share one
 *     kernel apart from the matrix instruction and the conversions); probabilities, scores and
 *     score gradients are always float32; indices are int32 (routed rows R = T*K < 2^31);
 *   - routed-row order is the reference's (moe.py:367-382): grouped by expert ascending,
 *     inside an expert ascending flat slot f = k*T + t.
 */
#ifndef ARCTIC_MOE_HIP_H
#define ARCTIC_MOE_HIP_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define AMOE_OK 0
#define AMOE_ERR_BAD_ARG (-1)     /* null pointer, non-positive size, bad enum */
#define AMOE_ERR_UNSUPPORTED (-2) /* shape outside what the kernels cover */
#define AMOE_ERR_WORKSPACE (-3)   /* workspace too small */
#define AMOE_ERR_LAUNCH (-4)      /* HIP reported a launch failure */

#define AMOE_F32 0
#define AMOE_BF16 1
#define AMOE_F16 2 /* IEEE half precision */

#define AMOE_ACT_SILU 0
#define AMOE_ACT_GELU 1
#define AMOE_ACT_RELU 2
#define AMOE_ACT_GPT_OSS 3 /* x * sigmoid(1.702 x), utils.py:118-123 */

#define AMOE_MAX_EXPERTS 512
#define AMOE_MAX_TOPK 16

/* library version (major*10000 + minor*100 + patch) */
int amoe_version(void);
/* message of the last error on the calling thread ("" if none) */
const char* amoe_last_error(void);

/*
 * Router softmax + top-k.  Replaces top_k_gating (top_k_gating.h:15-22,
 * top_k_gating_cuda.cu:74-147) and moe.py:360-366.
 *   logits [T,E] dtype  ->  probs [T,E] f32 (softmax evaluated in f32),
 *   topk_idx [T,K] i32 (value descending, lowest expert index first among equal logits),
 *   scores [T,K] f32 = the selected probabilities, divided by their sum when `normalize`,
 *   then rounded through `dtype` (the reference casts the scores to the model dtype).
 */
int amoe_router_topk_fwd(const void* logits, int dtype, int T, int E, int K, int normalize, float* probs,
                         int32_t* topk_idx, float* scores, void* stream);

/*
 * Router backward.  Replaces top_k_gating_bwd (top_k_gating.h:24-28,
 * top_k_gating_cuda.cu:243-294) plus the load-balance hook moe.py:393-406.
 *   d_scores [T,K] f32, probs [T,E] f32, topk_idx [T,K], counts [E] i32 (routed rows per
 *   expert) -> d_logits [T,E] dtype.
 *   d_probs = scatter(normalise-backward(d_scores)) + lb_coeff * counts/sum(counts);
 *   d_logits = probs * (d_probs - sum_e probs*d_probs).   lb_coeff = loss_coeff / T / ep_size.
 */
int amoe_router_bwd(const float* d_scores, const float* probs, const int32_t* topk_idx, const int32_t* counts,
                    int dtype, int T, int E, int K, int normalize, float lb_coeff, void* d_logits, void* stream);

/*
 * Permutation plan.  Replaces the atomics of top_k_gating plus the prefix sum and slot
 * computation of moe_scatter (moe_scatter_cuda.cu:69-139) with the deterministic order of
 * moe.py:367-382.
 *   assign [T,K] i32 (expert of slot (t,k)) ->
 *   counts [E], offsets [E+1] (exclusive prefix), token_of [R] (row -> token, the
 *   reference's token_mapped_slots), slot_of [R] (row -> flat slot f = k*T+t, the
 *   reference's pre-modulo permutation), row_of [T,K] (slot -> row, the custom path's
 *   mapped_slots).  Optionally scores [T,K] f32 -> scores_perm [R] f32, the scores in row
 *   order (moe.py:379); both may be null.
 *   workspace: amoe_permute_workspace_bytes(T*K, E) bytes.
 */
size_t amoe_permute_workspace_bytes(int R, int E);
int amoe_permute_plan(const int32_t* assign, const float* scores, int T, int K, int E, int32_t* counts,
                      int32_t* offsets, int32_t* token_of, int32_t* slot_of, int32_t* row_of, float* scores_perm,
                      void* workspace, size_t workspace_bytes, void* stream);

/*
 * amoe_permute_plan that also builds the tile map of the row-grouped GEMMs which will run over
 * its offsets (its scan kernel holds the offsets anyway, so the map costs no launch of its own).
 * gemm_workspace is the workspace those GEMMs will be given (amoe_grouped_gemm_workspace_bytes
 * (T*K, E) bytes); dtype and tile_cfg are theirs.  Every row-grouped GEMM over these offsets may
 * then pass tile_cfg | AMOE_TILE_MAP_READY.
 */
int amoe_permute_plan_tiled(const int32_t* assign, const float* scores, int T, int K, int E, int32_t* counts,
                            int32_t* offsets, int32_t* token_of, int32_t* slot_of, int32_t* row_of, float* scores_perm,
                            void* workspace, size_t workspace_bytes, void* gemm_workspace, size_t gemm_workspace_bytes,
                            int dtype, int tile_cfg, void* stream);

/*
 * amoe_permute_plan for callers that cannot allocate device memory (code recorded into a HIP
 * graph, tight serving loops, harnesses that forbid hipMalloc).  No counterpart in the
 * reference.  Same arguments and results as amoe_permute_plan without the workspace: the
 * per-chunk counters live in a fixed array of AMOE_PERMUTE_STATIC_MAX_COUNTS int32 (4 MiB) in
 * device memory that the library owns on every GPU it runs on until the process ends.  The call
 * allocates and frees nothing.  Limit: ceil(T*K/512) * E <= AMOE_PERMUTE_STATIC_MAX_COUNTS
 * (e.g. T*K = 1M routed rows at E = 512, or 4M at E = 128); beyond it AMOE_ERR_UNSUPPORTED.
 * All calls on one GPU share that array: calls that overlap in time on one GPU (two streams, two
 * threads) race; calls ordered on one stream are safe.  The first call on a device looks up the
 * array's device address (a host-side query, not a stream operation), so make it once before
 * recording a graph.
 */
#define AMOE_PERMUTE_STATIC_MAX_COUNTS (1 << 20)
int amoe_permute_plan_static(const int32_t* assign, const float* scores, int T, int K, int E, int32_t* counts,
                             int32_t* offsets, int32_t* token_of, int32_t* slot_of, int32_t* row_of,
                             float* scores_perm, void* stream);

/*
 * Row gather  xp[r,:] = x[token_of[r],:]  (moe.py:356; forward half of moe_scatter,
 * moe_scatter_cuda.cu:141-154).  x [T,H], xp [R,H].
 */
int amoe_gather_rows_fwd(const void* x, const int32_t* token_of, void* xp, int dtype, int R, int H, void* stream);

/*
 * Backward of the row gather (moe_scatter_backward, moe_scatter.h:25-29):
 *   dx[t,:] = (addend ? addend[t,:] : 0) + sum_k d_xp[row_of[t,k],:]   (f32 accumulate)
 */
int amoe_gather_rows_bwd(const void* d_xp, const int32_t* row_of, const void* addend, void* dx, int dtype, int T,
                         int K, int H, void* stream);

/*
 * Weighted combine  y[t,:] = sum_k scores[t,k] * moe_out[row_of[t,k],:]  (moe.py:450-461;
 * moe_gather, moe_gather.cpp:28-60), f32 accumulate, one rounding.  scores == null sums the
 * rows unweighted (for rows that were already scaled by their score upstream).
 */
int amoe_combine_fwd(const void* moe_out, const int32_t* row_of, const float* scores, void* y, int dtype, int T,
                     int K, int H, void* stream);

/*
 * Backward of the combine (moe_gather_backward, moe_gather.cpp:75-102) as the true
 * derivative of the forward above:
 *   d_moe_out[row_of[t,k],:] = dy[t,:] * scores[t,k];   d_scores[t,k] = <dy[t,:], moe_out[row,:]>.
 * d_moe_out may be null (only d_scores wanted).
 */
int amoe_combine_bwd(const void* dy, const void* moe_out, const int32_t* row_of, const float* scores,
                     void* d_moe_out, float* d_scores, int dtype, int T, int K, int H, void* stream);

/* workspace every grouped GEMM below needs (tile map built on the device from offsets) */
size_t amoe_grouped_gemm_workspace_bytes(int R, int E);

/*
 * May be OR-ed into `tile_cfg` of the three row-grouped GEMMs below: the workspace passed in
 * still holds the tile map that an earlier row-grouped call built from the same offsets, R, E,
 * dtype and tile shape, and nobody has written to it since; the map is then not built again
 * (the forward and backward GEMMs of one layer step all use the same map).
 */
#define AMOE_TILE_MAP_READY 0x100

/*
 * Grouped gate_up GEMM with the gated activation fused (moe.py:54-60 + 187-191):
 *   gate_up[rows_e, :] = xp[rows_e, :] @ w_gate_up[e]                          [R,2I]
 *   inter[r, i] = row_scale[r] * gate_up[r, 2i+1] * act(gate_up[r, 2i])        [R,I]
 * xp [R,H]; w_gate_up [E,H,2I] (gate in even, up in odd columns); offsets [E+1].
 * When `a_row_map` is non-null, row r of the A operand is read from xp[a_row_map[r], :]
 * (the gather of moe.py:356 folded into the GEMM; xp is then the un-permuted [T,H]).
 * row_scale [R] f32 may be null (= 1); passing the row-ordered scores folds the multiply of
 * moe.py:460 into this epilogue (the down projection is linear, so scaling its input rows
 * equals scaling its output rows).  gate_up may be null when only inter is wanted.
 * tile_cfg: 0 = library default; 1, 2, 3, 5 = other tile shapes, for tuning.  float16 with tile_cfg 3
 * is not built for any of the three row-grouped products (AMOE_ERR_UNSUPPORTED).
 * A (at most R source rows of H elements) and one expert of the weights must each stay below 4 GiB:
 * the kernels address them with 32-bit byte offsets (AMOE_ERR_UNSUPPORTED otherwise; the same holds
 * for the two products below and for amoe_grouped_gemm_nt_gated_bwd).
 */
int amoe_grouped_gemm_gateup_act_fwd(const void* xp, const int32_t* a_row_map, const void* w_gate_up,
                                     const int32_t* offsets, const float* row_scale, void* gate_up, void* inter,
                                     int dtype, int R, int E, int H, int I, int act, void* workspace,
                                     size_t workspace_bytes, int tile_cfg, void* stream);

/*
 * Grouped GEMM, B not transposed (moe.py:54-60):  C[rows_e,:] = A[rows_e,:] @ B[e]
 * A [R,Kd] (rows optionally gathered through a_row_map), B [E,Kd,N], C [R,N].  Used for
 * the down projection.
 */
int amoe_grouped_gemm_nn(const void* A, const int32_t* a_row_map, const void* B, const int32_t* offsets, void* C,
                         int dtype, int R, int E, int Kd, int N, void* workspace, size_t workspace_bytes,
                         int tile_cfg, void* stream);

/*
 * Grouped data-gradient GEMM:  C[rows_e,:] = A[rows_e,:] @ B[e]^T
 * A [R,N], B [E,Kd,N] (the forward weight), C [R,Kd].  The autograd of moe.py:59 w.r.t. A.
 */
int amoe_grouped_gemm_nt(const void* A, const int32_t* a_row_map, const void* B, const int32_t* offsets, void* C,
                         int dtype, int R, int E, int Kd, int N, void* workspace, size_t workspace_bytes,
                         int tile_cfg, void* stream);

/*
 * Data gradient of the down projection with the backward of the gated activation as its
 * epilogue (autograd of moe.py:187-192 through moe.py:59, plus the score gradient that the
 * reference takes in the backward of moe.py:460): d_inter = dy_rows @ w_down[e]^T is formed in
 * registers and never stored;
 *   d_gate_up[r,2i]   = row_scale[r] * d_inter[r,i] * up * act'(gate)
 *   d_gate_up[r,2i+1] = row_scale[r] * d_inter[r,i] * act(gate)          (gate, up) = gate_up[r,2i..2i+1]
 *   score_partials[p][r] = sum over the i of N tile p of d_inter[r,i] * up * act(gate)
 * dy [., H] (rows gathered through a_row_map when non-null), w_down [E,I,H], gate_up [R,2I] of
 * the forward pass, row_scale [R] f32 or null (= 1), d_gate_up [R,2I].  score_partials is
 * [amoe_gated_bwd_score_parts(I, tile_cfg)][R] f32 or null; summing it over p gives the gradient
 * of row_scale[r] (amoe_score_grad_gather does that and takes the rows back to their slots).
 * 16-bit dtypes only, tile_cfg 0, 1 or 2 (AMOE_ERR_UNSUPPORTED otherwise: such callers run
 * amoe_grouped_gemm_nt and amoe_gated_act_bwd).  Same result as those two calls up to the rounding of d_inter to the
 * model dtype, which this path skips.
 */
int amoe_gated_bwd_score_parts(int I, int tile_cfg);
int amoe_grouped_gemm_nt_gated_bwd(const void* dy, const int32_t* a_row_map, const void* w_down, const int32_t* offsets,
                                   const void* gate_up, const float* row_scale, void* d_gate_up, float* score_partials,
                                   int dtype, int R, int E, int I, int H, int act, void* workspace, size_t workspace_bytes,
                                   int tile_cfg, void* stream);

/*
 * d_scores[t,k] = sum_p score_partials[p][row_of[t,k]]: the row sums of
 * amoe_grouped_gemm_nt_gated_bwd (score_partials [n_parts][T*K]) added up in a fixed order and
 * taken from routed-row order back to the slots [T,K] (the scatter that autograd performs for
 * topk_scores[token_mapped_slots], moe.py:379).
 */
int amoe_score_grad_gather(const float* score_partials, int n_parts, const int32_t* row_of, float* d_scores, int T, int K,
                           void* stream);

/*
 * Grouped weight-gradient GEMM:  C[e] = A[rows_e,:]^T @ B[rows_e,:]   (zeros for an empty
 * expert).  A [R,Kd], B [R,N], C [E,Kd,N].  The autograd of moe.py:59 w.r.t. B[e].
 * One of the operands may be gathered: with a_row_map [R], row r of A is read from
 * A[a_row_map[r],:] (A then has as many rows as the map addresses); likewise b_row_map for B.
 * tile_cfg: 0 default, or 1, 2, 3, 5 (other tile shapes, for tuning).
 */
int amoe_grouped_gemm_wgrad(const void* A, const int32_t* a_row_map, const void* B, const int32_t* b_row_map,
                            const int32_t* offsets, void* C, int dtype, int R, int E, int Kd, int N, int tile_cfg,
                            void* stream);

/*
 * Backward of inter[r,i] = row_scale[r] * up * act(gate) (autograd of moe.py:189-191, and of
 * the score multiply of moe.py:460 when row_scale carries the scores):
 *   d_gate_up[r,2i]   = row_scale[r] * d_inter[r,i] * up * act'(gate)
 *   d_gate_up[r,2i+1] = row_scale[r] * d_inter[r,i] * act(gate)
 *   d_row_scale[t,k]  = sum_i d_inter[r,i] * up * act(gate)   for the slot (t,k) of row r
 * row_scale may be null (= 1).  d_row_scale [T,K] f32 may be null; when given, slot_of [R]
 * (row -> flat slot k*T+t) locates the slot and T*K must equal R.
 */
int amoe_gated_act_bwd(const void* gate_up, const void* d_inter, const float* row_scale, const int32_t* slot_of,
                       void* d_gate_up, float* d_row_scale, int dtype, int R, int I, int T, int K, int act,
                       void* stream);

/*
 * Expert-weight re-layout, checkpoint format -> ArcticMoE parameters.  Replaces the torch
 * stack / view / transpose sequence of remap_orig_moe_mlp_params_to_arctic_moe
 * (arctic_training/model/moe/utils.py:232-266):
 *   out[e][h][G*i + g] = in_g[e][i][h],   in_g [E, I, H] (nn.Linear weights, [out, in]),
 * G = 2 when in1 is given (in0 = gate_proj, in1 = up_proj -> expert_gate_up [E, H, 2I] with
 * gate in the even and up in the odd columns), G = 1 when in1 is null (down_proj [E, H', I']
 * passed as I = H', H = I' -> expert_down: a batched transpose).  in_expert_stride is the
 * distance in elements between experts of in0 / in1 (I*H when they are dense; 2*I*H when both
 * are halves of one fused [E, 2I, H] tensor).  out is dense.  Bit-exact.
 */
int amoe_remap_pack(const void* in0, const void* in1, void* out, int dtype, int E, int I, int H,
                    long long in_expert_stride, void* stream);

/*
 * The inverse, ArcticMoE parameters -> checkpoint format
 * (remap_arctic_moe_to_orig_moe_mlp_params, utils.py:366-395):
 *   out_g[e][i][h] = in[e][h][G*i + g],   G = 2 when out1 is given, else 1.
 */
int amoe_remap_unpack(const void* in, void* out0, void* out1, int dtype, int E, int I, int H,
                      long long out_expert_stride, void* stream);

#ifdef __cplusplus
}
#endif
#endif /* ARCTIC_MOE_HIP_H */
