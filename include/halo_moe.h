/*
 * halo_moe.h -- C ABI of the MI355X (gfx950) MoE expert-path kernels.
 *
 * The reference has no FFI on this path: its boundary is the Python API of the halo/kernels ops and of the MoE block's
 * _compute_experts.  Each entry point below names the reference function whose device work it replaces
 * (paths relative to the reference checkout).  The Python package halo_amd binds these with ctypes.
 *
 * Conventions
 *   - every pointer is a device pointer owned by the caller (outputs and workspaces included); nothing is
 *     allocated, nothing is read back to the host, no call synchronises;
 *   - `stream` is a hipStream_t passed as void*; all work is enqueued on it;
 *   - row strides are in elements; `dtype` is an hmoe_dtype;
 *   - return value: 0 on success, a negative hmoe_status otherwise (hmoe_status_string names it);
 *   - re-entrant: no mutable global state, safe to call from autograd's backward thread (the one exception,
 *     hmoe_route_sort_static, says so where it is declared).
 */
#ifndef HALO_MOE_H
#define HALO_MOE_H

#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

typedef enum { HMOE_F32 = 0, HMOE_BF16 = 1 } hmoe_dtype;

typedef enum {
  HMOE_OK = 0,
  HMOE_INVALID_ARGUMENT = -1, /* a null pointer, a negative size, an unknown enum */
  HMOE_UNSUPPORTED = -2,      /* a shape or dtype no kernel covers (alignment, top_k or expert count too large) */
  HMOE_LAUNCH_FAILED = -3     /* hipGetLastError() after the launch was not hipSuccess */
} hmoe_status;

/* GLU activation ids, as halo/kernels/fused_glu.py:23-25. */
typedef enum { HMOE_GLU_SILU = 0, HMOE_GLU_GELU_TANH = 1, HMOE_GLU_CLAMPED_SILU = 2 } hmoe_glu_activation;

/* Router gate-weight rules. */
typedef enum {
  HMOE_ROUTER_SOFTMAX_ALL = 0, /* softmax over all experts, gather, optional renormalise (Qwen3 family) */
  HMOE_ROUTER_SOFTMAX_TOPK = 1 /* softmax over the k selected logits (gpt-oss) */
} hmoe_router_mode;

int hmoe_abi_version(void);
const char* hmoe_status_string(int status);

/* ------------------------------------------------------------------------------------------------ routing sort
 * Replaces _CountingSort.forward: halo/kernels/moe_route_sort.py:128-179 (kernels :40-125).
 * Stable counting sort of the valid slots (0 <= expert < num_local_experts) of experts[n_rows, top_k] by expert;
 * slot = row * top_k + k.  Outputs: sorted_token_idx i64[n_valid], sorted_weights[n_valid] (same element size as
 * weights), sorted_expert_ids[n_valid] (same integer type as experts), offs i32[num_local_experts] inclusive group
 * ends, inv_map i64[n_rows, top_k] (each row's sorted positions ascending, padded with n_valid), dest
 * i32[n_rows*top_k] (each slot's sorted position, n_valid for a dropped slot), ok i32[1] = (number of valid slots ==
 * n_valid).  When ok is 0 nothing past n_valid is written.  experts_elem_bytes is 4 or 8, weight_elem_bytes 2, 4 or 8.
 * Workspace: hmoe_route_sort_workspace_bytes(...) bytes, 16-byte aligned.  Three launches, no atomics on global
 * memory.
 */
int64_t hmoe_route_sort_workspace_bytes(int64_t n_rows, int top_k, int num_local_experts);
int hmoe_route_sort(const void* experts, int experts_elem_bytes, const void* weights, int weight_elem_bytes,
                    int64_t n_rows, int top_k, int num_local_experts, int64_t n_valid, int64_t* sorted_token_idx,
                    void* sorted_weights, void* sorted_expert_ids, int32_t* offs, int64_t* inv_map, int32_t* dest,
                    int32_t* ok, void* workspace, void* stream);

/* hmoe_route_sort without a workspace argument and without any allocation.  No counterpart in the reference: it is
 * for callers that cannot allocate device memory (code under HIP graph capture, tight serving loops, harnesses that
 * forbid hipMalloc).  Same arguments, outputs, launches and bits as hmoe_route_sort; the histogram / start table lives
 * in a 4 MiB device array inside the library (one copy per GPU, held until the process ends), whose address is looked
 * up once per device on the first call made with that device current.  A routing whose table does not fit
 * (hmoe_route_sort_workspace_bytes(...) > 4 MiB, i.e. sort blocks x local experts > 2^20) returns HMOE_UNSUPPORTED.
 * Calls that overlap on one GPU (two streams, two threads) share the array and race: serialise them per GPU.  Nothing
 * in the array needs clearing between calls: every entry read is written by the same call first.  The first call made
 * with a device current looks the array's address up (hipGetSymbolAddress, which may load the library's code object on
 * that device): make that call outside any stream capture; every later call on the device only launches kernels. */
int hmoe_route_sort_static(const void* experts, int experts_elem_bytes, const void* weights, int weight_elem_bytes,
                           int64_t n_rows, int top_k, int num_local_experts, int64_t n_valid,
                           int64_t* sorted_token_idx, void* sorted_weights, void* sorted_expert_ids, int32_t* offs,
                           int64_t* inv_map, int32_t* dest, int32_t* ok, void* stream);

/* Replaces _CountingSort.backward: halo/kernels/moe_route_sort.py:181-189.
 * grad_weights[slot] = dest[slot] < n_valid ? grad_sorted[dest[slot]] : 0. */
int hmoe_route_sort_bwd(const void* grad_sorted, const int32_t* dest, int64_t n_slots, int64_t n_valid,
                        int elem_bytes, void* grad_weights, void* stream);

/* Replaces sync_free_bincount: halo/kernels/histogram.py:9-18.
 * out[v] = number of indices equal to v (weights null) or the sum of their f32 weights, for 0 <= v < size; out is
 * f32 (out_is_i64 == 0) or i64 (counts only).  Indices outside [0, size) are ignored.  No limit on n or size: up to
 * 65536 indices and 8192 bins one workgroup counts in LDS; beyond that the output is cleared and many workgroups add
 * their shares with vector atomics (LDS counters first where the bins fit).  Counts are exact either way; a weighted
 * sum's order is not fixed (as the reference's scatter_add_), and a float count above 2^24 rounds as float32 does. */
int hmoe_bincount(const int64_t* indices, const float* weights, int64_t n, int64_t size, int out_is_i64, void* out,
                  void* stream);

/* ------------------------------------------------------------------------------------------- permute / combine
 * Replaces MoEGatherPermute.forward (tokens.index_select): halo/kernels/moe_permute.py:133-136, and
 * MoEExpertBiasGather.forward: :197-200.  out[j, :] = src[index[j], :]. */
int hmoe_gather_rows(const void* src, int64_t src_row_stride, const int64_t* index, int64_t n_out, int64_t hidden,
                     int dtype, void* out, void* stream);

/* Replaces _gather_reduce_kernel: halo/kernels/moe_permute.py:17-41, 92-112 (permute backward without a weight,
 * weighted unpermute forward with one).  out[r] = sum_k w[j] * src[j], j = inv_map[r, k] < n_src; fp32 multiply and
 * accumulate in slot order k = 0..top_k-1, one rounding to dtype.  weight may be null; it has src's dtype. */
int hmoe_gather_reduce(const void* src, const void* weight, const int64_t* inv_map, int64_t n_out, int top_k,
                       int64_t n_src, int64_t hidden, int dtype, void* out, void* stream);

/* The same with a second term added in the same pass: out[r] = round(round(sum) + round(scale[r] * addend[r])), the
 * roundings where the tensor operations `combined + scale * addend` have them.  Replaces the `routed + shared_fn()` of
 * _dispatch_compute_combine_shared (halo/distributed/expert_parallel/layer.py:270-299) behind the weighted unpermute,
 * with Qwen3.5's sigmoid gate on the shared expert (families/qwen3_5.py:41-42) as `addend_scale` [n_out] (null: no
 * scale).  addend is [n_out, hidden] with rows addend_row_stride elements apart, null for the plain reduction. */
int hmoe_gather_reduce_add(const void* src, const void* weight, const int64_t* inv_map, int64_t n_out, int top_k,
                           int64_t n_src, int64_t hidden, int dtype, const void* addend, int64_t addend_row_stride,
                           const void* addend_scale, void* out, void* stream);

/* Replaces _weighted_unpermute_bwd_kernel: halo/kernels/moe_permute.py:44-72, 158-189.
 * grad_expert[j] = w[j] * grad_out[tok[j]];  grad_weights[j] = <grad_out[tok[j]], expert_out[j]> in fp32 when
 * expert_out and grad_weights are non-null. */
int hmoe_unpermute_bwd(const void* grad_out, int64_t grad_out_row_stride, const void* expert_out,
                       const void* weights, const int64_t* token_idx, int64_t n_sorted, int64_t hidden, int dtype,
                       void* grad_expert, float* grad_weights, void* stream);

/* Replaces MoEExpertBiasGather.backward (one-hot GEMM): halo/kernels/moe_permute.py:202-208.
 * grad_bias[e, :] = sum of grad_out rows j with eids[j] == e, fp32 accumulate in row order, one rounding.
 * eids must be non-decreasing (expert-sorted rows, the only order the expert path produces).
 * workspace: hmoe_expert_colsum_workspace_bytes(...) bytes, 16-byte aligned, or NULL.  With it (and 16-byte-aligned
 * rows) the rows are summed in blocks of 128 whatever their expert and the block sums added per expert in block order,
 * two launches, so that one overloaded expert does not hold the launch up; without it, one workgroup per (expert,
 * column chunk).  Either way the order of the additions is fixed. */
int64_t hmoe_expert_colsum_workspace_bytes(int64_t n_rows, int64_t width, int num_experts);
int hmoe_expert_colsum(const void* grad_out, const int64_t* eids, int64_t n_rows, int64_t width, int num_experts,
                       int dtype, void* grad_bias, void* workspace, void* stream);

/* --------------------------------------------------------------------------------------------------- fused GLU
 * Replaces _glu_fwd_kernel / _glu_bwd_kernel: halo/kernels/fused_glu.py:118-205.  gate/up (and dgate/dup) are
 * row-strided so a packed [gate | up] buffer is read and its gradient written in place.  fp32 math. */
int hmoe_glu_fwd(const void* gate, const void* up, int64_t stride_gate, int64_t stride_up, int64_t n_rows,
                 int64_t width, int dtype, int activation, float alpha, float limit, int clamp_activated,
                 int up_plus_one, void* out, void* stream);
int hmoe_glu_bwd(const void* gate, const void* up, int64_t stride_gate, int64_t stride_up, const void* grad_out,
                 int64_t n_rows, int64_t width, int dtype, int activation, float alpha, float limit,
                 int clamp_activated, int up_plus_one, void* dgate, void* dup, int64_t stride_dgate,
                 int64_t stride_dup, void* stream);

/* The same pair with the combine's gate weight folded in (one weight per row, in the operands' dtype):
 *   fwd:  out[r] = round(w[r] * glu(gate[r], up[r]))             (fp32 product, one rounding)
 *   bwd:  (dgate, dup) = glu_grad(gate, up, w[r] * grad_out[r]),  grad_weight[r] = <grad_out[r], glu(gate[r], up[r])>
 * with grad_out the gradient of the weighted rows and grad_weight f32[n_rows], summed in fp32 in a fixed order.
 * Together with hmoe_grouped_gemm_dgrad_gather / _wgrad_gather_grad they replace the weight's multiply in
 * _gather_reduce_kernel (halo/kernels/moe_permute.py:33-41) and all of _weighted_unpermute_bwd_kernel (:44-72): since
 * sum_k w_k (act_k @ W) = sum_k (w_k act_k) @ W, the down projection runs on weighted rows, the combine is a plain
 * sum, and its backward needs neither the [R, H] gradient of the expert outputs nor the expert outputs themselves
 * (grad_weight[r] = <grad_out[tok r], y[r]> = <grad_out[tok r] @ W^T, act[r]>).
 * row_weight is [n_rows] of weight_dtype: `dtype`, or HMOE_F32 with bf16 operands, in which case each weight is rounded
 * to bf16 on the way in and each grad_weight value on the way out: the bits of casting the weights first
 * (sorted_weights.to(dtype), moe_layer/compute.py:241) and of the gradient that cast hands back, without the three
 * small cast launches. */
int hmoe_glu_fwd_weighted(const void* gate, const void* up, int64_t stride_gate, int64_t stride_up,
                          const void* row_weight, int weight_dtype, int64_t n_rows, int64_t width, int dtype,
                          int activation, float alpha, float limit, int clamp_activated, int up_plus_one, void* out,
                          void* stream);
int hmoe_glu_bwd_weighted(const void* gate, const void* up, int64_t stride_gate, int64_t stride_up,
                          const void* grad_out, const void* row_weight, int weight_dtype, int64_t n_rows,
                          int64_t width, int dtype, int activation, float alpha, float limit, int clamp_activated,
                          int up_plus_one, void* dgate, void* dup, int64_t stride_dgate, int64_t stride_dup,
                          float* grad_weight, void* stream);

/* ------------------------------------------------------------------------------------------------------ router
 * Replaces the softmax / top-k / renormalise / cast sequence of the family routers the layer calls
 * (halo/distributed/expert_parallel/moe_layer/shared_experts_layer.py:44-56; weights as routing.py:110-122 and
 * families/gpt_oss.py:82-84).  One wavefront per token.  indices i64[n_tokens, top_k] in descending score, equal
 * scores in ascending expert index; weights f32[n_tokens, top_k] hold values rounded to the logits' dtype. */
int hmoe_router_topk_fwd(const void* logits, int dtype, int64_t n_tokens, int num_experts, int top_k, int mode,
                         int normalize, float eps, int64_t* indices, float* weights, void* stream);
/* Gradient of the gate weights with respect to the logits (the router's softmax/renorm backward, aten in the
 * reference).  grad_logits[n_tokens, num_experts] in the logits' dtype. */
int hmoe_router_topk_bwd(const void* logits, int dtype, const int64_t* indices, const float* grad_weights,
                         int64_t n_tokens, int num_experts, int top_k, int mode, int normalize, float eps,
                         void* grad_logits, void* stream);

/* ------------------------------------------------------------------------------------------------ shared-expert gate
 * Replace the sigmoid output gate of a shared expert, torch.sigmoid(self.shared_expert_gate(hidden_states)) with
 * shared_expert_gate = nn.Linear(H, 1, bias=False) (halo/distributed/expert_parallel/families/qwen3_5.py:41-42), and
 * its autograd.  gate[t] = sigmoid(<x[t], w>) for x [n_rows, hidden] (row stride ldx) and w [hidden], in the operands'
 * dtype, rounded where the tensor operations round (the dot product in fp32 then rounded, the sigmoid in fp32 then
 * rounded).  hidden and ldx multiples of 16 bytes, x and w 16-byte aligned (HMOE_UNSUPPORTED otherwise). */
int hmoe_row_gate_fwd(const void* x, int64_t ldx, const void* w, int64_t n_rows, int hidden, int dtype, void* gate,
                      void* stream);
/* Backward: gs[t] = round(grad_gate[t] * (1 - gate[t]) * gate[t]); grad_x[t] = gs[t] * w (row stride ld_grad_x; may be
 * NULL) and grad_w = sum_t gs[t] * x[t] (may be NULL), the sum in fp32 in a fixed order through `workspace`
 * (hmoe_row_gate_bwd_workspace_bytes(n_rows, hidden) bytes, caller-owned; needed when grad_w is given). */
int64_t hmoe_row_gate_bwd_workspace_bytes(int64_t n_rows, int hidden);
int hmoe_row_gate_bwd(const void* x, int64_t ldx, const void* w, const void* gate, const void* grad_gate,
                      int64_t n_rows, int hidden, int dtype, void* grad_x, int64_t ld_grad_x, void* grad_w,
                      void* workspace, void* stream);

/* ------------------------------------------------------------------------------------------------ device probe
 * No counterpart in the reference: a measuring stick for benchmarks.  Runs `iterations` rounds of eight independent
 * bf16 MFMAs per wavefront on register operands, two wavefronts per SIMD on every compute unit, and returns the
 * floating-point operations the launch performs (time it with events on `stream`), or a negative hmoe_status.
 * shape 0 = v_mfma_f32_32x32x16_bf16 (what the GEMM kernels issue), 1 = v_mfma_f32_16x16x32_bf16; operands 0 = small
 * integers (few bits toggle), 1 = pseudo-random values of mixed sign (the power real operands draw: the clock the part
 * holds, and so the rate, depends on it).  `sink` is a device buffer of at least one float per compute unit (never
 * written in practice). */
int64_t hmoe_probe_mfma_bf16(int64_t iterations, int shape, int operands, void* sink, void* stream);
/* The same kind of stick for the memory side: reads `bytes` (a multiple of 16, 16-byte aligned) from `src` once with
 * non-temporal 16-byte fetches and stores nothing; returns the bytes read, or a negative hmoe_status.  `sink` is 16
 * bytes of device memory (never written in practice). */
int64_t hmoe_probe_hbm_read(const void* src, int64_t bytes, void* sink, void* stream);

/* ------------------------------------------------------------------------------------------------ grouped GEMM
 * Replace F.grouped_mm as called by halo/kernels/grouped_mm.py:16-47 (forward :39, dgrad :25, wgrad :26).
 * offs i32[num_groups] are inclusive row ends (null: one group holding every row).  b is [num_groups, K, N]
 * contiguous.  fp32 accumulate, one rounding to dtype.  Rows past offs[num_groups-1] are not written by
 * fwd/dgrad.  An empty group's wgrad is exact zeros.  Deterministic (no split accumulation across workgroups).
 * The bf16 products exist in three tile configurations with the same bits: a 256 x 256 output tile on one workgroup
 * per compute unit, a 128 x 256 tile on two and a 128 x 128 tile on three; each call takes the largest of which the
 * product has at least one tile per compute unit.
 */

/* Forces a tile configuration for every later bf16 product of the process: 0 = by size (the default), 1 = 256 x 256,
 * 2 = 128 x 256, 3 = 128 x 128; the environment variable HALO_GEMM_TILE=mono|duo|small sets the initial value.
 * Returns the previous setting, or HMOE_INVALID_ARGUMENT.  A tuning and test switch with no counterpart in the
 * reference; the one piece of process-wide state besides hmoe_route_sort_static's table, and harmless to race on
 * (all tiles give the same bits). */
int hmoe_set_gemm_tile(int tile);
int hmoe_grouped_gemm_fwd(const void* a, int64_t lda, const void* b, const int32_t* offs, int64_t total_rows,
                          int num_groups, int64_t k, int64_t n, int dtype, void* out, int64_t ldo, void* stream);
int hmoe_grouped_gemm_dgrad(const void* grad_out, int64_t ldg, const void* b, const int32_t* offs,
                            int64_t total_rows, int num_groups, int64_t k, int64_t n, int dtype, void* grad_a,
                            int64_t lda, void* stream);
int hmoe_grouped_gemm_wgrad(const void* a, int64_t lda, const void* grad_out, int64_t ldg, const int32_t* offs,
                            int64_t total_rows, int num_groups, int64_t k, int64_t n, int dtype, void* grad_b,
                            void* stream);

/* The forward GEMM plus the expert's bias row: replaces `out + MoEExpertBiasGather.apply(bias, eids)` behind a grouped
 * projection (halo/distributed/expert_parallel/families/gpt_oss.py:153-159 with halo/kernels/moe_permute.py:192-200).
 * bias is [num_groups, N] in dtype; rows of group g get bias[g].  The product is rounded to dtype first and the sum
 * rounded again, as the two tensor operations it replaces do, so the result is theirs bit for bit. */
int hmoe_grouped_gemm_fwd_bias(const void* a, int64_t lda, const void* b, const void* bias, const int32_t* offs,
                               int64_t total_rows, int num_groups, int64_t k, int64_t n, int dtype, void* out,
                               int64_t ldo, void* stream);

/* The forward product scaled and added to an existing [total_rows, n] tensor: out = addend + scale * (a[s:e] @ b[g]),
 * element by element with the roundings of those tensor operations (the product to dtype, its multiple by scale to
 * dtype, the sum to dtype).  Replaces the `out + scaling * grouped_mm(hidden, lora_b)` of the adapted expert projection
 * (halo/distributed/expert_parallel/moe_layer/compute.py:283-294): the low-rank delta joins the base projection in the
 * second adapter product's epilogue, so neither the delta nor its multiple is written.  out may be addend itself. */
int hmoe_grouped_gemm_fwd_addto(const void* a, int64_t lda, const void* b, const int32_t* offs, int64_t total_rows,
                                int num_groups, int64_t k, int64_t n, int dtype, const void* addend,
                                int64_t ld_addend, float scale, void* out, int64_t ldo, void* stream);

/* The input gradient added to an existing [total_rows, k] tensor: grad_a = addend + grad_out[s:e] @ b[g]^T, element by
 * element with the roundings of the two tensor operations (the product to dtype, the sum to dtype).  Where two
 * projections read the same rows (gate and up stored apart, halo/distributed/expert_parallel/families/gpt_oss.py:
 * 139-152), autograd adds their two input gradients (the sum the engine forms at the rows' node); here the second
 * projection's input gradient joins the first's in its epilogue, so neither the second product nor the pass that adds
 * the two exists.  grad_a may be addend itself. */
int hmoe_grouped_gemm_dgrad_addto(const void* grad_out, int64_t ldg, const void* b, const int32_t* offs,
                                  int64_t total_rows, int num_groups, int64_t k, int64_t n, int dtype,
                                  const void* addend, int64_t ld_addend, void* grad_a, int64_t lda, void* stream);

/* The same two GEMMs with the rows of A gathered: logical row r of A is a[row_index[r]], a holding a_rows rows; an
 * index outside [0, a_rows) reads as a row of zeros.  This folds MoEGatherPermute.forward
 * (halo/kernels/moe_permute.py:133-136, tokens.index_select(0, sorted_token_idx)) into the first expert GEMM and its
 * weight gradient (halo/kernels/grouped_mm.py:39, :26), so the permuted copy of the tokens is never written.
 * bf16 only (HMOE_UNSUPPORTED otherwise). */
int hmoe_grouped_gemm_fwd_gather(const void* a, int64_t lda, int64_t a_rows, const int64_t* row_index, const void* b,
                                 const int32_t* offs, int64_t total_rows, int num_groups, int64_t k, int64_t n,
                                 int dtype, void* out, int64_t ldo, void* stream);
int hmoe_grouped_gemm_wgrad_gather(const void* a, int64_t lda, int64_t a_rows, const int64_t* row_index,
                                   const void* grad_out, int64_t ldg, const int32_t* offs, int64_t total_rows,
                                   int num_groups, int64_t k, int64_t n, int dtype, void* grad_b, void* stream);
/* hmoe_grouped_gemm_fwd_gather with the expert's bias row added in the epilogue as hmoe_grouped_gemm_fwd_bias adds it
 * (halo/distributed/expert_parallel/families/gpt_oss.py:154-160 over the rows of halo/kernels/moe_permute.py:133-136):
 * a biased projection that fetches its rows through the sort's index.  bf16 only. */
int hmoe_grouped_gemm_fwd_gather_bias(const void* a, int64_t lda, int64_t a_rows, const int64_t* row_index,
                                      const void* b, const void* bias, const int32_t* offs, int64_t total_rows,
                                      int num_groups, int64_t k, int64_t n, int dtype, void* out, int64_t ldo,
                                      void* stream);

/* The two gradients of a product whose OUTPUT rows were then summed per token (the plain combine behind a down
 * projection on weighted rows): logical row r of the output gradient is grad_out[row_index[r]], grad_out holding
 * grad_rows rows (the tokens' gradient, read in place: no [R, N] gradient of the expert outputs is written).
 *   dgrad_gather:       grad_a[s:e] = grad_out[row_index[s:e]] @ b[g]^T
 *   wgrad_gather_grad:  grad_b[g]   = a[s:e]^T @ grad_out[row_index[s:e]]
 * Replace F.grouped_mm's two gradients (halo/kernels/grouped_mm.py:25-26) fed by _weighted_unpermute_bwd_kernel
 * (halo/kernels/moe_permute.py:44-72).  bf16 only. */
int hmoe_grouped_gemm_dgrad_gather(const void* grad_out, int64_t ldg, int64_t grad_rows, const int64_t* row_index,
                                   const void* b, const int32_t* offs, int64_t total_rows, int num_groups, int64_t k,
                                   int64_t n, int dtype, void* grad_a, int64_t lda, void* stream);
int hmoe_grouped_gemm_wgrad_gather_grad(const void* a, int64_t lda, const void* grad_out, int64_t ldg,
                                        int64_t grad_rows, const int64_t* row_index, const int32_t* offs,
                                        int64_t total_rows, int num_groups, int64_t k, int64_t n, int dtype,
                                        void* grad_b, void* stream);

/* ------------------------------------------------------------------------------------------------- block fp8
 * Replaces quantize_block_fp8: halo/kernels/lowp/block_fp8.py:23-34.  w is [batch, rows, cols]; q (e4m3fn bytes)
 * has its shape; scale is f32 [batch, ceil(rows/128), ceil(cols/128)], a power of two per 128x128 block. */
int hmoe_quantize_block_fp8(const void* w, int dtype, int64_t batch, int64_t rows, int64_t cols, uint8_t* q,
                            float* scale, void* stream);
/* Inverse (halo/checkpoint/tools/fp8_dequant.py:153-170): out = q * scale, one rounding to dtype. */
int hmoe_dequantize_block_fp8(const uint8_t* q, const float* scale, int64_t batch, int64_t rows, int64_t cols,
                              int dtype, void* out, void* stream);
/* Forward grouped GEMM with block-fp8 weights (the quantised-weight configuration): a bf16 [total_rows, K],
 * bq e4m3fn [num_groups, K, N] with b_scale f32 [num_groups, ceil(K/128), ceil(N/128)]; out bf16. */
int hmoe_grouped_gemm_fwd_fp8w(const void* a, int64_t lda, const uint8_t* bq, const float* b_scale,
                               const int32_t* offs, int64_t total_rows, int num_groups, int64_t k, int64_t n,
                               void* out, int64_t ldo, void* stream);

/* ----------------------------------------------------------------------------------- fp8 MFMA (activations too)
 * The quantised-weight configuration on the e4m3 matrix instruction.  The reference holds no kernel of its own for
 * it: block_fp8_quantization_config (halo/kernels/lowp/block_fp8.py:37-46) hands the checkpoint to the serving
 * engine with "activation_scheme": "dynamic", i.e. activations quantised per row and 128 values at run time.
 *
 * Both operands of the product lie in panels of 64 contraction values, [k / 64][rows][64], so that a tile's share
 * of one pipeline stage is a single contiguous run.
 *
 * hmoe_quantize_rows_fp8: x bf16 [x_rows, k] (row stride ldx) to q e4m3fn [k / 64][out_rows][64] and scale u8
 * [k / 128][out_rows]: values [64 p, 64 p + 64) of row r at q[(p * out_rows + r) * 64], and at
 * scale[b * out_rows + r] the biased exponent byte (e8m0) of the power-of-two scale of the row's block b of 128
 * values, the smallest that brings the block's largest magnitude to 448 or below.  Row r is x[row_index[r]] (the permute by expert of MoEGatherPermute, halo/kernels/moe_permute.py:130-141,
 * taken on the way; an index outside [0, x_rows) gives a row of zeros), or x[r] with row_index NULL (then x_rows ==
 * rows).  k must be a multiple of 128, out_rows >= rows. */
int hmoe_quantize_rows_fp8(const void* x, int64_t ldx, const int64_t* row_index, int64_t x_rows, int64_t rows, int64_t k,
                           uint8_t* q, uint8_t* scale, int64_t out_rows, void* stream);
/* hmoe_glu_fwd with its output quantised on the way: what hmoe_quantize_rows_fp8 makes of hmoe_glu_fwd's bf16
 * output, bit for bit (each value is rounded to bf16 before it is scaled), without that output being written.  bf16
 * operands with 16-byte rows, width a multiple of 128; q and scale as hmoe_quantize_rows_fp8 writes them. */
int hmoe_glu_fwd_quant_fp8(const void* gate, const void* up, int64_t stride_gate, int64_t stride_up, int64_t n_rows,
                           int64_t width, int activation, float alpha, float limit, int clamp_activated,
                           int up_plus_one, uint8_t* q, uint8_t* scale, int64_t out_rows, void* stream);
/* out bf16 [total_rows, n] = per group, (a_q * a_scale) [rows, k] @ (bq * b_scale) [k, n]: a_q and a_scale as
 * written by hmoe_quantize_rows_fp8 with out_rows = a_rows; bq e4m3fn [num_groups][k / 64][n][64] (value (kk, c)
 * of expert g at bq[((g * (k / 64) + kk / 64) * n + c) * 64 + kk % 64]) and b_scale f32
 * [num_groups, k / 128, ceil(n / 128)], not negative, any mantissa.  Accumulation in fp32, one rounding to bf16.
 * k must be a multiple of 128, n of 8. */
int hmoe_grouped_gemm_fwd_fp8(const uint8_t* a_q, const uint8_t* a_scale, int64_t a_rows, const uint8_t* bq,
                              const float* b_scale, const int32_t* offs, int64_t total_rows, int num_groups, int64_t k,
                              int64_t n, void* out, int64_t ldo, void* stream);

/* ------------------------------------------------------------------------------------------------------- MXFP8
 * The reference's "mxfp8" quant_format (halo/kernels/lowp/spec.py:11): e4m3 elements with one e8m0 power-of-two scale
 * per 32 values along the contraction axis.  expert_gemm(quant_format="mxfp8") of the reference is the bf16 product of
 * the two fake-quantised operands (halo/kernels/expert_gemm.py:33-38); here the quantised operands go to the scaled
 * e4m3 matrix instruction, which applies a scale per 32 values by itself, so the same products are summed in fp32
 * without the dequantised copies being read.
 *
 * hmoe_quantize_rows_mxfp8 replaces quantize_mxfp8(t, axis=-1) (halo/kernels/lowp/quantization.py:154-188, 236-245)
 * for x [x_rows, k] (HMOE_BF16 or HMOE_F32, row stride ldx): q e4m3fn in panels [ceil(k / 64)][out_rows][64] (values
 * [64 p, 64 p + 64) of row r at q[(p * out_rows + r) * 64]) and scale u8 [k / 32][out_rows], at
 * scale[b * out_rows + r] the e8m0 code of row r's block b: the biased exponent e + 127 of the smallest power of two
 * 2^e >= amax / 448, e clamped to [-127, 127]; 254 for a block holding an inf, 0xFF for one holding a NaN.  Row r is
 * x[row_index[r]] (an index outside [0, x_rows) gives zeros) or x[r] with row_index NULL.  k must be a multiple of 32.
 *
 * hmoe_dequantize_rows_mxfp8 replaces dequantize (quantization.py:277-297) for that pair: out bf16 [rows, k] =
 * code * 2^(scale - 127), q and scale holding q_rows rows.
 *
 * hmoe_quantize_weight_mxfp8 replaces quantize_mxfp8(w, axis=1) for expert weights w [groups, k, n]: q e4m3fn
 * [groups][ceil(k / 64)][n][64] (value (kk, c) of expert g at q[((g * ceil(k / 64) + kk / 64) * n + c) * 64 + kk % 64])
 * and scale u8 [groups][k / 32][n]; with dequant not NULL also the round trip's result (quantization.py:307-311) as
 * bf16 [groups, k, n], which the straight-through backward multiplies by.
 *
 * hmoe_grouped_gemm_fwd_mxfp8: out bf16 [total_rows, n] = per group, dequant(a_q, a_scale)[rows, k] @
 * dequant(bq, b_scale)[g]: operands as the two quantisers write them (a_rows = their out_rows); accumulation in fp32,
 * one rounding to bf16.  k must be a multiple of 64, n of 8. */
int hmoe_quantize_rows_mxfp8(const void* x, int dtype, int64_t ldx, const int64_t* row_index, int64_t x_rows,
                             int64_t rows, int64_t k, uint8_t* q, uint8_t* scale, int64_t out_rows, void* stream);
int hmoe_dequantize_rows_mxfp8(const uint8_t* q, const uint8_t* scale, int64_t q_rows, int64_t rows, int64_t k,
                               void* out, int64_t ldo, void* stream);
int hmoe_quantize_weight_mxfp8(const void* w, int dtype, int64_t groups, int64_t k, int64_t n, uint8_t* q,
                               uint8_t* scale, void* dequant, void* stream);
int hmoe_grouped_gemm_fwd_mxfp8(const uint8_t* a_q, const uint8_t* a_scale, int64_t a_rows, const uint8_t* bq,
                                const uint8_t* b_scale, const int32_t* offs, int64_t total_rows, int num_groups,
                                int64_t k, int64_t n, void* out, int64_t ldo, void* stream);

/* Whether hmoe_grouped_gemm_fwd_mxfp8 (panel_values 64) / hmoe_grouped_gemm_fwd_mxfp4 (panel_values 128) can address
 * operands of these sizes.  The quantised activations and the output may be of any size (the kernel rebases their
 * descriptors per pipeline stage and per tile); one expert's quantised weights, the rows' exponent bytes (counted as
 * four per row and panel) and 256 output rows (256 x ldo x 2 bytes) must each stay below 2 GiB; beyond that the entry
 * points return HMOE_UNSUPPORTED and a caller multiplies the round-tripped operands on the bf16 kernels (what
 * halo_amd.kernels.expert_gemm does).  1 or 0; launches nothing. */
int hmoe_grouped_gemm_mx_fits(int64_t a_rows, int64_t total_rows, int64_t k, int64_t n, int64_t ldo, int panel_values);

/* ------------------------------------------------------------------------------------------------------- MXFP4
 * The reference's "mxfp4" quant_format (halo/kernels/lowp/spec.py:11): e2m1 elements (magnitudes 0, 0.5, 1, 1.5, 2, 3,
 * 4, 6; code = sign << 3 | level) with one e8m0 power-of-two scale per 32 values along the contraction axis.
 * expert_gemm(quant_format="mxfp4") of the reference is the bf16 grouped product of the two fake-quantised operands
 * (halo/kernels/expert_gemm.py:33-38), and so it is here: these entries produce the round trip's bf16 result in one pass
 * (and the packed codes and exponents of the quantiser API), the product is hmoe_grouped_gemm_fwd's.
 *
 * hmoe_mxfp4_rows replaces quantize_mxfp4(t, axis=-1), dequantize and their composition the fake-quant round trip
 * (halo/kernels/lowp/quantization.py:154-180, 191-198, 208-211, 248-266, 277-297, 307-311) for x [x_rows, k] (HMOE_BF16
 * or HMOE_F32, row stride ldx).  Row r is x[row_index[r]] (an index outside [0, x_rows) gives zeros) or x[r] with
 * row_index NULL.  The block's scale code is the biased exponent e + 127 of the smallest power of two 2^e >= amax / 6,
 * e clamped to [-127, 127]; 254 for a block holding an inf, 0xFF for one holding a NaN.  An element's code is the level
 * nearest to |v| 2^-e (clamped to 6), a tie going to the level with the even code, with the sign of v 2^-e.  Outputs,
 * each optional (NULL), at least one of packed and round_trip given, scale required with packed: packed u8
 * [rows, k / 2] (element 2 i in the low nibble of byte i, 2 i + 1 in the high), scale u8 [rows, k / 32], round_trip
 * bf16 [rows, k] (row stride ldo) = level * sign * 2^(scale - 127).  k must be a multiple of 32.
 *
 * hmoe_mxfp4_weight is the same along axis 1 of expert weights w [groups, k, n] (quantize_mxfp4(w, axis=1)): packed u8
 * [groups, k / 2, n] (rows 2 i and 2 i + 1 of k in byte (i, c), the even one low), scale u8 [groups, k / 32, n],
 * round_trip bf16 [groups, k, n].
 *
 * hmoe_mxfp4_dequantize_rows replaces dequantize (quantization.py:277-297) for the pair hmoe_mxfp4_rows writes.
 *
 * The same products on the scaled matrix instruction with e2m1 operands (twice the e4m3 rate, a quarter of bf16's
 * operand bytes): hmoe_mxfp4_rows_panels and hmoe_mxfp4_weight_panels write the operands as the kernel loads them, in
 * panels of 128 contraction values (64 bytes): rows q [ceil(k / 128)][out_rows][64] (value 2 b of panel p of row r in
 * the low nibble of q[(p * out_rows + r) * 64 + b]) with scale u8 [ceil(k / 128)][out_rows][4] (the panel's four block
 * exponents side by side); weights q [groups][ceil(k / 128)][n][64] with scale [groups][ceil(k / 128)][n][4] and, with
 * round_trip not NULL, the round trip's bf16 [groups, k, n] for the straight-through backward.  Values past k are
 * zeros (code 0, exponent 0).  hmoe_mxfp4_dequantize_panels gives rows back as bf16 [rows, k] from that layout (q_rows
 * rows per panel).  hmoe_grouped_gemm_fwd_mxfp4: out bf16 [total_rows, n] = per group, dequant(a)[rows, k] @
 * dequant(b)[g] with a_rows = the row operand's out_rows; accumulation in fp32, one rounding to bf16; k a multiple of
 * 32, n of 8. */
int hmoe_mxfp4_rows(const void* x, int dtype, int64_t ldx, const int64_t* row_index, int64_t x_rows, int64_t rows,
                    int64_t k, uint8_t* packed, uint8_t* scale, void* round_trip, int64_t ldo, void* stream);
int hmoe_mxfp4_weight(const void* w, int dtype, int64_t groups, int64_t k, int64_t n, uint8_t* packed, uint8_t* scale,
                      void* round_trip, void* stream);
int hmoe_mxfp4_dequantize_rows(const uint8_t* packed, const uint8_t* scale, int64_t rows, int64_t k, void* out,
                               int64_t ldo, void* stream);
int hmoe_mxfp4_rows_panels(const void* x, int dtype, int64_t ldx, const int64_t* row_index, int64_t x_rows, int64_t rows,
                           int64_t k, uint8_t* q, uint8_t* scale, int64_t out_rows, void* stream);
int hmoe_mxfp4_weight_panels(const void* w, int dtype, int64_t groups, int64_t k, int64_t n, uint8_t* q, uint8_t* scale,
                             void* round_trip, void* stream);
int hmoe_mxfp4_dequantize_panels(const uint8_t* q, const uint8_t* scale, int64_t q_rows, int64_t rows, int64_t k,
                                 void* out, int64_t ldo, void* stream);
int hmoe_grouped_gemm_fwd_mxfp4(const uint8_t* a_q, const uint8_t* a_scale, int64_t a_rows, const uint8_t* bq,
                                const uint8_t* b_scale, const int32_t* offs, int64_t total_rows, int num_groups,
                                int64_t k, int64_t n, void* out, int64_t ldo, void* stream);
/* The two MX products with an expert bias row added in the epilogue: out = bf16(product) + bias[g] per row of group g,
 * each of the two rounded to bf16 as the reference's two tensor operations round (_expert_proj, then
 * + MoEExpertBiasGather.apply(bias, eids): halo/moe_layer/families/gpt_oss.py:153-159).  bias bf16 [num_groups, n]. */
int hmoe_grouped_gemm_fwd_mxfp8_bias(const uint8_t* a_q, const uint8_t* a_scale, int64_t a_rows, const uint8_t* bq,
                                     const uint8_t* b_scale, const void* bias, const int32_t* offs, int64_t total_rows,
                                     int num_groups, int64_t k, int64_t n, void* out, int64_t ldo, void* stream);
int hmoe_grouped_gemm_fwd_mxfp4_bias(const uint8_t* a_q, const uint8_t* a_scale, int64_t a_rows, const uint8_t* bq,
                                     const uint8_t* b_scale, const void* bias, const int32_t* offs, int64_t total_rows,
                                     int num_groups, int64_t k, int64_t n, void* out, int64_t ldo, void* stream);

/* ------------------------------------------------------------------------------------------------------- NVFP4
 * The reference's "nvfp4" quant_format (halo/kernels/lowp/spec.py:11): e2m1 elements, two per byte, with one e4m3
 * scale per 16 values along the contraction axis and one fp32 power-of-two scale per tensor
 * (halo/kernels/lowp/quantization.py:209-226: global = the smallest power of two >= amax_tensor / 2688, scale =
 * e4m3(min(amax_block / 6 / global, 448)), code = e2m1(value / (f32(scale) * global)), a zero divisor taken as 1).
 * expert_gemm(quant_format="nvfp4") of the reference is the bf16 grouped product of the two fake-quantised operands
 * (halo/kernels/expert_gemm.py:33-38), and so it is here: the scaled matrix instruction takes power-of-two scales only.
 *
 * tensor_amax: one float in device memory, the largest magnitude of the whole tensor (NaN if it holds one), reduced by
 * the caller.  hmoe_nvfp4_rows replaces quantize_nvfp4(t, axis=-1), dequantize and the round trip
 * (quantization.py:248-270, 277-297, 307-311) for x [x_rows, k] (HMOE_BF16 or HMOE_F32, row stride ldx; row r is
 * x[row_index[r]], zeros for an index outside [0, x_rows), or x[r] with row_index NULL).  Outputs, each optional (NULL),
 * at least one of packed and round_trip given, scale required with packed: packed u8 [rows, k / 2] (element 2 i in the
 * low nibble of byte i), scale u8 [rows, k / 16] (e4m3fn bits), round_trip bf16 [rows, k] (row stride ldo), global_out
 * (one float: the tensor's scale).  k must be a multiple of 16.  hmoe_nvfp4_weight is the same along axis 1 of
 * w [groups, k, n] under one scale for the whole bank: packed [groups, k / 2, n], scale [groups, k / 16, n], round_trip
 * bf16 [groups, k, n].  hmoe_nvfp4_dequantize_rows gives rows back as bf16 = level * sign * (f32(scale) * global). */
int hmoe_nvfp4_rows(const void* x, int dtype, int64_t ldx, const int64_t* row_index, int64_t x_rows, int64_t rows,
                    int64_t k, const float* tensor_amax, uint8_t* packed, uint8_t* scale, void* round_trip, int64_t ldo,
                    float* global_out, void* stream);
int hmoe_nvfp4_weight(const void* w, int dtype, int64_t groups, int64_t k, int64_t n, const float* tensor_amax,
                      uint8_t* packed, uint8_t* scale, void* round_trip, float* global_out, void* stream);
int hmoe_nvfp4_dequantize_rows(const uint8_t* packed, const uint8_t* scale, const float* global_scale, int64_t rows,
                               int64_t k, void* out, int64_t ldo, void* stream);

#ifdef __cplusplus
}
#endif
#endif /* HALO_MOE_H */
