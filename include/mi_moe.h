/*
 * mi_moe.h -- C ABI of the MI355X (gfx950) scattered-MoE forward kernels.
 *
 * One shared library (libmi_moe.so), plain C types only.  Every function
 *   - takes device pointers the CALLER allocated (inputs, outputs and workspace); the library
 *     never allocates, frees or keeps a pointer after it returns (mi_moe_sort_bin_static, which brings
 *     its own fixed scratch array, is the one documented exception to "workspace");
 *   - validates its arguments on the host BEFORE anything is launched and returns
 *       0  on success,
 *      <0  an MI_MOE_E* argument / shape / alignment / dtype error (nothing was launched),
 *      >0  the hipError_t of a failed launch;
 *   - is asynchronous: work is enqueued on `stream` (a hipStream_t passed as void*, NULL = the
 *     default stream); there is no host synchronisation and no device-to-host copy;
 *   - is re-entrant and keeps no mutable global state (values the library reads once and then only
 *     reads back -- device attributes, the address of that scratch array -- are cached per device).
 *
 * Index tensors are int32 inside the ABI.  Matrices are row-major and contiguous.  Expert weights
 * are read in the module's native (E, out_features, in_features) layout, i.e. the contraction
 * dimension is contiguous for both operands; no transposed copy is ever made.
 *
 * The reference reaches this path through a Python function boundary into the external
 * `cute_kernels` package (lm_engine/hf_models/modeling_utils/mlp_blocks/moe.py:22-24); each entry
 * point below names the reference call site it stands in for.
 */
#ifndef MI_MOE_H
#define MI_MOE_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define MI_MOE_ABI_VERSION 1

/* element types of activations / weights / logits */
#define MI_MOE_F32 0
#define MI_MOE_F16 1
#define MI_MOE_BF16 2

/* error codes (negative) */
#define MI_MOE_OK 0
#define MI_MOE_ENULL (-1)      /* a required pointer is NULL */
#define MI_MOE_ESHAPE (-2)     /* a dimension is out of the supported range */
#define MI_MOE_EDTYPE (-3)     /* unsupported element type for this entry point */
#define MI_MOE_EALIGN (-4)     /* a pointer or leading dimension is not aligned as required */
#define MI_MOE_EWORKSPACE (-5) /* workspace missing or too small */
#define MI_MOE_EUNSUPPORTED (-6)
#define MI_MOE_ETOOLARGE (-7)  /* input needs more scratch than a non-allocating entry point holds */

typedef void* mi_moe_stream_t; /* hipStream_t */

int mi_moe_abi_version(void);

/* Human-readable text for a return code of any function below (static storage). */
const char* mi_moe_strerror(int rc);

/*
 * Router top-k + softmax over the selected logits.
 * Replaces: MoE._get_topk + F.softmax(...float()).type_as (moe.py:250-255, 338-344).
 *   logits    (T, E) of `dtype`, 1 <= k <= E <= 1024
 *   gates_out (T, k) of `dtype`  -- softmax in fp32 over the k selected values, rounded once
 *   idx_out   (T, k) int32       -- experts in order (value descending, expert index ascending);
 *                                   NaN orders as the largest value
 */
int mi_moe_router_topk_softmax(const void* logits, int T, int E, int k, int dtype,
                               void* gates_out, int32_t* idx_out, mi_moe_stream_t stream);

/*
 * Fused router: logits = x @ gate_w^T rounded to `dtype` (+ optional per-expert fp32 bias, rounded
 * again), then the top-k softmax above, in ONE pass over x.
 * Replaces: MoE._compute_routing_weights (moe.py:246-257).
 *   x (T, H), gate_w (E, H) of `dtype`.  F16 / BF16 with E <= 64, k <= 8, H % 16 == 0 run the streaming
 *   kernels (gate weights resident in LDS, x read once at HBM rate); F32 (H % 8 == 0), 65 .. 256 experts
 *   and k up to 64 run a general kernel (one workgroup per 16 tokens) -- no shape of the layer needs a library
 *   GEMM for its logits.  Anything else: MI_MOE_EUNSUPPORTED.
 *   bias       (E,) fp32 or NULL
 *   logits_out (T, E) of `dtype` or NULL (the training-time aux loss and the backward read it)
 *   ws / ws_bytes  optional scratch, 16-byte aligned.  With at least
 *                  mi_moe_router_fused_workspace_bytes(T, H, E) bytes (non-zero for T <= 1024) the
 *                  contraction is split over many workgroups and finished by a second small launch -- a few
 *                  tokens alone cannot keep more than T/16 compute units busy; with NULL one launch does it all.
 *                  More than 64 experts: non-zero for few tokens too (the general kernel then cuts the
 *                  contraction into ranges over many workgroups and a second launch adds them in order), and
 *                  for T * E >= 2^20: F16 / BF16 without a
 *                  bias then take their logits from the grouped GEMM's tile kernels (one expert that owns every
 *                  row; the logits go to logits_out or, without one, into the workspace) and run the top-k
 *                  kernel on them -- the general kernel re-reads the gate weights for every 16 tokens.
 */
size_t mi_moe_router_fused_workspace_bytes(int T, int H, int E);
int mi_moe_router_fused(const void* x, const void* gate_w, const float* bias, int T, int H, int E, int k,
                        int dtype, void* logits_out, void* gates_out, int32_t* idx_out, void* ws,
                        size_t ws_bytes, mi_moe_stream_t stream);

/*
 * Backward of the router's outputs w.r.t. its logits (the element-wise part of the gradient of
 * MoE._compute_routing_weights, moe.py:246-257, which the reference leaves to autograd):
 *   d_logits_out[t, e] = d_logits_extra[t, e] + (e == idx[t, j] ? p_j * (g_j - sum_i p_i g_i) : 0),
 * p = fp32 softmax of the k picked logits, g = d_gates[t, :]; the picked term is rounded to `dtype` before the sum
 * and the sum once more, as autograd's casts do on the eager branch.  d_gates (T, k) and d_logits_extra (T, E)
 * (the gradient that reaches the logits directly: the auxiliary loss) may each be NULL (= zero).  The two
 * products that complete the gradient -- d x = d_logits @ gate_w and d gate_w = d_logits^T @ x -- are
 * mi_moe_scattered_gemm and mi_moe_grouped_wgrad called with one expert that owns every row.
 *   logits (T, E), d_gates (T, k), d_logits_extra / d_logits_out (T, E) of `dtype` (F32 / F16 / BF16); k <= 64
 */
int mi_moe_router_dlogits(const void* logits, const int32_t* idx, const void* d_gates, const void* d_logits_extra,
                          int T, int E, int k, int dtype, void* d_logits_out, mi_moe_stream_t stream);

/*
 * Fused router followed by the expert sort / bin of mi_moe_sort_bin, with the seam between them removed.
 * Replaces: MoE._compute_routing_weights + the sort / bincount / cumsum of the scatter branch
 * (moe.py:246-257, 263-271).  Same outputs as the two separate calls, bit for bit.  Two forms:
 *   few tokens (T <= 1024 and T * k <= 8192; decode): the launch that finishes the split-K router also sorts (its
 *     last workgroup to finish does) -- two launches instead of three in a chain of short dependent launches;
 *   many tokens, gate weights resident in LDS (E * (2 H + 16) <= 156 KiB): the router's epilogue counts the
 *     selected experts per chunk of consecutive tokens (the sort's first pass, without a launch of its own or a
 *     second read of the expert ids), then the sort's scan and scatter passes run -- three launches instead of four.
 * Taken when mi_moe_router_fused_sort_workspace_bytes(T, H, E, k) is non-zero (F16 / BF16, E <= 64, k <= 8,
 * H % 16 == 0 and one of the two forms; the size depends on the device's compute-unit count, 0 without a device);
 * MI_MOE_EUNSUPPORTED otherwise.  ws: that many bytes, 16-byte aligned.
 */
size_t mi_moe_router_fused_sort_workspace_bytes(int T, int H, int E, int k);
int mi_moe_router_fused_sort(const void* x, const void* gate_w, const float* bias, int T, int H, int E, int k,
                             int dtype, void* logits_out, void* gates_out, int32_t* idx_out, int32_t* sorted_expert,
                             int32_t* sorted_scattered, int32_t* expert_offsets, void* ws, size_t ws_bytes,
                             mi_moe_stream_t stream);

/*
 * RMSNorm + fused router: x_norm = round(h * rsqrt(mean(h^2) + eps) * ln_weight) (computed in fp32, one rounding,
 * as torch.nn.RMSNorm does), written to x_norm_out, then the fused router above on x_norm -- in one kernel.
 * Replaces: ln_2 of the transformer block followed by MoE._compute_routing_weights
 * (mixins/dense/layer.py:58-59, normalization.py:19-34, moe.py:246-257).
 *   h (T, H), ln_weight (H,) of `dtype` or NULL (no scaling), x_norm_out (T, H).
 * The gate weights and ln_weight must fit in LDS: mi_moe_rmsnorm_router_fused_supported() says whether the shape
 * is taken (E * (2H + 16) + 4H <= 156 KiB, E <= 64, k <= 8, H % 16 == 0, F16 / BF16); otherwise
 * MI_MOE_EUNSUPPORTED and the caller runs the two steps separately.
 */
int mi_moe_rmsnorm_router_fused_supported(int H, int E, int k, int dtype);
int mi_moe_rmsnorm_router_fused(const void* h, const void* ln_weight, float eps, const void* gate_w,
                                const float* bias, int T, int H, int E, int k, int dtype, void* x_norm_out,
                                void* logits_out, void* gates_out, int32_t* idx_out, mi_moe_stream_t stream);

/*
 * Histogram of expert ids.
 * Replaces: continuous_count_cute / the bincount custom op (moe.py:27-44).
 *   ids (L,) int32 with values in [0, E); counts_out (E,) uint32.  1 <= E <= 1024.
 */
int mi_moe_count(const int32_t* ids, int L, int E, uint32_t* counts_out, mi_moe_stream_t stream);

/*
 * Expert sort / bin: stable counting sort of the flat (T*k,) expert ids.
 * Replaces: selected_experts.flatten().sort() + compute_bincount(...).cumsum(-1) (moe.py:263-271).
 *   topk_idx          (T*k,) int32, values in [0, E)
 *   sorted_expert     (T*k,) int32  non-decreasing expert ids
 *   sorted_scattered  (T*k,) int32  flat slot id (t*k + j) of each sorted row; stable
 *   expert_offsets    (E,)   int32  INCLUSIVE prefix sum of the per-expert counts
 *   ws / ws_bytes     scratch of at least mi_moe_sort_bin_workspace_bytes(T*k, E) bytes, 16-byte aligned
 */
size_t mi_moe_sort_bin_workspace_bytes(int L, int E);
int mi_moe_sort_bin(const int32_t* topk_idx, int T, int k, int E, int32_t* sorted_expert,
                    int32_t* sorted_scattered, int32_t* expert_offsets, void* ws, size_t ws_bytes,
                    mi_moe_stream_t stream);

/*
 * mi_moe_sort_bin without a workspace argument, for callers that cannot allocate device memory (code under HIP
 * graph capture, tight serving loops, harnesses that forbid hipMalloc).  No counterpart in the reference.
 * Same inputs, outputs and results as mi_moe_sort_bin; the chunk histograms live in a fixed array of
 * MI_MOE_SORT_BIN_STATIC_BYTES that the library keeps in device memory on every GPU it runs on (held until the
 * process ends).  Inputs that need more -- mi_moe_sort_bin_workspace_bytes(T*k, E) > MI_MOE_SORT_BIN_STATIC_BYTES,
 * e.g. more than about 2^18 / E * 2048 slots -- are refused with MI_MOE_ETOOLARGE before anything is launched.
 * Calls no hipMalloc / hipFree; the first call on a device looks the array's address up (hipGetSymbolAddress) and
 * keeps it, which is the only state the library holds (make that first call outside graph capture).  All calls on
 * one GPU share the array: calls that overlap on one GPU (different streams or host threads) race; calls on one
 * stream are ordered and safe.
 */
#define MI_MOE_SORT_BIN_STATIC_BYTES (1u << 20)
int mi_moe_sort_bin_static(const int32_t* topk_idx, int T, int k, int E, int32_t* sorted_expert,
                           int32_t* sorted_scattered, int32_t* expert_offsets, mi_moe_stream_t stream);

/*
 * Grouped ("scatter2scatter") GEMM:  for every sorted row i with expert e_i
 *     out[ orow(i), : ] = in[ irow(i), : ] @ w[e_i]^T
 *   irow(i) = i                              if grouped_in   else sorted_scattered[i] / k
 *   orow(i) = i                              if grouped_out  else sorted_scattered[i]
 * Replaces: scattered_experts(...) without gates (moe.py:91-101).
 *   in  (in_rows, K), w (E, N, K), out (L, N) of `dtype`; L = T*k rows in sorted order;
 *   expert e owns sorted rows [expert_offsets[e-1], expert_offsets[e]).
 * All three types run on the matrix cores (F32 with 32x32x2 instructions, fp32 accumulation throughout) and need
 * 16-byte chunks along K -- K % 8 == 0 for F16 / BF16, K % 4 == 0 for F32 --, N % 4 == 0 (MI_MOE_EUNSUPPORTED
 * otherwise), `in` and `w` 16-byte aligned and `out` aligned to four elements (MI_MOE_EALIGN otherwise); nothing
 * falls back to a slower kernel on its own -- a caller that wants such a problem computed anyway asks for the
 * one-thread-per-output kernel with mi_moe_scattered_gemm_cfg(..., cfg = 3).
 */
int mi_moe_scattered_gemm(const void* in, const void* w, void* out, const int32_t* sorted_scattered,
                          const int32_t* expert_offsets, int L, int K, int N, int E, int k,
                          int grouped_in, int grouped_out, int dtype, mi_moe_stream_t stream);

/*
 * The same product with the expert weights stored (E, K, N), i.e. out[orow(i), :] = in[irow(i), :] @ w_kn[e_i]:
 * the form of both data gradients of the backward of scattered_experts (moe.py:91-101), d_act = dy @ w_proj[e] and
 * dx = d_h @ w_fc[e], with the weights as the module keeps them (no transposed copy).  F16 / BF16, and only the
 * shapes the persistent tile kernel takes (K % 32 == 0, K >= 128, N % 8 == 0, E <= 256, 16-byte aligned
 * pointers); MI_MOE_EUNSUPPORTED otherwise (the caller can transpose and use mi_moe_scattered_gemm).
 */
int mi_moe_scattered_gemm_wt(const void* in, const void* w_kn, void* out, const int32_t* sorted_scattered,
                             const int32_t* expert_offsets, int L, int K, int N, int E, int k, int grouped_in,
                             int grouped_out, int dtype, mi_moe_stream_t stream);

/* Same call with an explicit kernel configuration (tuning / benchmarking / tests): cfg = -1 picks one
 * from the shape; 0 / 1 / 2 = register-staged 256x256 / 128x128 / 32x256 tiles (all three element types);
 * 3 = one thread per output element (any shape); 4 = DMA-staged 128x128 (K % 32 == 0); 7 = persistent
 * DMA-staged 256x256 tiles with 32-wide K slices and the two wave groups of a SIMD alternating between
 * LDS/DMA work and matrix instructions (K % 32 == 0, K >= 128, N % 8 == 0, E <= 256; what -1 picks for
 * large expert loads); 8 / 9 = 7 with the order in which the XCDs take the tiles fixed to "each XCD a contiguous
 * eighth of the tile list" / "consecutive 32-tile blocks of one chip-wide round" (7 picks the second from 8 column
 * tiles on; same results either way); 4 and 7 .. 9 are F16 / BF16 only.  A configuration that does not take the
 * shape or type returns MI_MOE_EUNSUPPORTED. */
int mi_moe_scattered_gemm_cfg(const void* in, const void* w, void* out, const int32_t* sorted_scattered,
                              const int32_t* expert_offsets, int L, int K, int N, int E, int k,
                              int grouped_in, int grouped_out, int dtype, int cfg, mi_moe_stream_t stream);

/*
 * The same three products with a workspace for the persistent tile kernel (cfg 7 / what -1 picks for large expert
 * loads; no counterpart in the reference, whose kernels launch one workgroup per tile).  That kernel gives every
 * CU a list of 256 x 256 tiles; when the tiles do not fill the last round, the CUs without a tile wait for one
 * tile time -- a tenth of the down-projection of a Mixtral-shape layer (4.5 rounds of tiles, each 14336 long).
 * With a workspace the tiles of that round are cut into 2 .. 4 ranges of K, each range writes an fp32 partial
 * tile, and a second small launch adds a tile's parts in a fixed order and applies the epilogue: results are
 * reproducible run to run, and equal to the unsplit kernel's up to the order of the fp32 sums.  Used only where it
 * pays (K >= 5120 and a last round at most half full); otherwise, and with ws == NULL, the call is exactly the one
 * without a workspace.  ws: mi_moe_grouped_gemm_workspace_bytes() bytes (one partial tile per CU of the current
 * device; 0 if there is no device), 16-byte aligned, MI_MOE_EWORKSPACE / MI_MOE_EALIGN otherwise; contents need
 * no initialisation and carry nothing between calls; calls that overlap in time need separate workspaces.
 * mi_moe_grouped_gemm_splits(K, dtype) tells a caller whether a product of contraction length K and that element
 * type can use the workspace at all (1) or would ignore it (0), so that it need not allocate one.
 */
size_t mi_moe_grouped_gemm_workspace_bytes(void);
int mi_moe_grouped_gemm_splits(int K, int dtype);
int mi_moe_scattered_gemm_ws(const void* in, const void* w, void* out, const int32_t* sorted_scattered,
                             const int32_t* expert_offsets, int L, int K, int N, int E, int k, int grouped_in,
                             int grouped_out, int dtype, int cfg, void* ws, size_t ws_bytes, mi_moe_stream_t stream);
int mi_moe_scattered_gemm_wt_ws(const void* in, const void* w_kn, void* out, const int32_t* sorted_scattered,
                                const int32_t* expert_offsets, int L, int K, int N, int E, int k, int grouped_in,
                                int grouped_out, int dtype, void* ws, size_t ws_bytes, mi_moe_stream_t stream);

/*
 * Up-projection with SwiGLU fused into the epilogue:
 *     h = x[sorted_scattered[i] / k] @ w_fc[e_i]^T  (2I wide: rows [0,I) of w_fc are "up", [I,2I) "gate")
 *     act_out[i, :] = h[:I] * silu(h[I:])           (grouped order, `dtype`)
 * Replaces: c_fc scattered_experts(grouped_out=True) + GLUActivation (moe.py:273-281, glu.py:42-43).
 *   x (T, H), w_fc (E, 2I, H), act_out (L, I).
 */
int mi_moe_up_swiglu(const void* x, const void* w_fc, void* act_out, const int32_t* sorted_scattered,
                     const int32_t* expert_offsets, int L, int H, int I, int E, int k, int dtype,
                     mi_moe_stream_t stream);

int mi_moe_up_swiglu_cfg(const void* x, const void* w_fc, void* act_out, const int32_t* sorted_scattered,
                         const int32_t* expert_offsets, int L, int H, int I, int E, int k, int dtype, int cfg,
                         mi_moe_stream_t stream);
/* ... and with the persistent kernel's workspace (see mi_moe_scattered_gemm_ws) */
int mi_moe_up_swiglu_ws(const void* x, const void* w_fc, void* act_out, const int32_t* sorted_scattered,
                        const int32_t* expert_offsets, int L, int H, int I, int E, int k, int dtype, int cfg,
                        void* ws, size_t ws_bytes, mi_moe_stream_t stream);

/*
 * The same up-projection for training: next to act_out it writes the (L, 2I) pre-activation h, which the backward
 * needs (SwiGLU's derivative and the weight gradient), from the same accumulators -- one launch and one pass over h
 * less than mi_moe_scattered_gemm followed by mi_moe_swiglu_forward.  h is rounded to `dtype` and act_out is formed
 * from the ROUNDED halves, as mi_moe_swiglu_forward forms it from the stored h (what GLUActivation does to the
 * output of the grouped GEMM, glu.py:42-43), with this kernel's reciprocal in place of that kernel's division.
 * F16 / BF16 and the shapes and loads for which cfg -1 picks the persistent tile kernel (H % 32 == 0, H >= 128,
 * I % 8 == 0, E <= 256, on average >= 192 rows per expert); MI_MOE_EUNSUPPORTED otherwise, and the caller makes
 * the two calls.  h_out 16-byte aligned.
 */
int mi_moe_up_swiglu_keep(const void* x, const void* w_fc, void* act_out, void* h_out, const int32_t* sorted_scattered,
                          const int32_t* expert_offsets, int L, int H, int I, int E, int k, int dtype,
                          mi_moe_stream_t stream);

/*
 * Gate-weighted combine:  y[t, :] = sum_j gates[t, j] * o[t*k + j, :]   (fp32 accumulation).
 * Replaces: the gates contraction inside scattered_experts(gates=...) (moe.py:282-290).
 *   o (T*k, H), gates (T, k), y (T, H) of `dtype`.
 */
int mi_moe_combine(const void* o, const void* gates, void* y, int T, int k, int H, int dtype,
                   mi_moe_stream_t stream);

/*
 * Combine with the tail of the transformer block folded in:
 *     r = round(sum_j gates[t, j] * o[t*k + j, :])          (the call above)
 *     r = round(r + shared[t, :])        if shared          (shared experts, moe.py:214)
 *     r = round(r * residual_scale)      if has_scale       (m_residual, mixins/dense/layer.py:61-62)
 *     y[t, :] = round(r + residual[t, :]) if residual       (mixins/dense/layer.py:64)
 * Every step is rounded to `dtype` as the separate torch operations round it, so the result equals
 * running them after mi_moe_combine bit for bit; two (T, H) round trips through HBM less.
 *   shared, residual (T, H) of `dtype` or NULL.
 */
int mi_moe_combine_block_tail(const void* o, const void* gates, const void* shared, const void* residual,
                              float residual_scale, int has_scale, void* y, int T, int k, int H, int dtype,
                              mi_moe_stream_t stream);

/*
 * Element-wise pieces of the backward pass (training through the kernel branch).  The reference gets its
 * gradients from the autograd function of the external scattermoe package (moe.py:91-101); these two are
 * the parts of that backward that are neither a grouped GEMM nor a library GEMM.  F32 / F16 / BF16; row lengths
 * are whole 16-byte chunks (a multiple of 8 values of a 16-bit type, of 4 for F32).
 *
 * mi_moe_swiglu_backward, one pass over the sorted rows i = 0..L-1:
 *   h (L, 2I) = [up | gate] pre-activation, d_act (L, I) = gradient w.r.t. a = up * silu(gate)
 *   (activations/glu.py:42-43) BEFORE the router weight is applied, i.e. dy[token(i)] @ w_proj[expert(i)];
 *   g_i = gates[slot(i)] with slot(i) = sorted_scattered[i] (gates NULL: 1; sorted_scattered NULL: slot = i).
 *   d_h (L, 2I) out = [g d_act * silu(gate) | g d_act * up * silu'(gate)]
 *   act_g (L, I) out or NULL = g * a               (operand of the down-projection's weight gradient)
 *   d_gates (T*k) out or NULL: d_gates[slot(i)] = <d_act[i], a[i]>   (= <dy[t], w_proj[e] a>, gradient of the
 *   router weight; every slot is written exactly once).  I % 8 == 0 (F32: I % 4 == 0).
 */
int mi_moe_swiglu_backward(const void* h, const void* d_act, const void* gates, const int32_t* sorted_scattered,
                           void* d_h, void* act_g, void* d_gates, int L, int I, int dtype, mi_moe_stream_t stream);
/* The activation on its own, act_out (L, I) = h[:, :I] * silu(h[:, I:]) for a stored pre-activation h (L, 2I):
 * the GLUActivation the reference applies to the output of the up-projection (moe.py:281, glu.py:42-43).  A
 * training step that keeps h for the backward uses the unfused pair (mi_moe_scattered_gemm, this) in place of
 * mi_moe_up_swiglu.  I % 8 == 0 (F32: I % 4 == 0). */
int mi_moe_swiglu_forward(const void* h, void* act_out, int L, int I, int dtype, mi_moe_stream_t stream);
/* d_gates[t, j] = <dy[t, :], o[t*k + j, :]>: the gradient of mi_moe_combine w.r.t. the gates.  H % 8 == 0 (F32: H % 4 == 0). */
int mi_moe_combine_grad_gates(const void* o, const void* dy, void* d_gates, int T, int k, int H, int dtype,
                              mi_moe_stream_t stream);

/*
 * Per-expert weight gradients (the "X^T dY" of the backward of scattered_experts, moe.py:91-101):
 *     dw[e, m, n] = sum over sorted rows r of expert e of  a[ai(r), m] * b[bi(r), n]
 * with ai(r) = a_idx[r] (or r if a_idx is NULL), same for b.  a (rows_a, M), b (rows_b, N), dw (E, M, N) of
 * `dtype` (F16 / BF16), fp32 accumulation, one rounding.  Deterministic: an expert's rows are summed in a fixed
 * order (partial sums per group of rows in the workspace, then added up in group order); experts without rows
 * get zeros.  M % 8 == 0, N % 8 == 0, E <= 256 and both operands below 4 GiB (a_rows, b_rows: their row counts),
 * else MI_MOE_EUNSUPPORTED.  Index values are not checked.
 * Uses: d c_fc[e] = d_h[rows]^T x[token(rows)] (a = d_h in sorted order, b = x gathered), and
 *       d c_proj[e] = dy[token(rows)]^T act[rows] (a = dy gathered, b = act in sorted order).
 */
size_t mi_moe_grouped_wgrad_workspace_bytes(int L, int E, int M, int N);
int mi_moe_grouped_wgrad(const void* a, const int32_t* a_idx, const void* b, const int32_t* b_idx,
                         const int32_t* expert_offsets, void* dw, void* workspace, size_t workspace_bytes,
                         int L, int a_rows, int b_rows, int M, int N, int E, int dtype, mi_moe_stream_t stream);

/* The same sums for F32 operands on the fp32 matrix instruction (no counterpart of its own in the reference: its
 * scattermoe backward serves every dtype): one workgroup per (expert, 128 x 128 tile of dw) adds the expert's rows
 * in ascending order -- deterministic, no workspace.  M % 4 == 0, N % 4 == 0, 16-byte aligned operands, E <= 65535. */
int mi_moe_grouped_wgrad_f32(const float* a, const int32_t* a_idx, const float* b, const int32_t* b_idx,
                             const int32_t* expert_offsets, float* dw, int L, int M, int N, int E,
                             mi_moe_stream_t stream);

/* The same sums for any shape and for F32 as well (the matrix-core kernel above takes 16-bit operands with
 * M % 8 == N % 8 == 0 only): one thread per element of dw, the expert's rows added in ascending order in fp32, one
 * rounding.  Slow; no workspace.  M <= 262140, E <= 65535. */
int mi_moe_grouped_wgrad_naive(const void* a, const int32_t* a_idx, const void* b, const int32_t* b_idx,
                               const int32_t* expert_offsets, void* dw, int L, int M, int N, int E, int dtype,
                               mi_moe_stream_t stream);

/*
 * Training-mode auxiliary loss of the router, moe.py:346-369 (one data-parallel rank), and its gradient:
 *   loss = E * sum_e normalize1(A)_e * normalize1(f)_e + 0.1 * mean_t(logsumexp(logits[t, :])^2),
 *   A_e = sum_t softmax(logits[t, :])_e,  f_e = occurrences of expert e in topk_idx (T, k).
 * logits (T, E) of `dtype` (F32 / F16 / BF16), fp32 arithmetic, E <= 256.  Deterministic (fixed-order sums).
 *   loss_w (1 + E floats) out: [0] the loss, [1 + e] d loss / d A_e (what the backward needs).
 * mi_moe_aux_loss_backward: d_logits (T, E) of `dtype` = grad[0] * d loss / d logits; `grad` is one float in
 * device memory (the gradient of the scalar loss).
 */
size_t mi_moe_aux_loss_workspace_bytes(int T, int E);
int mi_moe_aux_loss(const void* logits, const int32_t* topk_idx, float* loss_w, void* workspace, size_t workspace_bytes,
                    int T, int E, int k, int dtype, mi_moe_stream_t stream);
int mi_moe_aux_loss_backward(const void* logits, const float* loss_w, const float* grad, void* d_logits, int T, int E,
                             int dtype, mi_moe_stream_t stream);

/*
 * Decode-shape variants with fp8 (OCP e4m3fn) expert weights and one fp32 scale per output channel.
 * No counterpart in the reference (its fp8 support wraps nn.Linear only, lm_engine/fp8.py:63-73);
 * semantics = dequantise (w * scale[:, None]) then the two calls above.
 *   x / act / o are `dtype` (F16 / BF16); *_scale are (E, out) fp32.
 *   w_tiled == 0: w_* are (E, out, in) bytes, row-major.
 *   w_tiled == 1: w_* are in the streamed-tile layout (in % 128 == 0 only), mi_moe_fp8_tiled_bytes() bytes:
 *       [expert][unit u][K stage s][row t = 0..31][slot c = 0..7][16 bytes]
 *     where a unit is 16 output channels of the SwiGLU up-projection (rows t < 16: "up" channel 16u + t,
 *     rows t >= 16: "gate" channel 16u + t - 16) or 32 channels otherwise (channel 32u + t), and slot c of
 *     row t holds bytes [128 s + 16 c', 128 s + 16 c' + 16) of that channel's weight row with
 *     c' = c ^ (((t >> 1) & 1) | (((t >> 2) & 1) << 2)).  Channels past `out` are zero rows.  A wave then streams one contiguous run
 *     (results are bit-identical to the row-major layout; only the HBM access pattern changes).
 */
/* out = output channels (I for the SwiGLU up-projection, whose weight has 2I rows); 0 if the layout does not
 * exist for the shape (in % 128 != 0). */
size_t mi_moe_fp8_tiled_bytes(int E, int out, int in, int glu);
int mi_moe_up_swiglu_fp8(const void* x, const void* w_fc_q, const float* w_fc_scale, void* act_out,
                         const int32_t* sorted_scattered, const int32_t* expert_offsets, int L, int H, int I,
                         int E, int k, int dtype, int w_tiled, mi_moe_stream_t stream);
int mi_moe_down_fp8(const void* act, const void* w_proj_q, const float* w_proj_scale, void* o_out,
                    const int32_t* sorted_scattered, const int32_t* expert_offsets, int L, int I, int H,
                    int E, int dtype, int w_tiled, mi_moe_stream_t stream);
/* The same two calls with the kernel family chosen by the caller: cfg -1 picks by the batch (what the calls above
 * do), 0 the streaming kernels (an expert's weights are read once per 16 of its rows: decode), 1 the tile kernels of
 * the grouped GEMM with the fp8 bytes widened on their way into LDS (an expert's weights are read once per row tile:
 * from a few dozen rows per expert on). */
int mi_moe_up_swiglu_fp8_cfg(const void* x, const void* w_fc_q, const float* w_fc_scale, void* act_out,
                             const int32_t* sorted_scattered, const int32_t* expert_offsets, int L, int H, int I,
                             int E, int k, int dtype, int w_tiled, int cfg, mi_moe_stream_t stream);
int mi_moe_down_fp8_cfg(const void* act, const void* w_proj_q, const float* w_proj_scale, void* o_out,
                        const int32_t* sorted_scattered, const int32_t* expert_offsets, int L, int I, int H,
                        int E, int dtype, int w_tiled, int cfg, mi_moe_stream_t stream);
/* The same weights widened to `dtype` with the channel scale folded in: w_out (E, out, in) -- (E, 2 * out, in), up
 * rows first, with glu -- = round(w * scale[:, None]), from either layout.  For batches with many rows per expert,
 * where the two calls above (which stream an expert's weights once per 16 of its rows) lose to the tiled 16-bit
 * kernels on a widened copy (mi_moe_up_swiglu / mi_moe_scattered_gemm); the caller owns the copy.  in % 16 == 0. */
int mi_moe_fp8_dequant(const void* w_q, const float* w_scale, void* w_out, int E, int out, int in, int glu,
                       int w_tiled, int dtype, mi_moe_stream_t stream);

/*
 * Diagnostics (no counterpart in the reference; nothing in the layer calls them): the pieces of the persistent
 * grouped GEMM's inner loop in isolation, for a benchmark that wants a measured ceiling beside the GEMM's own
 * figure.  One workgroup of eight waves per compute unit runs `slices` K slices of a 256 x 256 bf16 tile the way
 * the GEMM does (32 matrix instructions 16x16x32, twelve 16-byte LDS fragment reads and four 1 KiB DMA
 * instructions per wave and slice, ring of four 32 KiB stages) with parts switched off:
 *   mode 0  matrix instructions only        mode 1  + the LDS fragment reads
 *   mode 2  DMA only (L2 -> LDS fill)       mode 3  everything, in the GEMM's two-group ping-pong schedule
 * Per workgroup and slice: 2 * 256 * 256 * 32 flops, 32 KiB of DMA.  data: at least 2 MiB + 4 KiB of bytes of the
 * caller's choice (random bf16 values draw more power than zeros), 16-byte aligned, read only; sink:
 * mi_moe_probe_sink_bytes() bytes that the kernels write (one float per thread, so that nothing is optimised away).
 */
size_t mi_moe_probe_sink_bytes(void);
int mi_moe_probe_kloop(int mode, const void* data, size_t data_bytes, int slices, void* sink, size_t sink_bytes,
                       mi_moe_stream_t stream);

#ifdef __cplusplus
}
#endif
#endif /* MI_MOE_H */
