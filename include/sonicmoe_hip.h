/* C ABI of libsonicmoe_hip.so and libsonicmoe_hip_f16.so: the gfx950 (MI355X) kernels behind the `sonicmoe::*`
 * operators of the MoE layer.
 *
 * Two libraries, one interface.  Both are built from the same sources and export every entry point declared here with
 * the same arguments.  They differ in the 16-bit ELEMENT TYPE of the tensors that the grouped GEMMs, the gather-sums,
 * the bias / score-gradient kernels, the router weight gradient and the fp8 quantisers read and write: bf16 in
 * libsonicmoe_hip.so, fp16 in libsonicmoe_hip_f16.so - the two types the reference's grouped GEMMs take
 * (sonicmoe/functional/grouped_gemm.py:3033-3044).  "bf16" in the comments below means that element type.  A caller
 * links or dlopen()s the one that matches its tensors.  Both may be loaded into one process with dlopen(): the symbol
 * names are the same, so look the entry points up per handle (dlsym), and each library is linked -Bsymbolic so that it
 * keeps calling its own kernels even next to an RTLD_GLOBAL copy of the other.  Entry points that take an smoe_dtype code (top-k, switch loss, token
 * rounding) behave identically in both; smoe_router_forward_fused exists for bf16 only and returns
 * SMOE_ERR_UNSUPPORTED in the fp16 library.  Tuning knobs and the last-error text are per library.
 *
 * Conventions
 *   - every pointer is a DEVICE pointer owned by the caller; the library never allocates device memory
 *   - `stream` is a hipStream_t passed as void* (NULL = default stream); all work is asynchronous on it
 *   - return value: 0 = SMOE_OK, otherwise an smoe_status; smoe_last_error() gives the message of the last
 *     failing call on the calling thread
 *   - activations / weights are the library's 16-bit element type (raw bits), routing scores fp32, all indices int32
 *   - weights are addressed in the PARAMETER layout of the reference module: W1 (E, 2I, H) and W2 (E, H, I),
 *     innermost dimension contiguous, with explicit expert and row strides in ELEMENTS (the reference hands its
 *     kernels permuted views of exactly these buffers: sonicmoe/moe.py:223-225)
 *   - rows of the grouped tensors z, y1, y2, dz, y1s, dx_expanded are in expert-sorted order: rows
 *     [off[e], off[e+1]) belong to expert e; row m was routed from token x_gather_idx[m] and flat routing
 *     slot s_scatter_idx[m]
 *   - a `workspace` argument is scratch memory of at least the matching *_workspace_bytes(); contents are
 *     undefined before and after the call
 *
 * File:line citations name the reference interface each entry point replaces (paths relative to the
 * reference tree).
 */
#ifndef SONICMOE_HIP_H
#define SONICMOE_HIP_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

typedef enum {
  SMOE_OK = 0,
  SMOE_ERR_INVALID = 1,     /* bad argument (null pointer, negative size, ...) */
  SMOE_ERR_UNSUPPORTED = 2, /* shape / dtype outside what the kernels support */
  SMOE_ERR_HIP = 3,         /* a HIP runtime call or launch failed */
  SMOE_ERR_WORKSPACE = 4    /* workspace too small */
} smoe_status;

typedef enum { SMOE_DT_BF16 = 0, SMOE_DT_F16 = 1, SMOE_DT_F32 = 2 } smoe_dtype;

/* sonicmoe/enums.py:18-26 */
typedef enum {
  SMOE_ACT_SWIGLU = 0,
  SMOE_ACT_GEGLU = 1,
  SMOE_ACT_REGLU = 2,
  SMOE_ACT_RELU_SQ = 3,
  SMOE_ACT_RELU = 4,
  SMOE_ACT_GELU = 5,
  SMOE_ACT_SILU = 6
} smoe_activation;

int smoe_version(void);
const char* smoe_last_error(void);

/* Kernel-selection knobs.  Each is read from the environment once, at the first launch that needs it; this call
 * overrides one afterwards (value < 0 restores the default).  Results do not depend on any of them (the two kernel
 * families "gemm_asm" selects between group the score gradient's partial sums differently: ds agrees to 1e-5); they
 * exist for tuning and so that tests can walk through every kernel.  No counterpart in the reference.
 *   "gemm_asm"             SMOE_GEMM_ASM             1 (default): the bf16 grouped GEMMs run on the hand-scheduled
 *                                                    four-wavefront loop where their shape allows; 0: on the
 *                                                    compiler-scheduled eight-wavefront kernels
 *   "gemm_stream"          SMOE_GEMM_STREAM          1: token-grouped GEMMs run as tile streams (default); 0: one tile
 *                                                    per workgroup
 *   "gemm_stream_grid"     SMOE_GEMM_STREAM_GRID     workgroups of a tile-stream launch; 0 = one per compute unit
 *   "dz_stream"            SMOE_DZ_STREAM            1 (default) the bf16 dz kernel is a tile stream too; 0 one tile per
 *                                                    workgroup for dz alone
 *   "gemm_group_tiles"     SMOE_GEMM_GROUP_TILES     tile order of the token-grouped streams: most token tiles of one
 *                                                    expert that sweep the feature tiles together (default 8, 1..127)
 *   "gemm_group_snake"     SMOE_GEMM_GROUP_SNAKE     1 (default): consecutive groups sweep in opposite directions
 *   "varlen_k_tile_order"  SMOE_VARLEN_K_TILE_ORDER  eight-wavefront weight-gradient kernel: 2 blocked (default),
 *                                                    0 round-robin, 1 whole experts per XCD */
int smoe_set_tuning(const char* name, int value);

/* ---------------------------------------------------------------------------------------------------------
 * Routing
 * ------------------------------------------------------------------------------------------------------ */

/* Expert histogram + INCLUSIVE prefix sum.  Replaces sonicmoe::count_cumsum_cuda
 * (sonicmoe/count_cumsum/__init__.py:11-29, sonicmoe/count_cumsum/kernel.cu:92-205).
 *   x        : n int32 (x_is_int64 = 0) or int64 (= 1) values in [0, E)
 *   count    : E int32 out;  cumsum : E int32 out or NULL (do_cumsum = False)
 * Limits: 1 <= E <= 65536 (the reference needs E % 4 == 0 and E <= 50000: kernel.cu:18, :161-162). */
int smoe_count_cumsum(const void* x, int x_is_int64, int64_t n, int E, int32_t* count, int32_t* cumsum,
                      void* stream);

/* Fused top-K + softmax over router logits.  Replaces sonicmoe::_softmax_topk_fwd / sonicmoe::_topk_fwd
 * (sonicmoe/functional/forward.py:20-50, :224-237; kernel sonicmoe/functional/topk_softmax.py:85-193).
 *   logits (T, E) of `dtype` with row stride `row_stride` elements; scores (T, K) fp32; indices (T, K) int32
 *   winners ordered by descending value, ties towards the lower column; softmax != 0 normalises the K winners
 *   fp32 logits are compared with their low log2(next_pow2(E)) mantissa bits cleared, as the reference does
 *   (topk_softmax.py:127-142).
 * Limits: E <= 4096, K <= min(E, 64). */
int smoe_topk_softmax_fwd(const void* logits, int dtype, int64_t T, int E, int K, int64_t row_stride,
                          float* scores, int32_t* indices, int softmax, void* stream);

/* dlogits[t, idx[t,k]] = s_k (ds_k - sum_j ds_j s_j) (+ dlogits_add[t, idx[t,k]] when dlogits_add is not NULL: the
 * reference's optional `dlogits` argument, a gradient that reached the selected logits some other way; same dtype and
 * row stride as dlogits, may be dlogits itself); other entries are left untouched (caller zero-fills).
 * Replaces sonicmoe::_softmax_topk_bwd (sonicmoe/functional/backward.py:487-556). dlogits has `dtype`. */
int smoe_softmax_topk_bwd(void* dlogits, int dtype, int64_t row_stride, const void* dlogits_add, const float* dscores,
                          const float* scores, const int32_t* indices, int64_t T, int K, void* stream);

/* Backward of the top-K WITHOUT softmax (smoe_topk_softmax_fwd with softmax == 0): dlogits[t, indices[t, k]] =
 * dvalues[t, k]; the caller zero-fills dlogits.  Replaces sonicmoe::_topk_bwd (sonicmoe/functional/backward.py:559-610;
 * no caller inside the reference's layer entry points).  dvalues (T, K) fp32 contiguous, dlogits has `dtype`. */
int smoe_topk_bwd(void* dlogits, int dtype, int64_t row_stride, const float* dvalues, const int32_t* indices, int64_t T,
                  int K, void* stream);

/* Routing metadata by a stable counting sort over expert ids.  Replaces TC_topk_router_metadata and
 * general_routing_router_metadata incl. their count_cumsum / argsort / index kernels
 * (sonicmoe/functional/__init__.py:19-46, :49-82).
 *   expert_idx (TK) int32 in [0, E)
 *   token_idx  (TK) int32 sorted ascending, or NULL for token-choice top-K where slot j belongs to token j / K
 *   outputs: freq (E), off (E+1, leading 0), x_gather_idx / s_scatter_idx / s_reverse_scatter_idx (TK),
 *            tok_off (T+1) per-token slot offsets (may be NULL)
 * Limits: E <= 4096. */
size_t smoe_routing_metadata_workspace_bytes(int64_t TK, int E);
int smoe_routing_metadata(const int32_t* expert_idx, const int32_t* token_idx, int64_t TK, int64_t T, int E, int K,
                          int32_t* freq, int32_t* off, int32_t* x_gather_idx, int32_t* s_scatter_idx,
                          int32_t* s_reverse_scatter_idx, int32_t* tok_off, void* workspace, size_t workspace_bytes,
                          void* stream);

/* smoe_routing_metadata for callers that cannot allocate device memory (code under HIP graph capture, serving loops,
 * harnesses that forbid hipMalloc) and have no workspace to hand in.  No counterpart in the reference.  Same
 * arguments, results and limits as smoe_routing_metadata minus the workspace: the two (E, ceil(TK / 1024)) int32
 * tables of the counting sort live in an array of SMOE_ROUTING_METADATA_STATIC_BYTES that is part of the library
 * image (each GPU the library runs on holds one copy until the process ends).  The call allocates and frees nothing.
 *   - sizes with smoe_routing_metadata_workspace_bytes(TK, E) > SMOE_ROUTING_METADATA_STATIC_BYTES are rejected with
 *     SMOE_ERR_WORKSPACE (e.g. TK = 262144 fits up to E = 2048, E = 128 up to TK = 4194304)
 *   - every call on one GPU uses that GPU's one array: calls that may overlap on a GPU (different streams or
 *     threads) race; order them.  Nothing in the array has to be cleared between calls. */
#define SMOE_ROUTING_METADATA_STATIC_BYTES (4u << 20)
size_t smoe_routing_metadata_static_capacity(void);
int smoe_routing_metadata_static(const int32_t* expert_idx, const int32_t* token_idx, int64_t TK, int64_t T, int E,
                                 int K, int32_t* freq, int32_t* off, int32_t* x_gather_idx, int32_t* s_scatter_idx,
                                 int32_t* s_reverse_scatter_idx, int32_t* tok_off, void* stream);

/* ---------------------------------------------------------------------------------------------------------
 * Grouped GEMMs (bf16 in, fp32 MFMA accumulate, bf16 out)
 * ------------------------------------------------------------------------------------------------------ */

/* Workspace needed by every grouped GEMM below (tile map built from `off` on the device).
 *
 * expert_schedule_order (the reference operators' argument of that name, sonicmoe/functional/forward.py:61, :79-82;
 * its tile scheduler's batch_idx_permute, grouped_gemm.py:819-822, :948): NULL, or E int32 on the device holding a
 * permutation of 0 .. E-1.  The kernels then take up the experts' tiles in that order (position i of the schedule
 * works on expert order[i]) -- e.g. largest expert first, so that the long contractions of the weight-gradient
 * kernels do not start last.  Results do not depend on it bit for bit.  An array that is not a permutation leaves
 * the outputs of the missing experts unwritten; the library does not check it (that would need a host round trip). */
size_t smoe_gemm_workspace_bytes(int64_t TK, int E);

/* z[m] = x[x_gather_idx[m]] W1[e]^T (+ b1[e]);  y1[m] = f(z_even) * z_odd for the gated activations (gate = even
 * columns), f(z) otherwise; f = silu / gelu (erf form) / relu / relu^2 as the activation code says.
 * Replaces sonicmoe::_up_projection_forward (sonicmoe/functional/forward.py:53-129; activation epilogue
 * sonicmoe/functional/grouped_gemm.py:423-439, :1273-1357).
 *   x (T, H); w1 (E, N1, H) with N1 = 2I (gated) or I; b1 (E, N1) contiguous or NULL; z (TK, N1) or NULL
 *   (inference: not stored); y1 (TK, I)
 * Limits: H % 64 == 0, I % 64 == 0. */
int smoe_up_projection_forward(const void* x, const void* w1, int64_t w1_stride_e, int64_t w1_stride_row,
                               const void* b1, void* z, void* y1, const int32_t* off,
                               const int32_t* expert_schedule_order, const int32_t* x_gather_idx, int64_t T,
                               int64_t TK, int H, int I, int E, int activation, void* workspace,
                               size_t workspace_bytes, void* stream);

/* y2[m] = y1[m] W2[e]^T (+ b2[e]).  Replaces sonicmoe::_down_projection_forward
 * (sonicmoe/functional/forward.py:132-178).
 *   y1 (TK, I); w2 (E, H, I); b2 (E, H) contiguous or NULL; y2 (TK, H) */
int smoe_down_projection_forward(const void* y1, const void* w2, int64_t w2_stride_e, int64_t w2_stride_row,
                                 const void* b2, void* y2, const int32_t* off, const int32_t* expert_schedule_order,
                                 int64_t TK, int H, int I, int E, void* workspace, size_t workspace_bytes,
                                 void* stream);

/* The down projection FUSED with the score-weighted combine: o[x_gather_idx[m]] += scores[s_scatter_idx[m]] *
 * (y1[m] W2[e]^T (+ b2[e])), y2 is never stored.  No counterpart in the reference, which stores y2
 * (sonicmoe/functional/forward.py:132-178) and reduces it with a second kernel (forward.py:181-236,
 * reduction_over_k_gather.py:441-517); what it replaces is that pair.
 *   o (T, H) bf16, MUST BE ZERO on entry; scores fp32 flat slots; the other arguments as above and as in
 *   smoe_down_projection_backward
 * A token's rows come from different experts' tiles, so the additions are packed-bf16 atomics: every addition rounds
 * to bf16 and their order is not fixed, i.e. the result is within bf16 accumulation error of the two-kernel path and
 * not bit-reproducible from run to run.  Slower than the two kernels on MI355X (measured); kept as an option. */
int smoe_down_projection_forward_combine(const void* y1, const void* w2, int64_t w2_stride_e, int64_t w2_stride_row,
                                         const void* b2, void* o, const float* scores, const int32_t* off,
                                         const int32_t* expert_schedule_order, const int32_t* x_gather_idx,
                                         const int32_t* s_scatter_idx, int64_t T, int64_t TK, int H, int I, int E,
                                         void* workspace, size_t workspace_bytes, void* stream);

/* out[t] = sum_{j in [tok_off[t], tok_off[t+1])} w[j] * src[ridx[j]]  (w == NULL: unweighted), fp32 accumulate.
 * Replaces sonicmoe::_router_forward and sonicmoe::_token_broadcast_backward
 * (sonicmoe/functional/forward.py:181-202, backward.py:464-484; kernel reduction_over_k_gather.py:441-517).
 *   tok_off == NULL means fixed K slots per token (slot j of token t is t*K + j). */
int smoe_gather_sum(const void* src, void* out, const float* w, const int32_t* ridx, const int32_t* tok_off,
                    int64_t T, int K, int H, void* stream);

/* Backward of down projection + combine.  Replaces sonicmoe::_down_projection_backward
 * (sonicmoe/functional/backward.py:286-461; bias part backward.py:31-107; epilogue math
 * sonicmoe/functional/grouped_gemm.py:1154-1271, :1311-1333, :2536-2561).
 *   dy1 = dout[x_gather_idx] W2[e] (never stored); with s = scores[s_scatter_idx[m]] and y1 = act(z) recomputed:
 *   dz (TK, N1) = s * dy1 * d(act)/dz, y1s = s*y1 (TK, I),
 *   ds[s_scatter_idx[m]] = sum_i dy1*y1 (+ <dout[t_m], b2[e]> when b2 is given) (fp32, flat-slot order),
 *   dw2 (E, H, I) = sum_m dout[t_m]^T (x) y1s[m]  (zeros for empty experts),
 *   db2 (E, H) contiguous = sum_m s * dout[t_m]  (bf16, zeros for empty experts).
 *   ds_partial: fp32 scratch of TK * smoe_dz_partial_cols(I) elements.
 *   dw2 == NULL / db2 == NULL skip those gradients; dz == NULL skips the activation gradient (y1s must then hold
 *   the values a previous call produced). */
int smoe_dz_partial_cols(int I);
int smoe_down_projection_backward(const void* dout, const void* z, const void* w2, int64_t w2_stride_e,
                                  int64_t w2_stride_row, const void* b2, void* dw2, int64_t dw2_stride_e,
                                  int64_t dw2_stride_row, void* db2, void* dz, void* y1s, float* ds,
                                  float* ds_partial, const float* scores, const int32_t* off,
                                  const int32_t* expert_schedule_order, const int32_t* x_gather_idx,
                                  const int32_t* s_scatter_idx, int64_t T, int64_t TK, int H, int I, int E,
                                  int activation, void* workspace, size_t workspace_bytes, void* stream);

/* dW1[e] = sum_m dz[m]^T (x) x[t_m];  db1[e] = sum_m dz[m];  dx_expanded[m] = dz[m] W1[e].
 * Replaces sonicmoe::_up_projection_backward (sonicmoe/functional/backward.py:195-283; db1 backward.py:109-168).
 *   dz (TK, N1) with N1 = 2I for gated activations, I otherwise; db1 (E, N1) contiguous, bf16
 *   dw1 == NULL, db1 == NULL or dx_expanded == NULL skips that output (frozen weights / no input gradient). */
int smoe_up_projection_backward(const void* x, const void* w1, int64_t w1_stride_e, int64_t w1_stride_row,
                                const void* dz, void* dw1, int64_t dw1_stride_e, int64_t dw1_stride_row, void* db1,
                                void* dx_expanded, const int32_t* off, const int32_t* expert_schedule_order,
                                const int32_t* x_gather_idx, int64_t T, int64_t TK, int H, int I, int E,
                                int activation, void* workspace, size_t workspace_bytes, void* stream);

/* Weight gradient of the router's linear layer, dWr = dlogits^T x, split over the tokens: partial[c] (E, H) bf16 is the
 * product over tokens [c * ceil(T / chunks), ...) and the caller sums the `chunks` partials.  The reference leaves this
 * GEMM to torch (router_logits = F.linear(x, router_w), sonicmoe/functional/__init__.py:438); with E rows of output and
 * T = tens of thousands of contraction elements a library GEMM without a split fills an eighth of the chip.
 * dlogits (T, E) and x (T, H) contiguous bf16; E and H multiples of 8. */
int smoe_router_weight_grad(const void* dlogits, const void* x, void* partial, int64_t T, int E, int H, int chunks,
                            void* stream);

/* The router in one pass over x (bf16): logits = x Wr^T, the top-K winners of every row with their softmax scores, and
 * optionally the column sums of the full row softmax, all from the GEMM's accumulators.  Replaces the chain
 * router_logits = F.linear(x, router_w) -> sonicmoe::_softmax_topk_fwd (sonicmoe/functional/__init__.py:438-439,
 * forward.py:224-237) and feeds the load-balancing loss (sonicmoe/moe.py:247-274) without another pass over the logits.
 *   x (T, H), wr (E, H), logits (T, E) bf16 contiguous; scores (T, K) fp32; indices (T, K) int32
 *   colsum_partial: NULL, or smoe_router_fused_partials(T, E) x E floats: per-workgroup column sums of
 *   softmax(logits) in fp32, to be handed to smoe_switch_loss_from_partials.
 * Top-K and both softmaxes are evaluated on the logits as stored (rounded to bf16): scores and indices equal
 * smoe_topk_softmax_fwd applied to the stored logits bit for bit.  The logits themselves differ from a library GEMM's
 * in the last bf16 bit (different summation order), so near-ties may route differently than after F.linear.
 * Limits: E % 16 == 0, 16 <= E <= 256; H % 256 == 0; 1 <= K <= E. */
int64_t smoe_router_fused_partials(int64_t T, int E);
int smoe_router_forward_fused(const void* x, const void* wr, int64_t T, int H, int E, int K, void* logits,
                              float* scores, int32_t* indices, float* colsum_partial, void* stream);
/* acc, aux of smoe_switch_loss_fwd from column-sum partials (n_partial, E) some other kernel produced. */
int smoe_switch_loss_from_partials(const float* partial, int64_t n_partial, int E, const int32_t* freq, float* acc,
                                   float* aux, void* stream);

/* Load-balancing auxiliary loss of MoE.forward (sonicmoe/moe.py:247-274: softmax of the (T, E) logits in fp32, column
 * sums, two L1 normalisations, a dot product -- six torch kernels and a (T, E) fp32 tensor there):
 *   acc[e] = sum_t softmax(logits[t, :])[e],   aux[0] = E * <acc / max(|acc|_1, 1e-12), freq / max(|freq|_1, 1e-12)>.
 * logits (T, E) of `dtype` (smoe_dtype), rows `row_stride` elements apart; freq (E) int32; acc (E) and aux (1) fp32
 * out.  workspace: smoe_switch_loss_workspace_bytes(T, E).  1 <= E <= 4096.  Deterministic (no atomics). */
size_t smoe_switch_loss_workspace_bytes(int64_t T, int E);
int smoe_switch_loss_fwd(const void* logits, int dtype, int64_t row_stride, int64_t T, int E, const int32_t* freq,
                         float* acc, float* aux, void* workspace, size_t workspace_bytes, void* stream);
/* Backward of the above (the reference leaves it to autograd through the six torch ops): dlogits (T, E), same dtype as
 * the logits, = grad_aux[0] * d aux / d logits; acc as written by smoe_switch_loss_fwd; grad_aux (1) fp32 on the
 * device.  Every element of the (T, E) block is written. */
int smoe_switch_loss_bwd(const void* logits, int dtype, int64_t row_stride, int64_t T, int E, const int32_t* freq,
                         const float* acc, const float* grad_aux, void* dlogits, int64_t dlogits_row_stride,
                         void* stream);

/* ---------------------------------------------------------------------------------------------------------
 * Token-rounding router (benchmarks/moe-token-rounding.py:139-191 of the reference, there a chain of torch ops
 * with a dense (T, E) argsort).  Chain: smoe_tr_softmax -> smoe_topk_softmax_fwd(probs, softmax = 0) ->
 * smoe_count_cumsum -> smoe_tr_rank -> (targets = rounded counts) -> smoe_tr_select -> smoe_tr_row_counts ->
 * (exclusive scan of the counts) -> smoe_tr_compact.  `dtype` is SMOE_DT_BF16 or SMOE_DT_F16; E <= 4096.
 * ------------------------------------------------------------------------------------------------------ */

/* probs (T, E) = softmax(logits, fp32) rounded to `dtype` (:149) */
int smoe_tr_softmax(const void* logits, int dtype, int64_t T, int E, int64_t row_stride, void* probs, void* stream);

/* Renormalise the K picks of every token by their sum, write them back into probs, and fill
 * rank[t, e] = renormalised value for a pick, probs[t, e] - 1 otherwise (:158-164); top_v / top_i (T, K) are the
 * picks' values (fp32 images of the 16-bit probabilities) and columns. */
int smoe_tr_rank(void* probs, void* rank, int dtype, const float* top_v, const int32_t* top_i, int64_t T, int E,
                 int K, void* stream);

/* keep[t, e] = 1 for the target[e] tokens of expert e with the largest rank[t, e] (ties: lower token first), else 0
 * (:167-184). */
int smoe_tr_select(const void* rank, int dtype, const int32_t* target, uint8_t* keep, int64_t T, int E,
                   void* stream);

/* counts[t] = number of kept experts of token t */
int smoe_tr_row_counts(const uint8_t* keep, int64_t T, int E, int32_t* counts, void* stream);

/* The kept pairs of token t, experts ascending, at positions [tok_off[t], tok_off[t+1]): scores = probs[t, e] in
 * `dtype`, token_idx = t, expert_idx = e (:187-191; the reference leaves the order inside a token unspecified). */
int smoe_tr_compact(const uint8_t* keep, const void* probs, int dtype, const int32_t* tok_off, int64_t T, int E,
                    void* scores, int32_t* token_idx, int32_t* expert_idx, void* stream);

/* ---------------------------------------------------------------------------------------------------------
 * fp8 forward path (OCP e4m3 elements, one power-of-two scale per 32 contraction elements)
 * No counterpart in the reference, which computes in bf16 only; the shapes and epilogues are those of
 * smoe_up_projection_forward / smoe_down_projection_forward above.
 * ------------------------------------------------------------------------------------------------------ */

/* Quantise a bf16 matrix along its rows.
 *   src (R, C) bf16 with row stride `src_stride` elements; C % 128 == 0
 *   q (R, C) bytes: e4m3 of src / scale, round to nearest even, never saturating
 *   scales (C / 128, R) uint32: byte b of word [g][r] is the biased exponent (2^(byte-127)) shared by elements
 *          [128 g + 32 b, 128 g + 32 b + 32) of row r: the smallest power of two with amax / scale <= 448 */
int smoe_mx_quantize(const void* src, int64_t src_stride, int64_t R, int C, void* q, void* scales, void* stream);

/* Workspace of the two fp8 operators whose token operand is gathered (smoe_up_projection_forward_fp8 and
 * smoe_down_projection_backward_fp8, contraction size K = H): the tile map of smoe_gemm_workspace_bytes followed by
 * room for the gathered rows' scale words in grouped order, (K / 128) * TK words, which the operator fills with a
 * small kernel of its own so that the GEMM reads two cache lines of scales per 64 rows instead of 64.  Both operators
 * also accept the smaller smoe_gemm_workspace_bytes(TK, E): the GEMM then fetches every row's scale word through the
 * gather index (same results, a few per cent slower).  No counterpart in the reference. */
size_t smoe_fp8_gemm_workspace_bytes(int64_t TK, int E, int K);

/* As smoe_up_projection_forward with x and W1 given in the quantised form above:
 *   xq (T, H) bytes + x_scales (H/128, T); w1q (E, N1, H) bytes contiguous + w1_scales (H/128, E*N1)
 *   z (TK, N1) bf16 or NULL; y1 (TK, I) bf16 or NULL;
 *   y1q (TK, I) bytes + y1q_scales (I/128, TK) or both NULL: the activation output quantised in the epilogue from
 *   the fp32 values, ready for smoe_down_projection_forward_fp8 (needs I % 128 == 0).
 * Limits: H % 128 == 0, I % 64 == 0; at least one of y1, y1q. */
int smoe_up_projection_forward_fp8(const void* xq, const void* x_scales, const void* w1q, const void* w1_scales,
                                   const void* b1, void* z, void* y1, void* y1q, void* y1q_scales,
                                   const int32_t* off, const int32_t* x_gather_idx, int64_t T, int64_t TK, int H,
                                   int I, int E, int activation, void* workspace, size_t workspace_bytes,
                                   void* stream);

/* As smoe_down_projection_forward with y1 and W2 quantised:
 *   y1q (TK, I) bytes + y1_scales (I/128, TK); w2q (E, H, I) bytes contiguous + w2_scales (I/128, E*H)
 *   y2 (TK, H) bf16.  Limits: I % 128 == 0, H % 64 == 0. */
int smoe_down_projection_forward_fp8(const void* y1q, const void* y1_scales, const void* w2q, const void* w2_scales,
                                     const void* b2, void* y2, const int32_t* off, int64_t TK, int H, int I, int E,
                                     void* workspace, size_t workspace_bytes, void* stream);

/* The same kernel serves dx_expanded = dz W1[e] (the activation-gradient half of sonicmoe::_up_projection_backward,
 * sonicmoe/functional/backward.py:195-283) with fp8 operands: pass dzq (TK, N1) + its scales as y1q, the transposed
 * quantised W1 (E, H, N1) as w2q, and N1 for I. */

/* Quantise the TRANSPOSES of E bf16 matrices along their rows:
 *   src: matrix e is (R, C) at src + e * src_stride_e, row stride src_stride_r elements; R % 128 == 0, C % 64 == 0
 *   q (E, C, R) bytes contiguous: q[e][c][r] = e4m3 of src[e][r][c] / scale, 32 consecutive r sharing a scale
 *   scales (R / 128, E * C) uint32, laid out as smoe_mx_quantize lays out the scales of an (E * C, R) matrix.
 * This is the weight operand of the two activation-gradient GEMMs, which contract over the weights' output index:
 * W2 (E, H, I) -> (E, I, H) for dz, W1 (E, N1, H) -> (E, H, N1) for dx. */
int smoe_mx_quantize_transposed(const void* src, int64_t src_stride_e, int64_t src_stride_r, int E, int R, int C,
                                void* q, void* scales, void* stream);

/* Both quantised copies of E weight matrices from ONE pass over them (no counterpart in the reference, which has no
 * fp8 path): q_rows (E * R, C) / scales_rows (C / 128, E * R) exactly as smoe_mx_quantize(src viewed as (E * R, C))
 * writes them - the forward GEMMs' operand - and q_t / scales_t exactly as smoe_mx_quantize_transposed writes them -
 * the activation-gradient GEMMs' operand.  R % 128 == 0, C % 128 == 0.  A training step that runs forward and backward
 * on fp8 operands calls this once per weight in forward and keeps the transposed copy for its backward pass. */
int smoe_mx_quantize_both(const void* src, int64_t src_stride_e, int64_t src_stride_r, int E, int R, int C,
                          void* q_rows, void* scales_rows, void* q_t, void* scales_t, void* stream);

/* The activation-gradient half of smoe_down_projection_backward with fp8 operands (no counterpart in the reference,
 * whose sonicmoe::_down_projection_backward, sonicmoe/functional/backward.py:286-461, is bf16):
 *   dy1 = doutq[x_gather_idx] w2tq[e]^T with the block scales applied (never stored), then as the bf16 operator:
 *   dz (TK, N1) bf16, y1s (TK, I) bf16, ds (TK) fp32 in flat-slot order; and dz once more quantised from its bf16
 *   values: dzq (TK, N1) bytes + dzq_scales (N1/128, TK), the operand of the fp8 dx GEMM.
 *   doutq (T, H) bytes + dout_scales (H/128, T); w2tq (E, I, H) bytes + w2t_scales (H/128, E*I)
 *   (smoe_mx_quantize_transposed of W2); z (TK, N1) bf16; ds_partial: TK * smoe_dz_partial_cols(I) floats.
 * The weight and bias gradients are left to smoe_down_projection_backward with dz == NULL, which reads y1s.
 * Limits: H % 128 == 0, I % 64 == 0, N1 % 128 == 0; no b2 term in ds (smoe_score_grad_bias_term adds it). */
int smoe_down_projection_backward_fp8(const void* doutq, const void* dout_scales, const void* w2tq,
                                      const void* w2t_scales, const void* z, void* dz, void* dzq, void* dzq_scales,
                                      void* y1s, float* ds, float* ds_partial, const float* scores,
                                      const int32_t* off, const int32_t* x_gather_idx, const int32_t* s_scatter_idx,
                                      int64_t T, int64_t TK, int H, int I, int E, int activation, void* workspace,
                                      size_t workspace_bytes, void* stream);

/* ds[s_scatter_idx[m]] += <dout[x_gather_idx[m]], b2[e(m)]> for the TK grouped rows m (e(m) from off): what the
 * down-projection bias adds to the score gradient, the "dot(dout, b2)" of the reference's db2_and_ds_kernel
 * (sonicmoe/functional/backward.py:36-107, called at :410-436).  smoe_down_projection_backward does this itself when it
 * is given b2; this entry point is for a backward pass whose dz came from smoe_down_projection_backward_fp8.
 * dout (T, H) bf16, b2 (E, H) bf16 contiguous, ds (TK) fp32 already holding the GEMM's part; H % 8 == 0. */
int smoe_score_grad_bias_term(const void* dout, const void* b2, const int32_t* off, const int32_t* x_gather_idx,
                              const int32_t* s_scatter_idx, float* ds, int64_t TK, int H, int E, void* stream);

#ifdef __cplusplus
}
#endif
#endif /* SONICMOE_HIP_H */
