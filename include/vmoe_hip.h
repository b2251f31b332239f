/* vmoe_hip.h -- C ABI of libvmoe_hip.so: the inference-time V-MoE layer on one
 * MI355X (gfx950).
 *
 * The reference (google-research/vmoe) is pure Python on JAX/XLA and has no
 * native interface; each entry point below replaces a group of XLA ops of the
 * reference, cited as file:line relative to the reference checkout.  These are
 * the symbols a jax.ffi custom-call shim or a ctypes binding attaches to.
 *
 * Conventions
 *  - All pointers are DEVICE pointers unless stated; arrays are dense,
 *    row-major, in the shapes given.  The caller owns every buffer, including
 *    workspaces; no entry point allocates, frees or synchronises the host.
 *  - `stream` is a hipStream_t passed as void* (0 = the null stream).
 *  - Return value: 0 on success, a negative VMOE_E_* code for rejected
 *    arguments (nothing was launched), a positive value is a hipError_t.
 *  - dtype: VMOE_F32 (float) or VMOE_BF16 (bfloat16 storage, float32 math).
 *  - Symbols: G groups, S items per group, E experts, K selected experts per
 *    item, C capacity (slots per expert per group), D item width, M hidden
 *    width of the expert MLP, T = G*S.
 *  - A "slot row" is the flat row index e*(G*C) + r(g,c) into the expert
 *    buffer (E, G*C, ...), where r(g,c) is the row order produced by
 *    vmoe/moe.py:488-500 (_dispatch): ((g % Q)*E + g / Q)*C + c with Q = G/E
 *    when G % E == 0, else g*C + c.
 *  - Re-entrant: calls on distinct streams with distinct buffers may overlap.
 */
#ifndef VMOE_HIP_H_
#define VMOE_HIP_H_

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define VMOE_ABI_VERSION 1

typedef void* vmoe_stream_t;

enum { VMOE_F32 = 0, VMOE_BF16 = 1 };
enum { VMOE_GELU_TANH = 0, VMOE_GELU_ERF = 1 };

enum {
  VMOE_OK = 0,
  VMOE_E_NULL = -1,        /* a required pointer is null */
  VMOE_E_SHAPE = -2,       /* a size is < 1, or K > E, or sizes disagree */
  VMOE_E_DTYPE = -3,       /* unknown dtype / enum value */
  VMOE_E_ALIGN = -4,       /* row width not a multiple of 16 bytes, or pointer misaligned */
  VMOE_E_OVERFLOW = -5,    /* an index would not fit in int32 */
  VMOE_E_UNSUPPORTED = -6, /* valid, but outside what the kernels cover (see each call) */
  VMOE_E_WORKSPACE = -7    /* workspace missing or too small */
};

int vmoe_abi_version(void);
const char* vmoe_error_string(int code);

/* ------------------------------------------------------------------ gating
 * Replaces vmoe/nn/routing.py:73-80 (nn.Dense without bias + softmax) fused
 * with the jax.lax.top_k of vmoe/moe.py:567.
 * logits = x @ w (float32 accumulate, rounded to dtype), gates = softmax over E
 * (float32 internals, rounded to dtype), then the K largest gates per item in
 * descending order, equal gates -> lower expert index first.
 * Limits: E <= 128; D % 8 == 0 (bf16) / D % 4 == 0 (f32).
 */
typedef struct {
  const void* x;           /* (G*S, D) dtype */
  const void* w;           /* (D, E) dtype: Router/dense/kernel */
  const float* logit_bias; /* optional (E,) float32 added to the logits; null = reference behaviour */
  void* gates;             /* optional out (G*S, E) dtype */
  float* topk_val;         /* out (G*S, K) float32 (values are exact dtype values) */
  int32_t* topk_idx;       /* out (G*S, K) */
  int32_t num_items;       /* T = G*S */
  int32_t D, E, K;
  int32_t dtype;
  float* logits;           /* optional out (G*S, E) float32: the logits (exact dtype values,
                              bias included), what the noisy branch of the router adds to */
} VmoeGateTopkParams;
int vmoe_gate_topk(const VmoeGateTopkParams* p, vmoe_stream_t stream);

/* Noisy branch of the routers, vmoe/nn/routing.py:92-114 (and :226-232):
 *   logits_noisy = logits + noise_std * noise;  gates_noisy = softmax(logits_noisy)
 * and, per group, the load loss of vmoe/nn/routing.py:159-183: with t the K-th
 * largest noisy logit of an item, p = 1 - Phi((t - logits) / noise_std) averaged
 * over the group's items per expert, loss = (std(p_mean) / mean(p_mean))^2.
 * noise is standard normal (the caller draws it); noise_std is the effective
 * standard deviation, (1 / E) * the router's noise_std.  E <= 128, 1 <= K <= E. */
typedef struct {
  const float* logits;     /* (G*S, E) float32 */
  const float* noise;      /* (G*S, E) float32, standard normal */
  float* gates_noisy;      /* out (G*S, E) float32 */
  float* load_loss;        /* optional out (G,) float32 */
  int32_t G, S, E, K;
  float noise_std;
} VmoeNoisyGatesParams;
int vmoe_noisy_gates(const VmoeNoisyGatesParams* p, vmoe_stream_t stream);

/* Top-k alone on given gates (G*S, E) float32: the jax.lax.top_k of
 * vmoe/moe.py:567.  Bit-exact selection; E <= 1024. */
typedef struct {
  const float* gates;
  float* topk_val;   /* (num_items, K) */
  int32_t* topk_idx; /* (num_items, K) */
  int32_t num_items, E, K;
} VmoeTopkParams;
int vmoe_topk(const VmoeTopkParams* p, vmoe_stream_t stream);

/* ------------------------------------------------------------------ metrics
 * Replaces vmoe/nn/routing.py:81-91,133-157,247-252: per group,
 * importance_loss = (std/mean)^2 of sum_s gates[s,:] (population std),
 * gshard_loss = mean_e(mean_s onehot(top1) * mean_s gates) * E^2,
 * auxiliary_loss = sum of weight*loss over weights > 0.  E <= 1024.
 */
typedef struct {
  const void* gates;        /* (G, S, E) dtype */
  const int32_t* top1_idx;  /* first-choice expert of item i at top1_idx[i*top1_stride] */
  float* importance_loss;   /* out (G,) */
  float* gshard_loss;       /* out (G,) */
  float* auxiliary_loss;    /* out (G,) */
  float gshard_loss_weight, importance_loss_weight;
  int32_t G, S, E, top1_stride;
  int32_t dtype;
} VmoeRouterMetricsParams;
int vmoe_router_metrics(const VmoeRouterMetricsParams* p, vmoe_stream_t stream);

/* ------------------------------------------------------------------ slot assignment
 * Replaces vmoe/moe.py:568-589 + :646-648 (_get_top_experts_per_item_common and
 * the indices dispatcher builder), for all groups at once (the jax.vmap of
 * vmoe/nn/routing.py:123-128).  Integer work, bit-exact:
 * position(s,k) = number of (s',k') of the same group with the same expert and
 * (k' < k, or k' == k and s' before s in priority order); priority order is
 * the item index, or with batch_priority the stable descending order of
 * topk_val[:,0].  Positions are not clipped; an assignment is kept iff
 * position < C.  Experts outside [0,E) get position -1.
 * Limits: 8*max(pow2ceil(S), 1024 + ceil(S/2)) (with batch_priority) + 8*E*ceil(S*K/32) +
 * 4*S + 4*E bytes of LDS <= 160 KiB.
 */
typedef struct {
  const float* topk_val;   /* (G, S, K); only [:, :, 0] is read, and only with batch_priority */
  const int32_t* topk_idx; /* (G, S, K) */
  int32_t* indices;        /* out (G, S, K, 2): (expert, position) */
  int32_t* token_slot;     /* out (G, S, K): slot row of the assignment, -1 if dropped */
  int32_t* slot_token;     /* out (E*G*C,): flat item index g*S+s feeding the slot row, -1 if empty */
  int32_t* fill;           /* optional out (G, E): min(C, demand) */
  int32_t G, S, E, K, C;
  int32_t batch_priority;
} VmoeRouteAssignParams;
int vmoe_route_assign(const VmoeRouteAssignParams* p, vmoe_stream_t stream);

/* vmoe_route_assign and vmoe_router_metrics in one launch (the losses run as extra
 * workgroups beside the slot assignment; both read the same top-k output and neither
 * reads what the other writes).  Same results as the two calls; m->G, m->S, m->E must
 * equal p's.  The deterministic branch of NoisyTopExpertsPerItemRouter
 * (vmoe/nn/routing.py:76-91 followed by :116-131) is this call after vmoe_gate_topk. */
int vmoe_route_assign_metrics(const VmoeRouteAssignParams* p, const VmoeRouterMetricsParams* m,
                              vmoe_stream_t stream);

/* Experts-choice ("top items per expert") routing, replacing
 * _get_top_items_per_expert_einsum_dispatcher (vmoe/moe.py:655-694): each expert
 * keeps the C items with its largest gates (jax.lax.top_k of the transposed
 * gates: descending, equal gates -> lower item index first).  The result has the
 * shape of vmoe_route_assign's with one choice per expert (K = E):
 * indices[g,s,e] = (e, rank of item s in expert e's order), kept iff rank < C;
 * weights[g,s,e] = gates[g,s,e] as float32.  The dense (G,S,E,C) one-hot
 * dispatch_weights / combine_weights of the reference follow with vmoe_densify.
 * sel_minmax (optional): per (g, e) the smallest and largest selected gate.
 * Limit: 8*pow2ceil(S) bytes of LDS <= 160 KiB. */
typedef struct {
  const void* gates;      /* (G, S, E), dtype */
  int32_t* indices;       /* out (G, S, E, 2) */
  int32_t* token_slot;    /* out (G, S, E): slot row, -1 if not selected */
  int32_t* slot_token;    /* out (E*G*C,): g*S+s, -1 for slots beyond S */
  float* weights;         /* out (G, S, E) */
  float* sel_minmax;      /* optional out (G, E, 2) */
  int32_t G, S, E, C;
  int32_t dtype;
} VmoeTopItemsParams;
int vmoe_top_items_per_expert(const VmoeTopItemsParams* p, vmoe_stream_t stream);

/* Builds the two slot maps from hand-made (expert, position) indices, as
 * vmoe/moe.py:190-197 and :202-206 interpret them: entries with expert >= E or
 * position >= C are dropped.  Negative entries are counted in
 * *num_invalid; slots targeted by more than one item are counted in
 * *num_duplicates (the reference would accumulate them; these kernels do not,
 * callers must treat a non-zero count as an error).  Both counters are device
 * int32 and must be zeroed by the caller. */
typedef struct {
  const int32_t* indices; /* (G, S, K, 2) */
  int32_t* token_slot;    /* out (G, S, K) */
  int32_t* slot_token;    /* out (E*G*C,) */
  int32_t* num_duplicates;
  int32_t* num_invalid;
  int32_t G, S, E, K, C;
} VmoeIndicesToSlotsParams;
int vmoe_indices_to_slots(const VmoeIndicesToSlotsParams* p, vmoe_stream_t stream);

/* Packed ("ragged") expert buffers.  The reference's buffer gives every (group, expert)
 * pair C rows whether or not items fill them (vmoe/moe.py:190-197); the expert MLP then
 * also runs over the empty rows.  This call renumbers the kept assignments so that
 * expert e's items occupy rows 0 .. rows_per_expert[e]-1 of its (G*C)-row block, groups
 * in order: token_row = e*G*C + sum_{g' < g} fill[g'][e] + position.  dispatch (with
 * slot_token null), the expert MLP (rows_per_expert) and combine take token_row in
 * place of token_slot; the layer's output is unchanged. */
typedef struct {
  const int32_t* fill;        /* (G, E) from vmoe_route_assign */
  const int32_t* token_slot;  /* (G, S, K) from vmoe_route_assign */
  int32_t* token_row;         /* out (G, S, K), -1 for dropped assignments */
  int32_t* rows_per_expert;   /* out (E,) */
  int32_t* prefix;            /* scratch (G, E): rows of expert e taken by the groups before g */
  int32_t* row_token;         /* optional out (E*G*C,): item (g*S + s) held by each packed row;
                                 rows past rows_per_expert[e] are not written */
  int32_t G, S, E, K, C;
} VmoeCompactRowsParams;
int vmoe_compact_rows(const VmoeCompactRowsParams* p, vmoe_stream_t stream);

/* vmoe_compact_rows without a scratch argument (no counterpart in the reference).  For
 * callers that cannot allocate device memory: code under HIP graph capture, tight serving
 * loops, harnesses that forbid hipMalloc.  `prefix` is ignored; the (G, E) scratch is a
 * static device array inside the library, VMOE_COMPACT_ROWS_STATIC_MAX_GE int32 per
 * device (256 KiB, held until the process ends).  G * E beyond that returns
 * VMOE_E_WORKSPACE.  The call allocates and frees nothing.  All calls on one device share
 * the array: calls that overlap on one device (two streams, two host threads) race; calls
 * on one stream, or otherwise ordered, do not.  Results equal vmoe_compact_rows'.
 * The first call on a device looks up the array's device address (hipGetSymbolAddress, once
 * per device, under a mutex): make one call on each device before the first capture; after
 * that a call only launches kernels (no memset node) and may be captured into a HIP graph. */
#define VMOE_COMPACT_ROWS_STATIC_MAX_GE 65536
int vmoe_compact_rows_static(const VmoeCompactRowsParams* p, vmoe_stream_t stream);

/* ------------------------------------------------------------------ dispatch / combine
 * dispatch replaces ExpertIndicesDispatcher.dispatch (vmoe/moe.py:190-197:
 * repeat + scatter_nd into zeros + _dispatch layout): out[slot] = x[item] for
 * kept assignments, 0 for empty slots.  Exact copy.
 * combine replaces ExpertIndicesDispatcher.combine (vmoe/moe.py:199-209):
 * out[item] = sum_k weights[item,k] * (slot >= 0 ? y[slot] : 0), products and
 * sums in float32 in k order, rounded once to dtype.
 * Row width D*sizeof(dtype) must be a multiple of 16 bytes.
 * With slot_token null, dispatch leaves unclaimed slot rows untouched instead of
 * zeroing them (for the packed layout of vmoe_compact_rows, where no one reads them).
 */
typedef struct {
  const void* x;             /* (num_items, D) dtype */
  const int32_t* token_slot; /* (num_items, K) */
  const int32_t* slot_token; /* (num_slots,) or null */
  void* out;                 /* (num_slots, D) dtype */
  int32_t num_items, num_slots, K, D;
  int32_t dtype;
} VmoeDispatchParams;
int vmoe_dispatch(const VmoeDispatchParams* p, vmoe_stream_t stream);

typedef struct {
  const void* y;             /* (num_slots, D) dtype */
  const int32_t* token_slot; /* (num_items, K) */
  const float* weights;      /* (num_items, K) float32 */
  void* out;                 /* (num_items, D) dtype */
  int32_t num_items, num_slots, K, D;
  int32_t dtype;
} VmoeCombineParams;
int vmoe_combine(const VmoeCombineParams* p, vmoe_stream_t stream);

/* Gradients of dispatch / combine (the gather <-> scatter duals; the reference gets them
 * from JAX's autodiff of vmoe/moe.py:190-209).  With combine  out[t] = sum_k w[t,k] *
 * y[slot(t,k)]:
 *   vmoe_combine_backward_data:     dy[slot(t,k)] = w[t,k] * dout[t]; slots no item claims
 *                                   get 0 (slot_token given) or stay untouched (null);
 *   vmoe_combine_backward_weights:  dweights[t,k] = <dout[t], y[slot(t,k)]>, 0 if dropped.
 * The gradient of dispatch with respect to its input, dx[t] = sum_k dbuf[slot(t,k)], is
 * vmoe_combine with unit weights.  Row width as for dispatch / combine. */
typedef struct {
  const void* dout;           /* (num_items, D) dtype: gradient of combine's output */
  const void* y;              /* (num_slots, D) dtype: combine's input (weights gradient only) */
  const int32_t* token_slot;  /* (num_items, K) */
  const float* weights;       /* (num_items, K) float32 (data gradient only) */
  const int32_t* slot_token;  /* (num_slots,) or null (data gradient only) */
  void* dy;                   /* out (num_slots, D) dtype */
  float* dweights;            /* out (num_items, K) float32 */
  int32_t num_items, num_slots, K, D;
  int32_t dtype;
} VmoeCombineBackwardParams;
int vmoe_combine_backward_data(const VmoeCombineBackwardParams* p, vmoe_stream_t stream);
int vmoe_combine_backward_weights(const VmoeCombineBackwardParams* p, vmoe_stream_t stream);

/* Dense (G,S,E,C) view of a sparse assignment, for callers that read
 * EinsumDispatcher.combine_weights / dispatch_weights (vmoe/moe.py:609-619):
 * combine[g,s,e,c] = weight of the kept assignment (s -> e,c), else 0;
 * dispatch[g,s,e,c] = 1 where an assignment is kept.  Outputs must be zeroed by
 * the caller; either may be null. */
typedef struct {
  const int32_t* indices; /* (G, S, K, 2) */
  const float* weights;   /* (G, S, K) */
  float* combine;         /* out (G, S, E, C) float32 */
  uint8_t* dispatch;      /* out (G, S, E, C) bool */
  int32_t G, S, E, K, C;
} VmoeDensifyParams;
int vmoe_densify(const VmoeDensifyParams* p, vmoe_stream_t stream);

/* ------------------------------------------------------------------ expert MLP
 * Replaces the expert vmap of vmoe/moe.py:434-439 over
 * vit_jax.models_vit.MlpBlock (called from vmoe/nn/vit_moe.py:38-45), dropout
 * off: for every expert e, y = gelu(x @ w0[e] + b0[e]) @ w1[e] + b1[e], all rows.
 * bf16: bf16 operands, float32 accumulate, results rounded to bf16 after each
 * matmul, after each bias add and after the GELU.
 * bf16 needs the kernels in K-contiguous order: pass w0t (E,M,D) / w1t (E,D,M)
 * made once by vmoe_pack_expert_weights; if they are null the call packs
 * w0/w1 into `workspace` first (extra HBM pass).  D % 8 == 0 and M % 8 == 0.
 * `workspace` holds the hidden activations (E, R, M), the call's status words, the launch
 * plans of a call with rows_per_expert and, for bf16, 64 MB through which the second
 * product's workgroups exchange float32 partial sums when the tiles of a last, partial round
 * are cut along k (results are deterministic; such a cut reorders one float32 addition per
 * output, so outputs of a call with rows_per_expert may differ from those of a call without
 * by one bfloat16 rounding step).  Calls that share a workspace must not overlap.
 * That exchange assumes that all 256 workgroups of the second product are resident at the
 * same time, which holds when the launch has the GPU to itself: a piece waits for pieces
 * in workgroups placed before its own.  Kernels of other streams that hold compute units
 * at that moment void the assumption.  The wait is bounded (about two seconds); a piece
 * that gives up writes NaN instead of sums it did not get, so the affected output rows are
 * NaN, and it is counted in the status words (vmoe_expert_mlp_status).
 */
typedef struct {
  const void* x;    /* (E, R, D) dtype */
  const void* w0;   /* (E, D, M) dtype: Mlp/Dense_0/kernel (may be null when w0t is given) */
  const void* b0;   /* (E, M) dtype or null */
  const void* w1;   /* (E, M, D) dtype: Mlp/Dense_1/kernel (may be null when w1t is given) */
  const void* b1;   /* (E, D) dtype or null */
  const void* w0t;  /* optional (E, M, D) dtype: w0 transposed per expert */
  const void* w1t;  /* optional (E, D, M) dtype: w1 transposed per expert */
  void* out;        /* (E, R, D) dtype */
  void* workspace;  /* vmoe_expert_mlp_workspace_bytes() bytes */
  size_t workspace_bytes;
  int32_t E, R, D, M;
  int32_t dtype;
  int32_t gelu;     /* VMOE_GELU_TANH (flax default) or VMOE_GELU_ERF */
  const int32_t* rows_per_expert; /* optional (E,): only the first rows_per_expert[e] rows of
                                     expert e hold data; the other rows of x are not read
                                     for results and their rows of out are left untouched */
  const int32_t* x_rows;          /* optional (E, R), needs rows_per_expert: x is then the
                                     (num_items, D) matrix of items itself and x_rows[e][r] the
                                     item in row r of expert e (row_token of vmoe_compact_rows):
                                     the first product gathers its rows, no dispatched buffer
                                     is needed.  D % 32 == 0 (both types), float32 also
                                     16-byte aligned x and w0 and items within 2 GiB
                                     (VMOE_E_UNSUPPORTED otherwise) */
  int32_t num_items;              /* rows of x when x_rows is given */
} VmoeExpertMlpParams;
size_t vmoe_expert_mlp_workspace_bytes(const VmoeExpertMlpParams* p);
int vmoe_expert_mlp(const VmoeExpertMlpParams* p, vmoe_stream_t stream);

/* vmoe_compact_rows and the planning launch of vmoe_expert_mlp in one launch (no counterpart
 * in the reference: the packed rows have none).  `mlp` is the parameter block of the MLP call
 * that follows, with its workspace and with rows_per_expert = c->rows_per_expert, x_rows =
 * c->row_token where the first product gathers its rows (only E, R, D, M, dtype, the
 * workspace and rows_per_expert are looked at here); that call is then made as
 * vmoe_expert_mlp_planned, which takes the launch plans in the workspace as written.
 * VMOE_E_UNSUPPORTED where the compaction needs its two-launch form (E > 256, fewer than 256
 * assignments per group, many groups of few experts) or the MLP plans nothing (float32):
 * make the separate calls.  Results equal those of the separate calls.
 * vmoe_expert_mlp_planned may be called any number of times after one
 * vmoe_compact_rows_planned, as long as the parameter block names the same shapes and
 * workspace and nothing else wrote the workspace in between (each call resets the exchange
 * counters it uses).  The plans carry a tag of the shapes they were written for; a call that
 * does not find its own tag (workspace never planned, or planned for other E, R, D, M)
 * launches kernels that do nothing, leaves `out` untouched and counts a plan mismatch in the
 * status words. */
int vmoe_compact_rows_planned(const VmoeCompactRowsParams* c, const VmoeExpertMlpParams* mlp,
                              vmoe_stream_t stream);
int vmoe_expert_mlp_planned(const VmoeExpertMlpParams* p, vmoe_stream_t stream);

/* Status words of the expert MLP calls made on p->workspace (no counterpart in the
 * reference).  *status receives the DEVICE address of VMOE_MLP_STATUS_WORDS int32 inside the
 * workspace, or null for float32 (those kernels keep no such state); nothing is launched.
 *   status[VMOE_MLP_STATUS_ABANDONED_WAITS]  pieces of the second product's shared round that
 *       gave up waiting for another piece's partial sums (their output rows are NaN);
 *   status[VMOE_MLP_STATUS_PLAN_MISMATCHES]  launches that did not find a plan written for
 *       their shapes and therefore did nothing.
 * Both only grow: the first call on a workspace sets them to zero (it recognises a fresh
 * workspace by a tag word beside them), later calls add.  Read them (hipMemcpy) once the
 * stream has finished; anything but zero means that an output of some call since then is
 * not the product it should be. */
enum { VMOE_MLP_STATUS_ABANDONED_WAITS = 0, VMOE_MLP_STATUS_PLAN_MISMATCHES = 1,
       VMOE_MLP_STATUS_WORDS = 2 };
int vmoe_expert_mlp_status(const VmoeExpertMlpParams* p, const int32_t** status);

/* (batch, rows, cols) -> (batch, cols, rows), 2- or 4-byte elements. */
typedef struct {
  const void* in;
  void* out;
  int32_t batch, rows, cols;
  int32_t dtype;
} VmoeTransposeParams;
int vmoe_pack_expert_weights(const VmoeTransposeParams* p, vmoe_stream_t stream);

/* ------------------------------------------------------------------ Soft MoE
 * soft_route replaces vmoe/projects/soft_moe/router.py:57-96 (no noise):
 * unit-normalise items and slot parameters (eps 1e-6 inside the rsqrt), scale
 * the smaller operand, logits[g,m,n] = x_hat . mu_hat, dispatch = softmax over
 * items m, combine = softmax over slots n.  N = num_experts*num_slots <= 1024,
 * the (S x N) logits of a group must fit the 160 KiB LDS as float32.
 */
typedef struct {
  const void* x;      /* (G, S, D) dtype */
  const void* mu;     /* (D, N) dtype: Router/mu reshaped (D, n*p) */
  float scale;        /* Router/scale */
  void* dispatch_w;   /* out (G, S, N) dtype */
  void* combine_w;    /* out (G, S, N) dtype */
  void* logits;       /* optional out (G, S, N) dtype */
  void* workspace;    /* vmoe_soft_route_workspace_bytes() bytes for the unit-norm, scaled mu (the
                         order is the kernel's own: for bfloat16 the order of its MFMA fragments) */
  size_t workspace_bytes;
  int32_t G, S, D, N;
  int32_t dtype;
  int32_t workspace_prepared; /* 1: `workspace` still holds what an earlier call with the same mu,
                                 scale, dtype and (G, S, D, N) left there; the slot parameters are
                                 not normalised again (they are constants at inference) */
} VmoeSoftRouteParams;
size_t vmoe_soft_route_workspace_bytes(const VmoeSoftRouteParams* p);
int vmoe_soft_route(const VmoeSoftRouteParams* p, vmoe_stream_t stream);

/* Monitoring scalars of SoftRouter.get_metrics (vmoe/projects/soft_moe/router.py:119-125):
 * partial[g] = (sum_s min_n combine_w, sum_s max_n combine_w, sum_n min_s dispatch_w,
 * sum_n max_s dispatch_w) for group g; a second launch adds them over g in index
 * order (bit-reproducible) and writes
 *   stats = (combine_weights_min_mean, combine_weights_max_mean,
 *            dispatch_weights_min_mean, dispatch_weights_max_mean, auxiliary_loss = 0). */
typedef struct {
  const void* combine_w;   /* (G, S, N) dtype */
  const void* dispatch_w;  /* (G, S, N) dtype */
  float* partial;          /* scratch (G, 4) float32 */
  float* stats;            /* out (5,) float32 */
  int32_t G, S, N;
  int32_t dtype;
} VmoeSoftStatsParams;
int vmoe_soft_router_stats(const VmoeSoftStatsParams* p, vmoe_stream_t stream);
/* vmoe_soft_route and vmoe_soft_router_stats on its outputs in one call (SoftRouter.__call__
 * with its get_metrics, vmoe/projects/soft_moe/router.py:57-125).  `stats` names the same
 * combine_w / dispatch_w, G, S, N and dtype as `route`.  Where the routing kernel can, it
 * leaves the (G, 4) partial sums itself (bfloat16, up to 256 items per group, the widths of
 * its two-role kernel) and only the launch that adds them up follows; otherwise the two
 * calls are made one after the other.  The scalars equal those of the separate calls up to
 * the order in which float32 sums are taken. */
int vmoe_soft_route_stats(const VmoeSoftRouteParams* route, const VmoeSoftStatsParams* stats,
                          vmoe_stream_t stream);

/* EinsumDispatcher.dispatch / .combine with dense weights
 * (vmoe/moe.py:148-161): per group,
 *   dispatch: out[slot(g,n)] = sum_s w[g,s,n] * x[g,s,:]
 *   combine:  out[g,s,:]     = sum_n w[g,s,n] * y[slot(g,n)]
 * with N = E*C and slot(g, n=e*C+c) the slot row defined at the top.
 * float32 accumulate, result rounded to out_dtype.  `w` is float32, bf16 or
 * bool (dispatch only; w_dtype = 2).
 */
enum { VMOE_W_F32 = 0, VMOE_W_BF16 = 1, VMOE_W_BOOL = 2 };
typedef struct {
  const void* w;     /* (G, S, E*C) */
  const void* data;  /* dispatch: (G, S, D); combine: (E*G*C, D) */
  void* out;         /* dispatch: (E*G*C, D); combine: (G, S, D) */
  int32_t G, S, E, C, D;
  int32_t w_dtype, data_dtype, out_dtype;
} VmoeEinsumParams;
int vmoe_einsum_dispatch(const VmoeEinsumParams* p, vmoe_stream_t stream);
int vmoe_einsum_combine(const VmoeEinsumParams* p, vmoe_stream_t stream);

/* Elementwise float32 <-> bfloat16 conversion (round to nearest even):
 * the _cast_to_bfloat16 / astype pair of Bfloat16Dispatcher, vmoe/moe.py:212-227. */
typedef struct {
  const void* in;
  void* out;
  size_t n;
  int32_t in_dtype, out_dtype;
} VmoeCastParams;
int vmoe_cast(const VmoeCastParams* p, vmoe_stream_t stream);

/* Residual add fused with the layer norm that follows it, the pattern of every
 * encoder block (vmoe/nn/vit_moe.py:162-179: `x = x + inputs; y = nn.LayerNorm(dtype)(x)`)
 * with flax.linen.LayerNorm's arithmetic (float32 statistics, var = E[x^2] - E[x]^2):
 *   x = residual (+ branch);  residual_out = x;
 *   norm_out = (x - mean) * rsqrt(var + eps) * scale + bias   in out_dtype.
 * residual (rows, D) float32; branch (rows, D) of branch_dtype or null (no add);
 * scale, bias (D,) float32 or null; residual_out float32 or null (may be the
 * residual itself); norm_out or null (add only).  One of the outputs is required. */
typedef struct {
  const float* residual;
  const void* branch;
  const float* scale;
  const float* bias;
  float* residual_out;
  void* norm_out;
  size_t rows;
  int32_t D;
  float eps;
  int32_t branch_dtype, out_dtype;
} VmoeAddLayerNormParams;
int vmoe_add_layer_norm(const VmoeAddLayerNormParams* p, vmoe_stream_t stream);

/* Multi-head softmax attention without mask or dropout, softmax(q k^T * scale) v per
 * (image, head): flax.linen.dot_product_attention as MultiHeadDotProductAttention
 * calls it for vmoe/nn/vit_moe.py:166-174 (float32 logits and statistics; the
 * probabilities enter the second product as bfloat16).
 * q (B, Sq, H, head_dim), k, v (B, Sk, H, head_dim) given by a base pointer and
 * element strides per image and per token (heads are contiguous: head h starts at
 * element h * head_dim), so the packed output of a fused q/k/v projection can be
 * passed without copies; out (B, Sq, H * head_dim) contiguous.  Strides are
 * multiples of 8 elements, pointers 16-byte aligned.
 * VMOE_E_UNSUPPORTED unless dtype is bfloat16, head_dim is 64, scale > 0 and the keys and
 * values of one head fit in LDS (Sk up to about 560). */
typedef struct {
  const void* q;
  const void* k;
  const void* v;
  void* out;
  int64_t q_stride_b, q_stride_s, k_stride_b, k_stride_s, v_stride_b, v_stride_s;
  int32_t B, H, Sq, Sk, head_dim;
  float scale;
  int32_t dtype;
} VmoeAttentionParams;
int vmoe_attention(const VmoeAttentionParams* p, vmoe_stream_t stream);

/* ---------------------------------------------------------------------------------------
 * Measurement aids.  Nothing below has a counterpart in the reference and no product path
 * calls it: these entry points produce the ceilings (copy rate, register-resident MFMA rate,
 * operand delivery rate) that the bandwidth and arithmetic figures are compared with.
 * --------------------------------------------------------------------------------------- */

/* Plain device copy kernel of n bytes (n % 16 == 0); the measured HBM ceiling
 * that bandwidth figures are compared with. */
int vmoe_copy_bytes(const void* in, void* out, size_t n, vmoe_stream_t stream);

/* Register-resident v_mfma_f32_32x32x16_bf16 loop: the measured arithmetic
 * ceiling that the expert GEMM figures are compared with (no counterpart in the
 * reference; measurement aid like vmoe_copy_bytes).  Operand fragments are read
 * once from `seed` (seed_bytes >= 16, 16-byte aligned); `sink` receives
 * blocks * 256 floats; *flops is set to the floating-point operations issued. */
int vmoe_mfma_probe(const void* seed, size_t seed_bytes, void* sink, int32_t blocks,
                    int32_t iters, double* flops, vmoe_stream_t stream);

/* Load-only counterpart of the 256 x 256 expert product (no counterpart in the
 * reference; measurement aid like vmoe_mfma_probe): issues exactly the operand-tile
 * loads of C[b] = A[b] (rows x kd) . Bt[b] (n x kd)^T, bfloat16, global memory -> LDS, in
 * the product's tile order and does nothing with them.  *bytes is set to the operand
 * bytes moved (tiles x 512 rows x kd x 2); bytes / time is the rate that bounds any
 * kernel of this tiling, and x 128 flop/byte its ceiling in FLOP/s.  kd % 32 == 0. */
int vmoe_operand_delivery_probe(const void* a, const void* bt, int32_t batch, int32_t rows,
                                int32_t n, int32_t kd, double* bytes, vmoe_stream_t stream);

/* The same with 64-wide k tiles, as the tile-walking second product requests them: a row
 * segment of a request is 128 bytes instead of 64 and one to two k tiles stay in flight
 * (no counterpart in the reference; measurement aid).  kd % 64 == 0. */
int vmoe_operand_delivery_probe_k64(const void* a, const void* bt, int32_t batch, int32_t rows,
                                    int32_t n, int32_t kd, double* bytes, vmoe_stream_t stream);

/* The same kind of requests over tiles that the workgroups share (no counterpart in the reference;
 * measurement aid): 256 workgroups walk tiles_per_workgroup tiles each, taken round robin
 * from the buf_bytes / (512 * row_bytes) tiles of 512 rows x row_bytes that `buf` holds, in
 * k_tiles steps of 128 bytes per row (k_tiles * 128 <= row_bytes), two steps in flight;
 * segment_bytes = 128: a request is 8 rows x 128 bytes, 64: 16 rows x 64 bytes.  *bytes is
 * set to the bytes moved into LDS.  With few tiles in `buf` (less than the caches hold)
 * hardly a request waits for HBM: bytes / time against the other delivery probes' rates is
 * what the products' misses cost at their ring depth. */
int vmoe_resident_delivery_probe(const void* buf, size_t buf_bytes, int32_t row_bytes,
                                 int32_t k_tiles, int32_t tiles_per_workgroup,
                                 int32_t segment_bytes, double* bytes, vmoe_stream_t stream);

#ifdef __cplusplus
}
#endif
#endif /* VMOE_HIP_H_ */
