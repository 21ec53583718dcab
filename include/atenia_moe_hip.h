/*
 * atenia_moe_hip.h -- C ABI of the MI355X (gfx950) mixture-of-experts layer forward.
 *
 * This is the boundary a host (Rust via `extern "C"`, C++, Python/ctypes) binds to run the
 * reference's MoE layer op on one GPU.  It takes the place of the reference's `src/cuda`
 * FFI for this path: plain pointers, `int` dimensions, `int` return codes, no exceptions
 * and no unwinding across the boundary -- the conventions of the reference's launchers
 * (`matmul_f32_launch_device`, src/cuda/matmul_kernel.cu:28-55 and src/cuda/matmul.rs:21-32;
 * `launch_linear_f32_device_ptrs`, src/cuda/linear_cuda.cu:36-73;
 * `int8_to_bf16_per_channel_launch_device`, src/cuda/int8_to_bf16.cu:42-71).
 *
 * Return codes (every entry point that returns `int`):
 *    0  success
 *    1  a stream/device synchronisation failed          (linear_cuda.cu:60-70 uses 1)
 *    2  a kernel launch or runtime call failed          (linear_cuda.cu:44-45 uses 2)
 *   -1  bad dimensions / null pointer / length mismatch (MoeDenseError::DimMismatch,
 *                                                        src/moe/dense.rs:31-49)
 *   -2  bad k: k == 0 or k > num_experts                (MoeSparseError::ZeroK /
 *                                                        KExceedsExperts, src/moe/sparse.rs:35-50)
 *   -3  a routing weight is not finite                  (MoeSparseError::NonFiniteWeight{index},
 *                                                        src/moe/sparse.rs:156-160); token and
 *                                                        expert via ..._layer_status (device
 *                                                        entry points) or ..._last_non_finite
 *   -4  out of device memory
 *   -5  invalid handle / unknown layer                  (MoeBindingError::LayerNotFound)
 *   -6  configuration not supported by this build
 * A non-zero code leaves the outputs unspecified; the reference's wrappers treat a non-zero
 * launcher code as "fall back to the CPU path" (src/cuda/matmul.rs:131-150) and a host
 * keeps that choice.  This library itself never computes on the CPU.
 *
 * Threading: any thread may call; one handle is NOT re-entrant (it owns one workspace) and
 * calls on the same handle are serialised by an internal mutex, as the reference serialises
 * forwards behind its registry mutex (src/moe/graph_op.rs:304-316).  The asynchronous entry
 * points keep that promise on the device as well: a call whose stream differs from the stream
 * of the handle's previous call first waits (hipStreamWaitEvent) for that call's kernels, so
 * two streams never use one workspace at the same time.  A stream may be destroyed as soon as
 * the call that took it has returned: the handle marks the end of each forward on a stream the
 * caller made with an event of its own and never touches that stream again (the null stream and
 * the handle's own streams are marked only when the next call changes the stream: one event per
 * forward costs a decode step microseconds).  The one exception is a stream that is
 * being captured into a HIP graph: no cross-stream wait is recorded there, and replays of graphs
 * that hold calls on one handle must be ordered by the caller.  Different handles may run
 * concurrently.  A layer with a shared expert owns a second stream (default priority): in
 * batches where that expert takes launches of its own they run there, beside the routed
 * experts' on the caller's stream, between an event recorded on the caller's stream and one it
 * waits for before the call's last launch -- everything a call enqueues is complete when the
 * caller's stream has passed the call (never under stream capture nor from the entry point that
 * allocates nothing: there all launches stay on the caller's stream).
 */
#ifndef ATENIA_MOE_HIP_H
#define ATENIA_MOE_HIP_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* MoeExecutionConvention (src/moe/layer.rs:185-195). */
#define ATENIA_MOE_CONVENTION_ATENIA 0           /* renormalise top-k weights; ungated shared */
#define ATENIA_MOE_CONVENTION_HUGGINGFACE_QWEN 1 /* raw softmax weights; sigmoid-gated shared */

/* Storage type of the expert weights, on the host side of `create` and in HBM. */
#define ATENIA_MOE_WEIGHT_F32 0        /* TensorStorage::Cpu      (src/tensor/tensor.rs:93-160) */
#define ATENIA_MOE_WEIGHT_BF16 1       /* TensorStorage::CpuBf16, raw u16 bit patterns          */
#define ATENIA_MOE_WEIGHT_INT8_W8A16 2 /* per-output-row int8 + f32 scales
                                          (src/tensor/disk_tier.rs:231-259)                     */
/* int8 with one f32 scale per output row and per group of `group_size` consecutive input
 * elements (Q8_0-style; the reference's per-group scheme, src/tensor/quantizer.rs:175-248, laid
 * out for [out, in] weights): scales are [.., rows, ceil(cols / group_size)]. */
#define ATENIA_MOE_WEIGHT_INT8_PER_GROUP 3

/* Element type of device activations handed to `forward_device`. */
#define ATENIA_MOE_ACT_F32 0
#define ATENIA_MOE_ACT_BF16 1
/* Arithmetic of the RMSNorm in front of the layer (atenia_moe_hip_layer_block_forward*). */
#define ATENIA_MOE_NORM_GRAPH_F32 0 /* graph nodes: f32 left-to-right sum, (x*inv)*gamma in f32 */
#define ATENIA_MOE_NORM_F64 1       /* imperative decoders: f64 sum and inverse root */

#define ATENIA_MOE_OK 0
#define ATENIA_MOE_ERR_SYNC 1
#define ATENIA_MOE_ERR_LAUNCH 2
#define ATENIA_MOE_ERR_DIM (-1)
#define ATENIA_MOE_ERR_K (-2)
#define ATENIA_MOE_ERR_NON_FINITE (-3)
#define ATENIA_MOE_ERR_OOM (-4)
#define ATENIA_MOE_ERR_HANDLE (-5)
#define ATENIA_MOE_ERR_UNSUPPORTED (-6)

typedef struct AteniaMoeLayer AteniaMoeLayer; /* opaque; owns weights + workspace in HBM */

/*
 * Everything `create` needs; all pointers are HOST pointers borrowed for the call only
 * (the reference's launch helpers borrow host slices the same way,
 * src/cuda/pool_helpers.rs:118-128).  Mirrors RealMoeLayer + MoeLayerConfig
 * (src/moe/layer.rs:37-43,200-212) with flat arrays.
 *
 * Expert weights are row-major "[out, in]" exactly as the reference holds them
 * (src/moe/dense.rs:203-210): gate/up `[E, f, d]`, down `[E, d, f]`.  The packed checkpoint
 * layout `[E, 2f, d]` (gate = rows 0..f, up = rows f..2f; src/moe/binding.rs:384-413) is
 * passed as `w_gate` with `w_up == NULL`.
 */
typedef struct AteniaMoeLayerDesc {
  int32_t num_experts;     /* E  >= 1                                                    */
  int32_t top_k;           /* k  = experts_per_token, 1 <= k <= E                        */
  int32_t d_model;         /* d                                                          */
  int32_t d_ff;            /* f  (routed expert width)                                   */
  int32_t d_ff_shared;     /* f_s, 0 = no shared expert                                  */
  int32_t convention;      /* ATENIA_MOE_CONVENTION_*                                    */
  int32_t weight_dtype;    /* ATENIA_MOE_WEIGHT_* (applies to routed and shared experts) */
  int32_t max_tokens_hint; /* workspace is sized for this many tokens up front (0 = lazy) */

  const float* w_router;    /* f32 [E, d]; the router is always f32 (src/moe/dense.rs:325-337) */
  const float* router_bias; /* f32 [E] added to the f32 logits before softmax, or NULL.
                               Extension with no counterpart in the reference router.    */

  const void* w_gate;       /* [E, f, d], or packed [E, 2f, d] when w_up == NULL         */
  const void* w_up;         /* [E, f, d] or NULL                                         */
  const void* w_down;       /* [E, d, f]                                                 */
  const float* scale_gate;  /* int8 only: f32 [E, f]  one scale per output row           */
  const float* scale_up;    /* int8 only: f32 [E, f]                                     */
  const float* scale_down;  /* int8 only: f32 [E, d]                                     */

  const void* s_gate;       /* shared expert [f_s, d]  (NULL when f_s == 0)              */
  const void* s_up;         /* [f_s, d]                                                  */
  const void* s_down;       /* [d, f_s]                                                  */
  const float* s_scale_gate; /* int8 only: f32 [f_s]                                     */
  const float* s_scale_up;   /* int8 only: f32 [f_s]                                     */
  const float* s_scale_down; /* int8 only: f32 [d]                                       */
  const float* shared_gate; /* f32 [d] sigmoid gate vector (src/moe/layer.rs:436-443) or NULL */
  int32_t group_size;       /* ATENIA_MOE_WEIGHT_INT8_PER_GROUP only: input elements per scale,
                               a multiple of 64 (128 = the reference's production value); the
                               scale arrays are then [E, f, ceil(d/gs)], [E, f, ceil(d/gs)],
                               [E, d, ceil(f/gs)] and [f_s, ..] / [d, ceil(f_s/gs)] for the
                               shared expert.  0 otherwise.                               */
} AteniaMoeLayerDesc;

/* 1 when a gfx950 device is present and usable, else 0.  Replaces `cuda_available()`
 * (src/cuda/mod.rs:61-70); the result is computed once per process. */
int atenia_moe_hip_available(void);

/* Human-readable text of the calling thread's most recent failure ("" if none). */
const char* atenia_moe_hip_last_error_string(void);

/* Per-group symmetric int8 quantisation of a row-major [rows, cols] weight, groups of
 * `group_size` consecutive elements of a row: scale = max(max|w| / 127, 1e-12), q = round(w /
 * scale) clamped to [-127, 127]; scales out: [rows, ceil(cols / group_size)].  The arithmetic of
 * absmax_per_group_symmetric (src/tensor/quantizer.rs:175-248), which walks a [K, N] weight in
 * groups along K; here K is the row's own direction.  Host function. */
int atenia_moe_quantize_per_group_i8(const float* w, size_t rows, size_t cols, size_t group_size,
                                     int8_t* q_out, float* scales_out);

/* Uploads the layer once; the handle owns the device copies, as the reference registry owns
 * its `Arc<RealMoeLayer>` (src/moe/graph_op.rs:228-232).  Replaces the per-call H->D upload of
 * the `Fast` policy (src/moe/dense.rs:146-152 -> src/cuda/matmul.rs:131-203). */
int atenia_moe_hip_layer_create(const AteniaMoeLayerDesc* desc, AteniaMoeLayer** out_layer);
int atenia_moe_hip_layer_destroy(AteniaMoeLayer* layer);

/* The op: `[T*d]` f32 in host memory -> `[T*d]` f32 in host memory, the WHOLE batch in one
 * call.  Replaces the per-row loop of `execute_real_moe_layer`
 * (src/moe/graph_op.rs:327-350) and everything below it (src/moe/layer.rs:405-431,
 * src/moe/sparse.rs:218-238, src/moe/dense.rs:253-270).  Synchronous.  T == 0 is a no-op. */
int atenia_moe_hip_layer_forward(AteniaMoeLayer* layer, const float* x_host, int n_tokens,
                                 float* out_host);

/* Same op on device-resident activations, asynchronous on `stream` (a hipStream_t; NULL =
 * the default stream).  x: [T, d] of `x_dtype`; out: [T, d] f32.  The call allocates only
 * when the workspace has to grow (n_tokens above every earlier call and the create hint).
 * Errors detected on the device (-3) are reported by atenia_moe_hip_layer_status. */
int atenia_moe_hip_layer_forward_device(AteniaMoeLayer* layer, const void* d_x, int x_dtype,
                                        int n_tokens, float* d_out, void* stream);

/* atenia_moe_hip_layer_forward_device for callers that cannot allocate: code under HIP graph
 * capture, tight serving loops, harnesses that forbid hipMalloc.  No counterpart in the
 * reference.  Same op, same arguments and the same kernels, but the workspace (routing, grouping,
 * the h rows, the per-pair expert outputs) is a 16 MiB buffer that lives in the library's own
 * device image from load time on, one per GPU, instead of the handle's grow-on-demand
 * allocation: the call makes no hipMalloc / hipFree and no allocating library call, whatever
 * n_tokens was seen before.  A batch whose workspace does not fit (about T * top_k * (2 * d_ff +
 * 4 * d_model) bytes for the streaming kernels that serve decode batches; the Mixtral shape fits
 * up to 85 tokens, i.e. every batch those kernels take) is refused with ATENIA_MOE_ERR_UNSUPPORTED and a message that names both sizes; so
 * is an int8 batch large enough to need the layer's bf16 copy (per-group scales: any batch for
 * the tiled kernels; W8A16: from 256 rows per expert) before an allocating call has made it.  All handles on one GPU share that GPU's buffer, which keeps the previous
 * call's contents: the call rewrites what must start from a known state with a small kernel on
 * `stream` (no memset nodes), and calls that overlap in time on one GPU -- different handles
 * included -- race on it; order them on one stream or with events.  The status word of
 * ..._layer_status and the taps (..._last_routing, ..._last_expert_outputs) work as after
 * atenia_moe_hip_layer_forward_device until the next no-alloc call on the GPU. */
int atenia_moe_hip_layer_forward_device_noalloc(AteniaMoeLayer* layer, const void* d_x, int x_dtype,
                                                int n_tokens, float* d_out, void* stream);

/* Switches the handle's router to DeepSeek-V3 routing (src/moe/v3_router.rs:36-52, 206-309):
 * scores = sigmoid(W_r x) instead of a softmax, selection on scores + e_score_correction_bias
 * ([E] f32, host) limited to the `topk_group` best of `n_group` expert groups (group score = its
 * two largest corrected scores), combine weights = the uncorrected scores of the top_k selected
 * experts, normalised when `norm_topk_prob`, times `routed_scaling_factor`.  top_k is the
 * layer's.  The shared expert, if any, is added ungated, as DeepSeek's shared experts are.
 * Configuration errors are the reference's V3RouterError cases (rc ATENIA_MOE_ERR_K, or
 * ATENIA_MOE_ERR_NON_FINITE for a non-finite bias, with its message text); a non-finite logit
 * at run time is reported like a non-finite routing weight (rc -3, token and expert).  Every
 * later forward / route / stage launch of the handle uses it. */
int atenia_moe_hip_layer_set_v3_router(AteniaMoeLayer* layer, int n_group, int topk_group,
                                       double routed_scaling_factor, int norm_topk_prob,
                                       const float* e_score_correction_bias_host);

/* The FFN block of a decoder layer around the op, on device-resident rows, asynchronous on
 * `stream`:  out[t] = x1[t] + MoE(RMSNorm(x1[t]) * gamma),  x1 / out: [T, d] f32, gamma: [d] f32.
 * Replaces steps 13-15 of the reference's layer loop -- the RmsNorm, BroadcastMul,
 * MoeRealLayerReference and Add nodes of src/moe/full_forward.rs:239-252 (also
 * src/moe/generate.rs:161-170, src/moe/decoder_layer.rs:199-210), whose executor copies every
 * node's tensor to the host (`ensure_cpu`, src/amg/graph.rs:5361, 5580) -- and the imperative
 * form of src/moe/mla.rs:442-453.  `norm_policy` picks the reference arithmetic of the norm:
 * ATENIA_MOE_NORM_GRAPH_F32 = src/nn/normalization.rs:8-37 + broadcast_mul
 * (src/amg/graph.rs:6647-6673); ATENIA_MOE_NORM_F64 = src/moe/mla.rs:230-239.
 * d_out may be d_x1 (the residual stream is updated in place).  Pointers are 16-byte aligned
 * when d % 4 == 0.  The normalised rows stay in the handle (tap: ..._last_normed). */
int atenia_moe_hip_layer_block_forward_device(AteniaMoeLayer* layer, const float* d_x1,
                                              int n_tokens, const float* d_gamma, float eps,
                                              int norm_policy, float* d_out, void* stream);

/* Same block with host buffers (x1, out: [T*d]; gamma: [d]); synchronous. */
int atenia_moe_hip_layer_block_forward(AteniaMoeLayer* layer, const float* x1_host, int n_tokens,
                                       const float* gamma_host, float eps, int norm_policy,
                                       float* out_host);

/* Waits for the handle's last forward and returns its device-side status: 0, or -3 with the
 * first offending token / expert (either pointer may be NULL). */
int atenia_moe_hip_layer_status(AteniaMoeLayer* layer, void* stream, int32_t* token,
                                int32_t* expert);

/* Where the most recent ATENIA_MOE_ERR_NON_FINITE of this handle was found: token (row of the
 * batch) and expert index, -1 / -1 if none was ever reported.  The index is the `index` of the
 * reference's MoeSparseError::NonFiniteWeight (src/moe/sparse.rs:41-42, 150-158); the host
 * entry points consume the device status themselves, so this is how their caller learns it. */
int atenia_moe_hip_layer_last_non_finite(AteniaMoeLayer* layer, int32_t* token, int32_t* expert);

/* Parity taps -------------------------------------------------------------------------- */

/* Router + softmax + top-k only (src/moe/dense.rs:325-337, src/moe/sparse.rs:142-191):
 * idx[T*k] ascending per token, w[T*k] the (re)normalised f32 weights; host buffers. */
int atenia_moe_hip_layer_route(AteniaMoeLayer* layer, const float* x_host, int n_tokens,
                               int32_t* idx_host, float* w_host);

/* Expert grouping of a given routing: counts[E], offsets[E+1], perm[T*k] (pair ids t*k+slot
 * in expert-major order, stable in pair id); host buffers.  No reference counterpart: the
 * contract is derived from the reference's visiting order (src/moe/graph_op.rs:345-348,
 * src/moe/sparse.rs:175). */
int atenia_moe_hip_layer_permute(AteniaMoeLayer* layer, const int32_t* idx_host, int n_tokens,
                                 int32_t* counts_host, int32_t* offsets_host,
                                 int32_t* perm_host);

/* ---- stage launchers: the four kernels of the pipeline, one call each, device pointers ----
 * Same convention as the reference's device launchers (matmul_f32_launch_device,
 * src/cuda/matmul.rs:37-47: raw device pointers and int dimensions in, int code out) applied to
 * the stages of src/moe/layer.rs:405-431.  Each stage reads what the stages before it left in
 * the handle's workspace, so they are called in order router -> permute -> expert_ffn ->
 * combine for the same n_tokens and the same activations; calling a stage whose predecessors
 * have not run for that n_tokens returns ATENIA_MOE_ERR_DIM.  All four are asynchronous on
 * `stream`; the four calls together are exactly atenia_moe_hip_layer_forward_device. */

/* Kernel 1 (src/moe/dense.rs:325-337, 172-187; src/moe/sparse.rs:142-191).  d_idx / d_w
 * (device, [n_tokens * top_k], either may be NULL) receive copies of the routing. */
int atenia_moe_router_launch_device(AteniaMoeLayer* layer, const void* d_x, int x_dtype,
                                    int n_tokens, int32_t* d_idx, float* d_w, void* stream);

/* Kernel 2 (expert grouping; contract of atenia_moe_hip_layer_permute).  d_counts [E],
 * d_offsets [E+1], d_perm [n_tokens * top_k]: device, any may be NULL. */
int atenia_moe_permute_launch_device(AteniaMoeLayer* layer, int n_tokens, int32_t* d_counts,
                                     int32_t* d_offsets, int32_t* d_perm, void* stream);

/* Kernel 3, both phases (src/moe/dense.rs:253-270), routed and shared experts.  d_x must be
 * the activations the router stage was given. */
int atenia_moe_expert_ffn_launch_device(AteniaMoeLayer* layer, const void* d_x, int x_dtype,
                                        int n_tokens, void* stream);

/* Kernel 4 (src/moe/sparse.rs:226-233, src/moe/layer.rs:415-429).  d_out: [n_tokens, d_model]
 * f32 on the device. */
int atenia_moe_combine_launch_device(AteniaMoeLayer* layer, int n_tokens, float* d_out,
                                     void* stream);

/* Routing/grouping of the handle's most recent forward, copied to host buffers (any pointer
 * may be NULL): idx[T*k], w[T*k], counts[E], offsets[E+1], perm[T*k]. */
int atenia_moe_hip_layer_last_routing(AteniaMoeLayer* layer, int32_t* idx_host, float* w_host,
                                      int32_t* counts_host, int32_t* offsets_host,
                                      int32_t* perm_host);

/* Per-(token, slot) expert outputs of the most recent forward, before the weighted combine:
 * y[T*k, d] f32 in pair order (row t*k+slot = expert idx[t,slot] applied to token t), and the
 * shared expert's y_shared[T, d] (NULL to skip / when there is none).  Host buffers.  Serves
 * the per-expert parity obligation of the reference's certification ladder
 * (docs/decisions/ADR-007-moe-certification-ladder.md:62-73). */
int atenia_moe_hip_layer_last_expert_outputs(AteniaMoeLayer* layer, float* y_host,
                                             float* y_shared_host);

/* Parity tap next to the one above: into how many k ranges the last forward's down launch cut the
 * tile behind each expert-output row and 256-column block, parts_host[n_tokens * top_k,
 * ceil(d_model / 256)] (1 everywhere unless the matrix-core down launch split the tiles of its
 * last, partly filled round; range i of S covers the 64-k stages [n*i/S, n*(i+1)/S) of the n =
 * ceil(d_ff / 64) stages).  An expert output there is the sum, in range order, of its partial
 * sums -- each rounded to bf16 first when the outputs travel as bf16 (atenia_moe_hip_plan_batch).
 * No counterpart in the reference; tests use it to restate the kernels' arithmetic exactly. */
int atenia_moe_hip_layer_last_down_split(AteniaMoeLayer* layer, uint8_t* parts_host);

/* The rows the MoE layer saw in the most recent block forward: RMSNorm(x1) * gamma, [T, d] f32,
 * host buffer (the `h2` of src/moe/full_forward.rs:243). */
int atenia_moe_hip_layer_last_normed(AteniaMoeLayer* layer, float* h2_host);

/* Stage timing with HIP events recorded on the forward's own stream.  After
 * `set_profiling(layer, 1)` every forward records an event before/after each stage;
 * `stage_ms` waits for the last forward and returns that forward's durations in
 * milliseconds: [0] router, [1] permute, [2] expert gate/up (+shared), [3] expert down
 * (+shared), [4] combine, [5] whole forward.  `stage_launches` returns the kernel count of
 * each stage so a per-launch mean can be formed. */
#define ATENIA_MOE_N_STAGES 6
int atenia_moe_hip_layer_set_profiling(AteniaMoeLayer* layer, int enabled);
int atenia_moe_hip_layer_stage_ms(AteniaMoeLayer* layer, float ms[ATENIA_MOE_N_STAGES]);
int atenia_moe_hip_layer_stage_launches(AteniaMoeLayer* layer, int32_t n[ATENIA_MOE_N_STAGES]);

/* Expert arithmetic of a layer with f32 weights, the reference's NumericPolicy
 * (src/moe/numeric_policy.rs:36-75; selection in `matvec_policy`, src/moe/dense.rs:159-168):
 *   CERTIFIED  f64 accumulation (default; the bit-exact reference arithmetic)
 *   STRICT     f32 accumulation, product and sum rounded separately, columns ascending
 *              (`matvec_f32`, src/moe/dense.rs:120-140)
 *   FAST       f32 on the GPU; the reference sends each projection through `cuda_matmul` and
 *              falls back to the Strict arithmetic, which is what this library computes
 * The router accumulates in f64 under every policy, so routing never changes.  Layers stored
 * as bf16 / int8 multiply on the matrix cores with f32 accumulation whatever the policy; the
 * call is accepted for them and changes nothing.  Takes effect from the next forward. */
#define ATENIA_MOE_POLICY_CERTIFIED 0
#define ATENIA_MOE_POLICY_STRICT 1
#define ATENIA_MOE_POLICY_FAST 2
int atenia_moe_hip_layer_set_numeric_policy(AteniaMoeLayer* layer, int policy);

/* Layer facts a host needs to size buffers: writes E, k, d, f, f_s, convention,
 * weight_dtype, bytes of expert weights per routed expert as stored in HBM. */
int atenia_moe_hip_layer_info(const AteniaMoeLayer* layer, int64_t info[8]);

/* Which expert kernels a batch of `n_tokens` tokens takes on this layer (a pure function of the
 * layer and the batch size, nothing is launched): family[0] for the routed experts, family[1]
 * for the shared expert (-1 without one); where the two phases differ, that of the gate/up phase.  No counterpart in the reference, whose CPU path has
 * one expert loop (src/moe/layer.rs:405-443); a host uses it to see where its batch sizes fall
 * and tests use it to know which kernel they exercised. */
#define ATENIA_MOE_KERNELS_STREAM 0 /* weights streamed once, token rows in registers (decode) */
#define ATENIA_MOE_KERNELS_MID 1    /* weights streamed once per 128 rows, token rows through LDS */
#define ATENIA_MOE_KERNELS_TILED 2  /* 256-row tiles, matrix-core bound (prefill) */
#define ATENIA_MOE_KERNELS_F32 3    /* f32 weights, f64 or f32 accumulation */
int atenia_moe_hip_layer_expert_kernels(const AteniaMoeLayer* layer, int64_t n_tokens,
                                        int32_t family[2]);

/* The same question without a layer or a device: which kernels a batch of `n_tokens` tokens takes
 * on a layer of these dimensions (weight_dtype / group_size as in AteniaMoeLayerDesc).  A pure
 * function of its arguments and of the tuning knobs in the environment.  plan[0] / plan[1]:
 * family of the routed experts' gate/up and down phase (ATENIA_MOE_KERNELS_*); plan[2] / plan[3]:
 * the same for the shared expert (-1 without one); plan[4] / plan[5]: 1 when the routed / shared
 * expert outputs travel to the combine as bf16 instead of f32 (bf16 layers on the matrix-core
 * kernels); plan[6]: 1 when row tiles may hold nine 32-row groups; plan[7]: bit 0 / bit 1 set when
 * the gate/up / down phase takes the tiled form with two workgroups per compute unit, bit 2 when
 * a W8A16 layer's tiled phases run on a bf16 copy of its int8 values (which the first such batch
 * makes: twice the int8 bytes again).  No counterpart in the reference; hosts and tests use it to
 * see where a batch size falls. */
int atenia_moe_hip_plan_batch(int num_experts, int top_k, int d_model, int d_ff, int d_ff_shared,
                              int weight_dtype, int group_size, int64_t n_tokens,
                              int32_t plan[8]);

/* Host-side weight preparation (load time, no GPU involved) ------------------------------ */

/* Per-output-row symmetric int8 quantisation, bit-identical to `quantize_per_row_i8`
 * (src/tensor/disk_tier.rs:231-248): scale = amax/127 (1 for an all-zero row),
 * q = clamp(round_half_away(w * (1/scale)), -127, 127). */
int atenia_moe_quantize_per_row_i8(const float* w, size_t rows, size_t cols, int8_t* q,
                                   float* scales);
/* Symmetric int8 quantisation of a row-major [K, N] weight in the reference's own orientation
 * (K = input, N = output channel): one scale per column (`absmax_per_channel_symmetric`,
 * src/tensor/quantizer.rs:67-117; scales [N]) or per column and group of `group_size`
 * consecutive k (`absmax_per_group_symmetric`, src/tensor/quantizer.rs:175-248; scales
 * [ceil(K / group_size), N]): scale = max(max|w| / 127, 1e-12), q = clamp(round(w / scale)). */
int atenia_moe_absmax_per_channel_symmetric(const float* w, size_t k, size_t n, int8_t* q,
                                            float* scales);
int atenia_moe_absmax_per_group_symmetric(const float* w, size_t k, size_t n, size_t group_size,
                                          int8_t* q, float* scales);
/* f32 -> bf16 bit patterns by truncation (`f32_to_bf16_bits`, src/tensor/tensor.rs:306-308). */
int atenia_moe_f32_to_bf16_trunc(const float* src, size_t n, uint16_t* dst);

/* INT8 -> BF16 dequantisation on the device ----------------------------------------------- */

/* out[k, n] = truncate_to_bf16((float)q[k, n] * scales[n]) over a row-major [K, N] int8 weight;
 * device pointers, asynchronous on `stream` (a hipStream_t; NULL = the default stream).
 * Returns 0, a negative value for bad arguments (-1 null pointer, -2 group_size <= 0) or the
 * runtime's launch status; k * n <= 0 is a no-op.  Replaces
 * `int8_to_bf16_per_channel_launch_device` (src/cuda/int8_to_bf16.cu:42-71). */
int atenia_moe_int8_to_bf16_per_channel_launch_device(const void* d_int8, const float* d_scales,
                                                      void* d_bf16, int k, int n, void* stream);
/* Same with scales [ceil(K / group_size), N]: scale of (k, n) = scales[(k / group_size) * N + n].
 * Replaces `int8_to_bf16_per_group_launch_device` (src/cuda/int8_to_bf16.cu:112-141). */
int atenia_moe_int8_to_bf16_per_group_launch_device(const void* d_int8, const float* d_scales,
                                                    void* d_bf16, int k, int n, int group_size,
                                                    void* stream);
/* The same two launchers under the reference's own symbol names and argument lists (default
 * stream), so that its FFI block (src/cuda/int8_to_bf16.rs:63-81) binds without a change. */
int int8_to_bf16_per_channel_launch_device(const void* d_int8, const float* d_scales,
                                           void* d_bf16, int k, int n);
int int8_to_bf16_per_group_launch_device(const void* d_int8, const float* d_scales, void* d_bf16,
                                         int k, int n, int group_size);

#ifdef __cplusplus
}
#endif
#endif /* ATENIA_MOE_HIP_H */
