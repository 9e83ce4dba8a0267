/*
 * rbmoe.h — C ABI of the MI355X (gfx950) mixture-of-experts layer.
 *
 * Drop-in boundary for RustingBrain's `MoeLayer`: the forward pass with the two
 * auxiliary losses (reference src/moe.rs:203-341), the backward pass
 * (src/moe.rs:348-489) and the block's RMSNorm and residual add either side of
 * the layer (src/transformer_block.rs:216-222, 257-263).  The reference
 * has no FFI seam for this layer; each entry point below names the reference
 * interface it stands in for, so that a Rust `extern "C"` block can bind them
 * one to one.  Plain pointers and sizes only.  Every function returns an
 * `rbmoe_status`; none throws, aborts or falls back to a CPU path.
 *
 * Matrices are row-major and contiguous, exactly like the reference `Matrix`
 * (src/matrix.rs:13-18).  A `Linear` weight is `[out_features, in_features]`
 * (src/param.rs:620-633): router `[E, d]`, gate/up `[F, d]`, down `[d, F]`.
 */
#ifndef RBMOE_H
#define RBMOE_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* Mirrors the `NetworkError` variants that can leave this path
 * (reference src/network.rs:19-83). */
typedef enum rbmoe_status {
    RBMOE_OK = 0,
    RBMOE_INVALID_INPUT = 1,      /* NetworkError::InvalidInput{expected, actual}      */
    RBMOE_INVALID_CONFIG = 2,     /* NetworkError::InvalidConfig(String)               */
    RBMOE_DEVICE_ERROR = 3,       /* NetworkError::Cuda(String): a HIP call failed     */
    RBMOE_BACKEND_UNAVAILABLE = 4,/* NetworkError::CudaFeatureDisabled: no usable GPU  */
    RBMOE_MEMORY_BUDGET = 5,      /* NetworkError::CudaMemoryBudget{estimated, budget} */
    RBMOE_OUT_OF_MEMORY = 6,      /* NetworkError::CudaOutOfMemory{requested, free}    */
    RBMOE_UNSUPPORTED = 7,        /* NetworkError::UnsupportedCuda(String)             */
    RBMOE_NULL_POINTER = 8        /* a required pointer argument was NULL              */
} rbmoe_status;

typedef enum rbmoe_dtype {
    RBMOE_F32 = 0,
    RBMOE_BF16 = 1,  /* raw 16-bit patterns, round-to-nearest-even from f32 */
    RBMOE_I8 = 2     /* weights only: symmetric int8 + one f32 scale per output row */
} rbmoe_dtype;

/* Which weight of the layer; the order is the reference's parameter traversal
 * (src/moe.rs:516-525 with src/ffn.rs:126-131). */
typedef enum rbmoe_weight {
    RBMOE_W_ROUTER = 0,       /* [E, d]              Router.projection  (src/moe.rs:91-100) */
    RBMOE_W_GATE = 1,         /* [F, d]  per expert  SwiGlu.gate        (src/ffn.rs:19-23)  */
    RBMOE_W_UP = 2,           /* [F, d]  per expert  SwiGlu.up                              */
    RBMOE_W_DOWN = 3,         /* [d, F]  per expert  SwiGlu.down                            */
    RBMOE_W_SHARED_GATE = 4,  /* [Fs, d]             MoeLayer.shared    (src/moe.rs:210)    */
    RBMOE_W_SHARED_UP = 5,    /* [Fs, d]                                                    */
    RBMOE_W_SHARED_DOWN = 6,  /* [d, Fs]                                                    */
    RBMOE_W_NORM = 7          /* [1, d]  feed_forward_norm.weight: rbmoe_get_weight_grad only  */
} rbmoe_weight;

/* `MoeConfig` (reference src/moe.rs:25-39) plus what a device layer must know
 * up front.  `shared_d_ff` exists because the reference's `shared` field is
 * public and may hold an expert of another width (src/moe.rs:210, used that way
 * at src/moe.rs:841-843); 0 means "same as d_ff". */
typedef struct rbmoe_config {
    int32_t d_model;
    int32_t num_experts;
    int32_t experts_per_token;
    int32_t d_ff;
    int32_t shared_expert;         /* 0 / 1 */
    int32_t shared_d_ff;           /* 0 = d_ff */
    float aux_loss_weight;         /* DEFAULT_AUX_LOSS_WEIGHT = 0.01 (src/moe.rs:20)           */
    float router_z_loss_weight;    /* DEFAULT_ROUTER_Z_LOSS_WEIGHT = 1e-3 (src/moe.rs:23)      */
    int32_t weight_dtype;          /* rbmoe_dtype of the expert weights                        */
    int32_t act_dtype;             /* rbmoe_dtype of x / out: RBMOE_F32 or RBMOE_BF16          */
    int32_t max_tokens;            /* workspace is sized for this many rows; forward allocates nothing */
} rbmoe_config;

/* Routing tables of the last forward, the bit-exact comparands.
 * Slot s = token * k + rank (rank 0 = highest probability), as the reference's
 * `assignments` (src/moe.rs:142-145).  All pointers are optional (NULL = skip)
 * and must be host memory. */
typedef struct rbmoe_routing {
    int32_t* expert_of;   /* [T*k]  expert per slot, -1 = UNROUTED (src/moe.rs:190-191) */
    float* gate_of;       /* [T*k]  renormalised gate per slot                          */
    int32_t* counts;      /* [E]    expert_tokens[e].len() (src/moe.rs:266-274)         */
    int32_t* offsets;     /* [E+1]  exclusive prefix of counts                          */
    int32_t* perm_slot;   /* [T*k]  expert_slots, experts concatenated; first offsets[E] valid  */
    int32_t* perm_token;  /* [T*k]  expert_tokens, experts concatenated                 */
    float* probabilities; /* [T*E]  MoeCache.probabilities (src/moe.rs:137-140)         */
    float* log_sum_exp;   /* [T]    MoeCache.log_sum_exp   (src/moe.rs:141-142)         */
} rbmoe_routing;

typedef struct rbmoe_ctx rbmoe_ctx;
typedef struct rbmoe_layer rbmoe_layer;

/* MoeConfig::new (src/moe.rs:41-51): defaults for everything but the three
 * arguments; dtypes default to f32, max_tokens to 0 (must be set). */
int rbmoe_config_init(rbmoe_config* cfg, int32_t d_model, int32_t num_experts,
                      int32_t experts_per_token, int32_t d_ff);

/* MoeConfig::validate (src/moe.rs:68-86) plus dtype/limit checks.  Touches no
 * GPU.  On failure writes a message (same wording as the reference where one
 * exists) into `msg` if `msg_cap` > 0. */
int rbmoe_validate(const rbmoe_config* cfg, char* msg, size_t msg_cap);

/* TransformerConfig::parameter_counts restricted to one layer
 * (src/transformer.rs:194-227; MoeLayer::num_parameters / active_parameters,
 * src/moe.rs:527-545). */
int rbmoe_parameter_counts(const rbmoe_config* cfg, uint64_t* total, uint64_t* active);

/* Opens device `device` with a memory budget in MiB (0 = unlimited): the role of
 * `CudaDevice::open` + `GpuContext` (src/param.rs:86-190,
 * src/gpu_transformer.rs:45-76).  Fails closed with RBMOE_BACKEND_UNAVAILABLE
 * when no GPU can be used. */
int rbmoe_ctx_create(int32_t device, size_t budget_mib, rbmoe_ctx** out);
void rbmoe_ctx_destroy(rbmoe_ctx* ctx);

/* Use the caller's HIP stream (a `hipStream_t` passed as void*) instead of the
 * context's own; NULL restores the context's own stream. */
int rbmoe_ctx_set_stream(rbmoe_ctx* ctx, void* hip_stream);

/* GpuContext::synchronize (src/gpu_transformer.rs:179-187). */
int rbmoe_synchronize(rbmoe_ctx* ctx);

/* Message of the last failure on this context (owned by the context). */
const char* rbmoe_last_error(const rbmoe_ctx* ctx);
/* Message of the last failure of a call that had no context to attach it to
 * (thread-local). */
const char* rbmoe_last_global_error(void);

/* MoeLayer::new (src/moe.rs:215-231) + TransformerLm::to_cuda's upload of the
 * layer (src/transformer.rs:1263-1296): validates, checks the budget BEFORE
 * allocating (src/param.rs:172-189), allocates weights (zeroed) and workspace. */
int rbmoe_layer_create(rbmoe_ctx* ctx, const rbmoe_config* cfg, rbmoe_layer** out);
void rbmoe_layer_destroy(rbmoe_layer* layer);

/* Behaviour switches of a layer, the counterpart of the reference's test hooks and environment switches
 * (CHUNK_ROWS_OVERRIDE src/gpu_model.rs:2948, cuda_flash::DISABLED src/cuda_flash.rs:898-907): every default is
 * the fast path, the other settings exist for A/B measurements and for tests that hold one kernel set against
 * another.  The library itself reads no environment variable. */
typedef enum rbmoe_option {
    RBMOE_OPT_FORCE_GENERIC = 0,   /* 1: the any-shape kernels for every product; only before the first weight is set */
    RBMOE_OPT_EXPLICIT_GATHER = 1, /* 1: gathered rows are written out instead of gathered inside the gate/up product */
    RBMOE_OPT_GROUP_M = 2,         /* row tiles that walk the column tiles together on one XCD; 0: each product's default */
    RBMOE_OPT_DECODE_PATH = 3,     /* 0: a few tokens take the large-batch kernels too */
    RBMOE_OPT_DECODE_FRONT = 4,    /* 0: decode-shaped calls route in a launch of their own */
    RBMOE_OPT_FUSED_ROUTER = 5,    /* 0: router logits and the routing behind them in separate launches */
    RBMOE_OPT_SIDE_STREAM = 6,     /* 0: everything on the context's one stream */
    RBMOE_OPT_WGRAD_MODE = 7,      /* cut experts' weight gradients: 0 fixed order (default), 1 f32 atomics, 2 never cut */
    RBMOE_OPT_WGRAD_GENERIC = 8,   /* 1: the plain kernel for the weight gradients */
    RBMOE_OPT_DECODE_COMBINE_FOLD = 9, /* 0: decode-shaped calls combine in a launch of their own */
    /* (not switches of a kernel choice, but of what rbmoe_set_weight does with f32 data) */
    RBMOE_OPT_QUANT_RULE = 10,     /* f32 -> int8 per row, scale = absmax / 127: 0 q = round(w / scale), the checkpoint
                                      writer's rule (src/transformer.rs:512-519); 1 q = round(w * (1 / scale)), the
                                      in-memory rule of Quantized::from_matrix (src/quantized.rs:29-51) */
    RBMOE_OPT_QUANTIZE_ROUTER = 11,/* 1: an f32 router is quantized at upload as well, as TransformerLm::quantize does
                                      (src/transformer.rs:899-910 via src/moe.rs:491-500), and the layer routes with the
                                      quantized product (sum x * q in 32 lanes) * scale (src/quantized.rs:55-62, :154-177) */
    RBMOE_OPT_DECODE_DOWN_BY_EXPERT = 12 /* (a kernel choice again) 0: the down launch of a decode-shaped call always
                                      finds its experts through the tile table, also behind RBMOE_OPT_DECODE_FRONT */
} rbmoe_option;
int rbmoe_layer_set_option(rbmoe_layer* layer, int32_t option, int32_t value);

/* DeviceParam::new (src/gpu_transformer.rs:471-490): copies one weight matrix
 * from HOST memory to the device (the caller keeps its buffer).  `dtype` is the
 * dtype of `data`; f32 data is converted to the layer's weight dtype (bf16 by
 * RNE; int8 by the checkpoint rule scale = absmax/127, q = round(w/scale),
 * src/transformer.rs:512-519, or the in-memory rule with RBMOE_OPT_QUANT_RULE).  For
 * RBMOE_I8 data, `scales` holds one f32 per row.  `expert` is ignored for the router and
 * the shared expert.  The router is kept in f32 whatever the experts' dtype, unless it is given
 * as RBMOE_I8 data or RBMOE_OPT_QUANTIZE_ROUTER is set: the layer then routes with the
 * quantized product of src/quantized.rs:55-62 (inference only). */
int rbmoe_set_weight(rbmoe_layer* layer, int32_t which, int32_t expert, const void* data,
                     int32_t dtype, const float* scales, int32_t rows, int32_t cols);

/* MoeLayer::forward_train (src/moe.rs:243-341) on DEVICE pointers, enqueued on
 * the context's stream; returns without synchronising.
 *   x        [T, cols] act_dtype; cols must equal d_model (else InvalidInput)
 *   valid    [T] bytes, 0 = padding row (Layout.valid, src/batch.rs:224-269), or NULL
 *   router_bias [E] f32 added to the logits, or NULL (the reference router is
 *            bias-free; this is a benchmark hook for skewed loads)
 *   residual [T, d] act_dtype added to the result (the block's residual add,
 *            src/transformer_block.rs:221-222), or NULL
 *   out      [T, d] act_dtype
 * Auxiliary losses and routing tables stay on the device until fetched. */
int rbmoe_forward(rbmoe_layer* layer, const void* x, int32_t T, int32_t cols, const uint8_t* valid,
                  const float* router_bias, const void* residual, void* out);

/* rbmoe_forward for callers that cannot allocate device memory and want no allocation made on their behalf
 * either: code under HIP graph capture, tight serving loops, harnesses that forbid hipMalloc.  It has no
 * counterpart in the reference.  Same arguments and same results as rbmoe_forward (bit for bit: the same
 * kernels run), but every intermediate buffer of the call (probabilities, routing tables, tile table, losses,
 * hidden and expert output rows) lies in a static device array of RBMOE_STATIC_SCRATCH_BYTES that is part of
 * the library's code object, instead of in the workspace that rbmoe_layer_create allocated.  The call makes
 * no hipMalloc, hipFree or other allocating call.
 * Limits: decode-shaped calls only, i.e. 1 to 32 tokens with tokens * num_experts <= 2048 on a layer with bf16
 * or int8 weights whose widths are multiples of 64 (bf16 rows, or f32 rows whose bf16 copy then lies in the
 * array as well), not in training mode; and the buffers of the call (about tokens * experts_per_token *
 * (d_ff + d_model) * 2 bytes, plus the shared expert's rows and the tables) must fit the array.  Anything else is RBMOE_UNSUPPORTED with a message that says which limit was hit.
 * Every call on one GPU, from any layer or context, uses that GPU's one array: calls that overlap in time on
 * one GPU race, and rbmoe_get_losses / rbmoe_get_routing / rbmoe_get_expert_rows after this call read the array,
 * so they describe this call only until the next static call on the same GPU. */
#define RBMOE_STATIC_SCRATCH_BYTES (8u << 20)
int rbmoe_forward_static(rbmoe_layer* layer, const void* x, int32_t T, int32_t cols, const uint8_t* valid,
                         const float* router_bias, const void* residual, void* out);

/* Same on HOST pointers: copies in, runs, synchronises, copies out. */
int rbmoe_forward_host(rbmoe_layer* layer, const void* x, int32_t T, int32_t cols,
                       const uint8_t* valid, const float* router_bias, const void* residual,
                       void* out);

/* MoeCache::aux_loss / z_loss (src/moe.rs:158-172) of the last forward.
 * Synchronises the stream. */
int rbmoe_get_losses(rbmoe_layer* layer, float* aux_loss, float* z_loss);

/* Routing tables of the last forward into host buffers.  Synchronises. */
int rbmoe_get_routing(rbmoe_layer* layer, rbmoe_routing* routing);

/* Expert hidden rows H [offsets[E], F] and expert output rows Y [offsets[E], d]
 * of the last forward, in permuted order, converted to f32, into host buffers
 * (either may be NULL) — the reference keeps both in MoeCache
 * (src/moe.rs:150-152, src/ffn.rs:27-33).  Synchronises. */
int rbmoe_get_expert_rows(rbmoe_layer* layer, float* hidden, float* expert_out);

/* ---- the block's steps either side of the layer ------------------------------------------
 * TransformerBlock::forward_train's feed-forward half (src/transformer_block.rs:216-222):
 *   normed = feed_forward_norm.forward(residual)   RmsNorm::forward, src/norm.rs:41-61
 *   output = moe.forward_train(normed) + residual  add_in_place, src/transformer_block.rs:310-323
 * rbmoe_set_feed_forward_norm uploads the norm's weight [d_model] (f32, host) and eps
 * (TransformerConfig::rmsnorm_eps, src/transformer.rs:42); the first call allocates the normed rows. */
int rbmoe_set_feed_forward_norm(rbmoe_layer* layer, const float* weight, int32_t cols, float eps);
/* out = x + layer(rmsnorm(x)) on DEVICE pointers ([T, d] act_dtype; `out` may be `x` itself).  The norm
 * runs as a prologue kernel with the reference's sequential sum of squares, so routing is decided on the
 * same normed rows as on the CPU; the residual add is part of the combine kernel.  Routing, losses and
 * the backward pass's state refer to the NORMED rows (rbmoe_backward then returns the gradient with
 * respect to them).  Other arguments as rbmoe_forward. */
int rbmoe_forward_block(rbmoe_layer* layer, const void* x, int32_t tokens, int32_t cols, const uint8_t* valid,
                        const float* router_bias, void* out);
/* Same on HOST pointers; synchronises. */
int rbmoe_forward_block_host(rbmoe_layer* layer, const void* x, int32_t tokens, int32_t cols,
                             const uint8_t* valid, const float* router_bias, void* out);

/* ---- backward pass (MoeLayer::backward, src/moe.rs:348-489) ------------------------------
 * Training mode makes the forward keep what MoeCache keeps for the backward pass (the input,
 * src/moe.rs:133-135; gate and up pre-activations, src/ffn.rs:27-33) and allocates f32 gradient
 * accumulators, the role of Param.grad (src/param.rs).  For every f32 / bf16 layer: bf16 layers with
 * widths that are multiples of 64 and all-f32 layers (multiples of 32) differentiate on the matrix
 * cores, any other shape or dtype mix on plain kernels; int8 layers report RBMOE_UNSUPPORTED, as the
 * reference has no backward for quantized experts (src/ffn.rs:87-93).
 * Call it before the weights are set.  A training layer always takes the large-batch kernels. */
int rbmoe_layer_enable_training(rbmoe_layer* layer);

/* MoeLayer::backward on DEVICE pointers for the last forward: `grad_output` [tokens, cols] act_dtype in,
 * `grad_input` [tokens, cols] act_dtype out; weight gradients are ACCUMULATED (as Param.grad is) until
 * rbmoe_zero_grads.  The gradients of the two auxiliary losses reach the router here, as in the
 * reference (src/moe.rs:343-347).  `tokens` and `cols` are the shape of both buffers and must be the
 * last forward's (the reference sizes the gradient from the cached input, src/moe.rs:349-350):
 * anything else is RBMOE_INVALID_INPUT and neither buffer is touched.  Enqueued on the context's stream. */
int rbmoe_backward(rbmoe_layer* layer, const void* grad_output, int32_t tokens, int32_t cols, void* grad_input);
/* Same on HOST pointers; synchronises. */
int rbmoe_backward_host(rbmoe_layer* layer, const void* grad_output, int32_t tokens, int32_t cols,
                        void* grad_input);
/* Param::zero_grad for every weight of the layer. */
int rbmoe_zero_grads(rbmoe_layer* layer);
/* One accumulated weight gradient as f32 [rows, cols] into host memory (same ids and shapes as
 * rbmoe_set_weight).  Synchronises. */
int rbmoe_get_weight_grad(rbmoe_layer* layer, int32_t which, int32_t expert, float* host, int32_t rows,
                          int32_t cols);

/* The feed-forward half of TransformerBlock::backward (src/transformer_block.rs:257-263) after
 * rbmoe_forward_block, on DEVICE pointers:
 *   grad_projected = moe.backward(cache, grad_output)
 *   grad_input     = feed_forward_norm.backward(residual, grad_projected) + grad_output
 * (RmsNorm::backward, src/norm.rs:63-121).  The norm's scale gradient accumulates like the other weight
 * gradients and is read with rbmoe_get_weight_grad(layer, RBMOE_W_NORM, 0, host, 1, d_model).  `grad_input`
 * may be `grad_output` itself.  Needs training mode and a norm (in either order).  `tokens` and `cols` as
 * for rbmoe_backward. */
int rbmoe_backward_block(rbmoe_layer* layer, const void* grad_output, int32_t tokens, int32_t cols,
                         void* grad_input);
/* Same on HOST pointers; synchronises. */
int rbmoe_backward_block_host(rbmoe_layer* layer, const void* grad_output, int32_t tokens, int32_t cols,
                              void* grad_input);

/* Per-stage timing of one forward with HIP events on the context's stream.
 * `ms` receives RBMOE_NUM_STAGES durations in milliseconds.  Synchronises.
 * Stage 1 brackets no work at all: it reads what one pair of event records adds to
 * every other stage (about 5 us), so callers can subtract it. */
#define RBMOE_NUM_STAGES 8
enum {
    RBMOE_STAGE_ROUTER = 0,   /* logits, softmax, top-k, block histograms       */
    RBMOE_STAGE_EMPTY = 1,    /* nothing: the cost of one event interval        */
    RBMOE_STAGE_DISPATCH = 2, /* layout scan, losses, permutation (+ row gather) */
    RBMOE_STAGE_GATE_UP = 3,  /* grouped gate/up product + SwiGLU               */
    RBMOE_STAGE_DOWN = 4,     /* grouped down product                           */
    RBMOE_STAGE_SHARED = 5,   /* shared expert (both products)                  */
    RBMOE_STAGE_COMBINE = 6,  /* gate-weighted combine (+ shared, + residual)   */
    RBMOE_STAGE_TOTAL = 7
};
int rbmoe_forward_timed(rbmoe_layer* layer, const void* x, int32_t T, int32_t cols,
                        const uint8_t* valid, const float* router_bias, const void* residual,
                        void* out, float* ms);

/* Kernel durations of one forward the way a kernel trace reports them: every launch of the forward carries its own
 * start and stop events, which receive the begin and end time stamps of that dispatch itself (no launch gap, no
 * event-pair overhead, no events between the stages).  `ms` receives RBMOE_NUM_STAGES values in milliseconds: per
 * stage the sum over its launches (RBMOE_STAGE_EMPTY: 0), RBMOE_STAGE_TOTAL: their sum - the time the device spent
 * inside kernels, which is less than the forward took by the gaps between the launches.  Synchronises.  Like
 * rbmoe_forward_timed, the call runs the shared expert on the main stream. */
int rbmoe_forward_kernel_times(rbmoe_layer* layer, const void* x, int32_t T, int32_t cols,
                               const uint8_t* valid, const float* router_bias, const void* residual,
                               void* out, float* ms);

/* Launch time of one stage by itself: enqueues the launches of stage `stage` (RBMOE_STAGE_ROUTER, _DISPATCH,
 * _GATE_UP, _DOWN or _COMBINE) of the LAST forward again, on the same buffers, once untimed and then `launches`
 * times back to back between ONE pair of events, and returns the average in milliseconds.  Synchronises.  The
 * stages read their inputs and overwrite their outputs with the same values, so the layer's state is unchanged.
 * A figure taken this way contains no event-pair overhead (one pair over many launches) and cannot fall below
 * what a kernel trace shows for the launch; the operands a stage shares with its neighbours in a forward may sit
 * in other cache levels here.  With ms_per_launch == NULL the launches are only enqueued (no warm-up, no events, no
 * synchronisation): for a caller that times a sequence of its own, e.g. the same stage of several layers in
 * rotation.  RBMOE_UNSUPPORTED when the last forward had no launch of its own for the stage. */
int rbmoe_replay_stage(rbmoe_layer* layer, int32_t stage, int32_t launches, float* ms_per_launch);

/* Name of the kernel variant the last forward used for the expert products
 * ("mfma_bf16", "generic", ...), for reports.  Static storage. */
const char* rbmoe_expert_kernel_name(const rbmoe_layer* layer);

/* Device memory helpers for hosts without their own HIP binding. */
int rbmoe_device_alloc(rbmoe_ctx* ctx, size_t bytes, void** out);
int rbmoe_device_free(rbmoe_ctx* ctx, void* ptr);
int rbmoe_copy_to_device(rbmoe_ctx* ctx, void* dst, const void* src, size_t bytes);
int rbmoe_copy_to_host(rbmoe_ctx* ctx, void* dst, const void* src, size_t bytes);
/* Device-to-device copy on the context's stream, then synchronise (also serves as the
 * plain copy of known size that hardware-counter readings are calibrated against). */
int rbmoe_copy_device(rbmoe_ctx* ctx, void* dst, const void* src, size_t bytes);


const char* rbmoe_version(void);

#ifdef __cplusplus
}
#endif
#endif /* RBMOE_H */
