// C ABI of the gfx950 mixture-of-experts layer (see include/rbmoe.h).
//
// Host-side orchestration only: configuration checks, weight upload and
// conversion, workspace, and the launch sequence of one forward pass
//   router -> scan -> dispatch -> gate/up (+SwiGLU) -> down -> shared -> combine
// which follows MoeLayer::forward_train (reference src/moe.rs:243-341) stage by
// stage without any host round trip between the stages.  There is no CPU
// fallback: without a usable GPU every device entry point fails.
#include "../../include/rbmoe.h"

#include <cmath>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <functional>
#include <mutex>
#include <string>
#include <vector>

#include "rbmoe_kernels.h"

using namespace rbmoe;

thread_local rbmoe::KernelTimer* rbmoe::g_kernel_timer = nullptr;

// Scratch of rbmoe_forward_static: device memory that exists without any allocation call.  Every GPU the library
// runs on holds its own copy of the array, at its own address, until the process ends.  In host code the
// array's name is only a handle for hipGetSymbolAddress: rbmoe_ctx_create resolves it once per device and host
// code uses the resolved pointer from then on.
// (No `used` attribute: the compiler makes a static device variable visible to the runtime's lookup by name
// because host code takes its address below, and only then; marked `used` it stays a local symbol, which
// hipGetSymbolAddress cannot find.)
static __device__ __align__(256) unsigned char rbmoe_static_scratch[RBMOE_STATIC_SCRATCH_BYTES];

namespace {

constexpr int kMaxDevices = 64;
std::mutex g_scratch_mutex;
void* g_scratch_ptr[kMaxDevices] = {};  // per device: the address of rbmoe_static_scratch there

// With `device` current.  Resolved once per device and kept.
hipError_t static_scratch_of(int device, void** out) {
    *out = nullptr;
    if (device < 0 || device >= kMaxDevices) return hipErrorInvalidDevice;
    std::lock_guard<std::mutex> lock(g_scratch_mutex);
    if (!g_scratch_ptr[device]) {
        void* p = nullptr;
        const hipError_t e = hipGetSymbolAddress(&p, HIP_SYMBOL(rbmoe_static_scratch));
        if (e != hipSuccess) return e;
        g_scratch_ptr[device] = p;
    }
    *out = g_scratch_ptr[device];
    return hipSuccess;
}

thread_local std::string g_global_error;

size_t dtype_size(int dt) { return dt == RBMOE_F32 ? 4 : dt == RBMOE_BF16 ? 2 : 1; }

uint16_t host_f32_to_bf16(float f) {
    uint32_t b;
    std::memcpy(&b, &f, 4);
    if ((b & 0x7fffffffu) > 0x7f800000u) return (uint16_t)((b >> 16) | 0x0040u);
    b += 0x7fffu + ((b >> 16) & 1u);
    return (uint16_t)(b >> 16);
}
float host_bf16_to_f32(uint16_t h) {
    uint32_t b = (uint32_t)h << 16;
    float f;
    std::memcpy(&f, &b, 4);
    return f;
}

std::string config_problem(const rbmoe_config* c) {
    char buf[256];
    // The first three are MoeConfig::validate (reference src/moe.rs:68-86), same wording.
    if (c->num_experts <= 0) return "a MoE layer needs at least one expert";
    if (c->experts_per_token <= 0 || c->experts_per_token > c->num_experts) {
        std::snprintf(buf, sizeof buf, "experts_per_token must be between 1 and num_experts (%d), got %d",
                      c->num_experts, c->experts_per_token);
        return buf;
    }
    if (c->d_ff <= 0) return "expert d_ff must be non-zero";
    if (c->d_model <= 0) return "d_model must be non-zero";
    if (c->shared_d_ff < 0) return "shared_d_ff must not be negative";
    if (c->weight_dtype != RBMOE_F32 && c->weight_dtype != RBMOE_BF16 && c->weight_dtype != RBMOE_I8)
        return "weight_dtype must be f32, bf16 or int8";
    if (c->act_dtype != RBMOE_F32 && c->act_dtype != RBMOE_BF16) return "act_dtype must be f32 or bf16";
    if (c->max_tokens < 0) return "max_tokens must not be negative";
    return "";
}

std::string limit_problem(const rbmoe_config* c) {
    char buf[256];
    if (c->num_experts > kMaxExperts) {
        std::snprintf(buf, sizeof buf, "more than %d experts (got %d)", kMaxExperts, c->num_experts);
        return buf;
    }
    if (c->experts_per_token > kMaxTopK) {
        std::snprintf(buf, sizeof buf, "experts_per_token above %d (got %d)", kMaxTopK, c->experts_per_token);
        return buf;
    }
    if ((int64_t)c->max_tokens * c->experts_per_token > (int64_t)1 << 28) return "max_tokens * experts_per_token above 2^28";
    return "";
}

}  // namespace

struct rbmoe_ctx {
    int device = 0;
    hipStream_t own_stream = nullptr;
    hipStream_t stream = nullptr;
    // The backward pass runs the router's branch beside the weight gradients: a second stream (default
    // priority, like the first) forked from and joined to `stream` with two events.  Created on first use.
    hipStream_t side_stream = nullptr;
    hipEvent_t ev_fork = nullptr, ev_fork2 = nullptr, ev_join = nullptr, ev_tables = nullptr;
    size_t budget_bytes = 0;
    size_t allocated = 0;
    void* static_scratch = nullptr;  // this device's copy of rbmoe_static_scratch (RBMOE_STATIC_SCRATCH_BYTES)
    std::string last_error;
    int refs = 1;  // the caller's handle + one per live layer; torn down when the last one goes
};

namespace {

struct Buf {
    void* p = nullptr;
    size_t bytes = 0;
};

int fail(rbmoe_ctx* ctx, int code, const std::string& msg) {
    if (ctx) ctx->last_error = msg;
    g_global_error = msg;
    return code;
}

int hip_fail(rbmoe_ctx* ctx, hipError_t e, const char* what) {
    std::string msg = std::string(what) + ": " + hipGetErrorString(e);
    if (e == hipErrorOutOfMemory) return fail(ctx, RBMOE_OUT_OF_MEMORY, msg);
    return fail(ctx, RBMOE_DEVICE_ERROR, msg);
}

#define HIP_TRY(ctx, expr)                                         \
    do {                                                           \
        hipError_t _e = (expr);                                    \
        if (_e != hipSuccess) return hip_fail((ctx), _e, #expr);   \
    } while (0)

}  // namespace

// Where one forward pass keeps its routing tables and expert rows: the layer's own workspace, or a carving of
// the static scratch array (rbmoe_forward_static).  The getters read the last forward's.
struct Work {
    float* P = nullptr;
    float* lse = nullptr;
    int* expert_of = nullptr;
    float* gate_of = nullptr;
    int* counts = nullptr;
    int* offsets = nullptr;
    int* tile_expert = nullptr;
    int* tile_row0 = nullptr;
    int* tile_rows = nullptr;
    int* ntiles = nullptr;
    float* losses = nullptr;
    int* perm_slot = nullptr;
    int* perm_token = nullptr;
    int* inv_pos = nullptr;
    void* h = nullptr;
    void* y = nullptr;
    void* hs = nullptr;
    void* ys = nullptr;
    void* hall = nullptr;  // hidden rows of every expert over every row, [E][T, F] (decode_front launches), or null
    void* x16 = nullptr;   // bf16 copy of f32 rows [T, d] (layers with cast_rows), or null
    int* cmb_counter = nullptr;  // arrival counters of a combine folded into the decode-shaped down launch (all zero between launches)
    unsigned int* expert_tokens = nullptr;  // [E] the tokens of every expert, one bit a token (decode_front launches), or null
};

struct rbmoe_layer {
    rbmoe_ctx* ctx = nullptr;
    rbmoe_config cfg{};
    int Fs = 0;       // shared expert width
    int max_T = 0;
    int max_S = 0;
    int max_nb = 0;
    int max_tiles = 0;
    bool force_generic = false;
    bool explicit_gather = false;  // materialise the gathered rows instead of gathering in the product
    bool use_stream = false;   // bf16 matrix-core kernels (packed weights); otherwise the generic kernels
    // f32 rows on the boundary of a layer with bf16 / int8 weights: the router reads the f32 rows, the expert
    // products run on the bf16 matrix cores over a bf16 copy of the rows (nearest even) that the routing kernels
    // write on the way, hidden and expert rows are bf16, and the combine sums them into f32 again
    bool cast_rows = false;
    bool use_f32_mc = false;   // all-f32 layer on the f32 matrix cores
    bool decode_path = true;   // few tokens: four launches that stream every touched weight once
    bool decode_front = true;  // ... three, with the routing beside the gate/up products, when most experts are touched
    bool shared_beside = true; // large batches: the shared expert's products on the side stream, beside the routing
    bool fused_router = true;  // logits and everything behind them in one launch where the shapes allow
    bool decode_fold = true;   // decode-shaped calls: the combine inside the down launch
    bool decode_down_by_expert = true;  // behind a decode_front launch: the down launch's workgroup rows are experts, not tile-table entries
    bool last_front = false;   // the last forward's hidden rows are per expert over all rows (Work::hall)
    int group_m = 0;
    const char* kernel_name = "none";
    int last_T = -1;
    int last_tile_m = kGenericTileM;  // rows per tile of the last forward's tile table
    Work last;  // tables of the last forward

    // weights
    Buf router;            // f32 [E, d]
    Buf router_q, router_s; // a quantized router: int8 [E, d], f32 scales [E]
    bool router_q8 = false; // the layer routes with the quantized product (src/quantized.rs:55-62)
    bool quantize_router = false;  // f32 router data is quantized at upload (TransformerLm::quantize reaches the router too)
    int quant_rule = 0;     // f32 -> int8 at upload: 0 the checkpoint writer's rule, 1 the in-memory rule
    Buf wgu, wd;           // [E, 2F, d], [E, d, F] weight dtype
    Buf sgu, sd;           // int8 scales [E, 2F], [E, d]
    Buf swgu, swd;         // shared [2Fs, d], [d, Fs]
    Buf ssgu, ssd;         // shared scales
    // workspace
    Buf P, lse, expert_of, gate_of, rank_in_block, blockcnt, partial, blockbase;
    Buf counts, offsets, tile_expert, tile_row0, tile_rows, ntiles, losses;
    Buf perm_slot, perm_token, inv_pos;
    Buf xg, h, y, hs, ys;
    Buf x16;               // [max_T, d] bf16 copy of f32 rows (cast_rows)
    Buf hall;              // [E][min(max_T, 32), F] hidden rows of decode_front launches
    Buf etok;              // [E] token bits of every expert (decode_front launches)
    Buf cmbcnt;            // [kDecodeCombineMaxBlocks] arrival counters of the folded decode combine
    // feed-forward norm in front of the layer (allocated by rbmoe_set_feed_forward_norm)
    Buf xn, norm_w;  // [max_T, d] activation dtype, [d] f32
    float norm_eps = 0.0f;
    bool norm_set = false;
    // training through the block step (allocated once both the norm and training mode are there)
    Buf xraw, dxn, inv_rms, norm_partial, g_norm;  // [T, d] x2 activation dtype, [T], [T/32][d], [d] f32
    bool last_was_block = false;
    // training (allocated by rbmoe_layer_enable_training)
    bool training = false;
    bool weights_set = false;
    Buf xc;                               // copy of the last input [T, d]
    Buf gu, gus;                          // pre-activations (gate | up): [S, 2F], shared [T, 2Fs]
    Buf dy, dgu, dxg;                     // [S, d], [S, 2F], [S, d]
    Buf g16;                              // [T, d] bf16 copy of an f32 upstream gradient (cast_rows)
    Buf dgus, dxs;                        // shared: [T, 2Fs], [T, d]
    Buf grad_gates, ones, dlogits, dxr, rpartial;
    Buf g_router, g_gu, g_down, g_sgu, g_sdown;   // f32 weight gradients, accumulated
    Buf wg_chunks;                        // chunk table of the weight-gradient products
    Buf wg_partial;                       // partial matrices of cut experts (ordered accumulation)
    bool wgrad_generic = false, side_branch = true;
    WgradSplit wgrad_split = WgradSplit::Ordered;
    // The expert gradients count as zero without having been cleared (set by rbmoe_zero_grads): the next
    // backward pass overwrites them.
    bool grads_clear = false;
    Buf wdT, wguT, swdT, swguT;           // transposed packed weights: [E][F, d], [E][d, 2F], [Fs, d], [d, 2Fs]
    Buf st_gout, st_gin;
    // staging for the host entry point
    Buf st_x, st_out, st_valid, st_bias, st_res;
    std::vector<Buf*> all;
    hipEvent_t ev[RBMOE_NUM_STAGES + 1] = {};
    bool have_events = false;
    KernelTimer ktimer[RBMOE_NUM_STAGES];  // rbmoe_forward_kernel_times: events carried by the stages' own dispatches
    bool have_ktimers = false;
    // the launches of the last forward, stage by stage, for rbmoe_replay_stage (empty: the stage had no launch)
    std::function<hipError_t(hipStream_t)> replay[RBMOE_NUM_STAGES];
};

namespace {

struct Plan {
    std::vector<std::pair<Buf*, size_t>> items;
    size_t total = 0;
    void add(Buf* b, size_t bytes) {
        bytes = (bytes + 255) & ~(size_t)255;
        if (bytes == 0) bytes = 256;
        items.push_back({b, bytes});
        total += bytes;
    }
};

// Which kernel sets the layer's shapes and dtypes allow (and `force_generic` does not rule out).
void choose_kernel_sets(rbmoe_layer* L) {
    const rbmoe_config* cfg = &L->cfg;
    L->use_stream = L->use_f32_mc = L->cast_rows = false;
    // bf16 matrix cores: bf16 activations, bf16 or int8 weights, widths that fit the packed layout
    // (f32 rows with bf16 / int8 weights - what a caller with f32 matrices and a quantized or bf16 checkpoint has -
    // take the same kernels over a bf16 copy of the rows)
    const bool mc = !L->force_generic && cfg->weight_dtype != RBMOE_F32;
    L->use_stream = mc && stream_shape_ok(cfg->d_ff, cfg->d_model) && stream_shape_ok(cfg->d_model, cfg->d_ff) &&
                    (!cfg->shared_expert ||
                     (stream_shape_ok(L->Fs, cfg->d_model) && stream_shape_ok(cfg->d_model, L->Fs)));

    L->use_f32_mc = !L->force_generic && cfg->act_dtype == RBMOE_F32 && cfg->weight_dtype == RBMOE_F32 &&
                    f32_shape_ok(cfg->d_ff, cfg->d_model) && f32_shape_ok(cfg->d_model, cfg->d_ff) &&
                    (!cfg->shared_expert || (f32_shape_ok(L->Fs, cfg->d_model) && f32_shape_ok(cfg->d_model, L->Fs)));
    {
        // the streaming kernel addresses activation rows with 32-bit byte offsets
        const size_t widest = (size_t)std::max(std::max(cfg->d_model, cfg->d_ff), L->Fs);
        const size_t rows = (size_t)cfg->max_tokens * (size_t)std::max(1, cfg->experts_per_token);
        if (rows * widest * 2 >= ((size_t)1 << 32)) L->use_stream = false;
    }
    if (cfg->act_dtype == RBMOE_F32 && L->use_stream) {
        // the bf16 copy is written in 8-element pieces of 16-byte aligned rows
        if (cfg->d_model % 8 == 0) L->cast_rows = true;
        else L->use_stream = false;
    }
}

Plan make_plan(rbmoe_layer* L) {
    const rbmoe_config& c = L->cfg;
    const size_t E = c.num_experts, d = c.d_model, F = c.d_ff, k = c.experts_per_token;
    const size_t Fs = L->Fs, T = L->max_T, S = L->max_S, nb = L->max_nb;
    const size_t ws = dtype_size(c.weight_dtype), as = dtype_size(c.act_dtype);
    Plan p;
    p.add(&L->router, E * d * 4);
    p.add(&L->router_q, E * d);
    p.add(&L->router_s, E * 4);
    p.add(&L->wgu, E * 2 * F * d * ws);
    p.add(&L->wd, E * d * F * ws);
    if (c.weight_dtype == RBMOE_I8) {
        p.add(&L->sgu, E * 2 * F * 4);
        p.add(&L->sd, E * d * 4);
    }
    if (c.shared_expert) {
        p.add(&L->swgu, 2 * Fs * d * ws);
        p.add(&L->swd, d * Fs * ws);
        if (c.weight_dtype == RBMOE_I8) {
            p.add(&L->ssgu, 2 * Fs * 4);
            p.add(&L->ssd, d * 4);
        }
        p.add(&L->hs, T * Fs * as);
        p.add(&L->ys, T * d * as);
    }
    p.add(&L->P, T * E * 4);
    p.add(&L->lse, T * 4);
    p.add(&L->expert_of, S * 4);
    p.add(&L->gate_of, S * 4);
    p.add(&L->rank_in_block, S * 4);
    p.add(&L->blockcnt, nb * E * 4);
    p.add(&L->partial, nb * (E + 1) * 4);
    p.add(&L->blockbase, nb * E * 4);
    p.add(&L->counts, E * 4);
    p.add(&L->offsets, (E + 1) * 4);
    p.add(&L->tile_expert, (size_t)L->max_tiles * 4);
    p.add(&L->tile_row0, (size_t)L->max_tiles * 4);
    p.add(&L->tile_rows, (size_t)L->max_tiles * 4);
    p.add(&L->ntiles, 8);
    p.add(&L->losses, 8);
    p.add(&L->perm_slot, S * 4);
    p.add(&L->perm_token, S * 4);
    p.add(&L->inv_pos, S * 4);
    if (L->cast_rows) p.add(&L->x16, T * d * 2);
    // decode_front launches need most experts touched (tokens * k >= 2 E, at most 32 tokens): none when E > 16 k
    if (L->use_stream && E <= 16 * k) {
        p.add(&L->hall, E * std::min<size_t>(T, kSmallRouteMaxTokens) * F * 2);
        p.add(&L->etok, E * 4);
    }
    p.add(&L->cmbcnt, kDecodeCombineCounterBytes);
    p.add(&L->xg, S * d * as);
    p.add(&L->h, S * F * as);
    p.add(&L->y, S * d * as);
    p.add(&L->st_x, T * d * as);
    p.add(&L->st_out, T * d * as);
    p.add(&L->st_res, T * d * as);
    p.add(&L->st_valid, T);
    p.add(&L->st_bias, E * 4);
    (void)k;
    return p;
}

void free_layer_buffers(rbmoe_layer* L) {
    for (Buf* b : L->all) {
        if (b->p) {
            (void)hipFree(b->p);
            if (L->ctx && L->ctx->allocated >= b->bytes) L->ctx->allocated -= b->bytes;
            b->p = nullptr;
            b->bytes = 0;
        }
    }
    L->all.clear();
}

}  // namespace

extern "C" {

const char* rbmoe_version(void) { return "rbmoe 0.1 (gfx950)"; }

const char* rbmoe_last_global_error(void) { return g_global_error.c_str(); }

int rbmoe_config_init(rbmoe_config* cfg, int32_t d_model, int32_t num_experts, int32_t experts_per_token,
                      int32_t d_ff) {
    if (!cfg) return fail(nullptr, RBMOE_NULL_POINTER, "cfg is NULL");
    std::memset(cfg, 0, sizeof *cfg);
    cfg->d_model = d_model;
    cfg->num_experts = num_experts;
    cfg->experts_per_token = experts_per_token;
    cfg->d_ff = d_ff;
    cfg->shared_expert = 0;
    cfg->shared_d_ff = 0;
    cfg->aux_loss_weight = 0.01f;
    cfg->router_z_loss_weight = 1e-3f;
    cfg->weight_dtype = RBMOE_F32;
    cfg->act_dtype = RBMOE_F32;
    cfg->max_tokens = 0;
    return RBMOE_OK;
}

int rbmoe_validate(const rbmoe_config* cfg, char* msg, size_t msg_cap) {
    if (!cfg) return fail(nullptr, RBMOE_NULL_POINTER, "cfg is NULL");
    std::string problem = config_problem(cfg);
    int code = RBMOE_INVALID_CONFIG;
    if (problem.empty()) {
        problem = limit_problem(cfg);
        code = RBMOE_UNSUPPORTED;
    }
    if (msg && msg_cap > 0) {
        std::snprintf(msg, msg_cap, "%s", problem.c_str());
    }
    if (problem.empty()) return RBMOE_OK;
    return fail(nullptr, code, problem);
}

int rbmoe_parameter_counts(const rbmoe_config* cfg, uint64_t* total, uint64_t* active) {
    if (!cfg) return fail(nullptr, RBMOE_NULL_POINTER, "cfg is NULL");
    const uint64_t d = cfg->d_model, E = cfg->num_experts, k = cfg->experts_per_token, F = cfg->d_ff;
    const uint64_t Fs = cfg->shared_d_ff > 0 ? cfg->shared_d_ff : cfg->d_ff;
    const uint64_t expert = 3 * d * F;
    const uint64_t shared = cfg->shared_expert ? 3 * d * Fs : 0;
    const uint64_t router = E * d;
    if (total) *total = router + E * expert + shared;
    if (active) *active = router + k * expert + shared;
    return RBMOE_OK;
}

int rbmoe_ctx_create(int32_t device, size_t budget_mib, rbmoe_ctx** out) {
    if (!out) return fail(nullptr, RBMOE_NULL_POINTER, "out is NULL");
    *out = nullptr;
    int n = 0;
    hipError_t e = hipGetDeviceCount(&n);
    if (e != hipSuccess || n <= 0) {
        (void)hipGetLastError();
        return fail(nullptr, RBMOE_BACKEND_UNAVAILABLE,
                    std::string("no usable HIP device: ") + (e != hipSuccess ? hipGetErrorString(e) : "device count is 0"));
    }
    if (device < 0 || device >= n) return fail(nullptr, RBMOE_INVALID_CONFIG, "device index out of range");
    hipDeviceProp_t prop;
    HIP_TRY(nullptr, hipGetDeviceProperties(&prop, device));
    if (std::strncmp(prop.gcnArchName, "gfx950", 6) != 0)
        return fail(nullptr, RBMOE_UNSUPPORTED, std::string("kernels are built for gfx950, device is ") + prop.gcnArchName);
    HIP_TRY(nullptr, hipSetDevice(device));
    void* scratch = nullptr;
    HIP_TRY(nullptr, static_scratch_of(device, &scratch));
    rbmoe_ctx* ctx = new rbmoe_ctx();
    ctx->device = device;
    ctx->static_scratch = scratch;
    ctx->budget_bytes = budget_mib << 20;
    hipError_t se = hipStreamCreateWithFlags(&ctx->own_stream, hipStreamNonBlocking);
    if (se != hipSuccess) {
        delete ctx;
        return hip_fail(nullptr, se, "hipStreamCreateWithFlags");
    }
    ctx->stream = ctx->own_stream;
    *out = ctx;
    return RBMOE_OK;
}

static void ctx_release(rbmoe_ctx* ctx) {
    if (!ctx || --ctx->refs > 0) return;
    if (ctx->side_stream) {
        (void)hipStreamSynchronize(ctx->side_stream);
        (void)hipStreamDestroy(ctx->side_stream);
    }
    if (ctx->ev_fork) (void)hipEventDestroy(ctx->ev_fork);
    if (ctx->ev_fork2) (void)hipEventDestroy(ctx->ev_fork2);
    if (ctx->ev_join) (void)hipEventDestroy(ctx->ev_join);
    if (ctx->ev_tables) (void)hipEventDestroy(ctx->ev_tables);
    if (ctx->own_stream) {
        (void)hipStreamSynchronize(ctx->own_stream);
        (void)hipStreamDestroy(ctx->own_stream);
    }
    delete ctx;
}

// Layers keep their context alive: destroying the context while layers exist
// only drops the caller's reference.
void rbmoe_ctx_destroy(rbmoe_ctx* ctx) { ctx_release(ctx); }

int rbmoe_ctx_set_stream(rbmoe_ctx* ctx, void* hip_stream) {
    if (!ctx) return fail(nullptr, RBMOE_NULL_POINTER, "ctx is NULL");
    ctx->stream = hip_stream ? static_cast<hipStream_t>(hip_stream) : ctx->own_stream;
    return RBMOE_OK;
}

int rbmoe_synchronize(rbmoe_ctx* ctx) {
    if (!ctx) return fail(nullptr, RBMOE_NULL_POINTER, "ctx is NULL");
    HIP_TRY(ctx, hipStreamSynchronize(ctx->stream));
    return RBMOE_OK;
}

const char* rbmoe_last_error(const rbmoe_ctx* ctx) { return ctx ? ctx->last_error.c_str() : g_global_error.c_str(); }

int rbmoe_layer_create(rbmoe_ctx* ctx, const rbmoe_config* cfg, rbmoe_layer** out) {
    if (!ctx || !cfg || !out) return fail(ctx, RBMOE_NULL_POINTER, "ctx, cfg or out is NULL");
    *out = nullptr;
    std::string problem = config_problem(cfg);
    if (!problem.empty()) return fail(ctx, RBMOE_INVALID_CONFIG, problem);
    problem = limit_problem(cfg);
    if (!problem.empty()) return fail(ctx, RBMOE_UNSUPPORTED, problem);
    if (cfg->max_tokens <= 0) return fail(ctx, RBMOE_INVALID_CONFIG, "max_tokens must be positive");
    if (router_lds_bytes(cfg->num_experts, cfg->experts_per_token) > (size_t)kMaxRouterLds)
        return fail(ctx, RBMOE_UNSUPPORTED, "router tile does not fit in LDS for this expert count and top-k");

    rbmoe_layer* L = new rbmoe_layer();
    L->ctx = ctx;
    L->cfg = *cfg;
    L->Fs = cfg->shared_d_ff > 0 ? cfg->shared_d_ff : cfg->d_ff;
    L->cfg.shared_d_ff = L->Fs;
    L->max_T = cfg->max_tokens;
    L->max_S = cfg->max_tokens * cfg->experts_per_token;
    L->max_nb = (cfg->max_tokens + kRouterTokens - 1) / kRouterTokens;
    L->max_tiles = L->max_S / kGenericTileM + cfg->num_experts + 1;
    // (behaviour switches keep their defaults here: rbmoe_layer_set_option changes them)
    // bf16 matrix cores: bf16 activations, bf16 or int8 weights, widths that fit the packed layout
    // (f32 rows with bf16 / int8 weights - what a caller with f32 matrices and a quantized or bf16 checkpoint has -
    // take the same kernels over a bf16 copy of the rows)
    choose_kernel_sets(L);

    Plan plan = make_plan(L);
    // Refuse before allocating anything, as the reference's budget check does
    // (src/param.rs:172-189).
    if (ctx->budget_bytes && ctx->allocated + plan.total > ctx->budget_bytes) {
        char buf[200];
        std::snprintf(buf, sizeof buf, "memory budget exceeded: estimated %zu MiB exceeds budget %zu MiB",
                      (ctx->allocated + plan.total + (1 << 20) - 1) >> 20, ctx->budget_bytes >> 20);
        delete L;
        return fail(ctx, RBMOE_MEMORY_BUDGET, buf);
    }
    hipError_t e = hipSetDevice(ctx->device);
    if (e != hipSuccess) {
        delete L;
        return hip_fail(ctx, e, "hipSetDevice");
    }
    for (auto& it : plan.items) {
        void* p = nullptr;
        e = hipMalloc(&p, it.second);
        if (e != hipSuccess) {
            size_t free_b = 0, total_b = 0;
            (void)hipGetLastError();
            (void)hipMemGetInfo(&free_b, &total_b);
            char buf[200];
            std::snprintf(buf, sizeof buf, "out of memory: an allocation of %zu MiB failed with %zu MiB free",
                          it.second >> 20, free_b >> 20);
            free_layer_buffers(L);
            delete L;
            return fail(ctx, RBMOE_OUT_OF_MEMORY, buf);
        }
        it.first->p = p;
        it.first->bytes = it.second;
        ctx->allocated += it.second;
        L->all.push_back(it.first);
        e = hipMemsetAsync(p, 0, it.second, ctx->stream);
        if (e != hipSuccess) {
            free_layer_buffers(L);
            delete L;
            return hip_fail(ctx, e, "hipMemsetAsync");
        }
    }
    e = hipStreamSynchronize(ctx->stream);
    if (e != hipSuccess) {
        free_layer_buffers(L);
        delete L;
        return hip_fail(ctx, e, "hipStreamSynchronize");
    }
    ++ctx->refs;
    *out = L;
    return RBMOE_OK;
}

void rbmoe_layer_destroy(rbmoe_layer* L) {
    if (!L) return;
    rbmoe_ctx* owner = L->ctx;
    if (L->ctx) (void)hipStreamSynchronize(L->ctx->stream);
    if (L->have_events)
        for (auto& ev : L->ev)
            if (ev) (void)hipEventDestroy(ev);
    if (L->have_ktimers)
        for (auto& kt : L->ktimer)
            for (auto& ev : kt.ev)
                if (ev) (void)hipEventDestroy(ev);
    free_layer_buffers(L);
    delete L;
    ctx_release(owner);
}

int rbmoe_set_weight(rbmoe_layer* L, int32_t which, int32_t expert, const void* data, int32_t dtype,
                     const float* scales, int32_t rows, int32_t cols) {
    if (!L) return fail(nullptr, RBMOE_NULL_POINTER, "layer is NULL");
    rbmoe_ctx* ctx = L->ctx;
    if (!data) return fail(ctx, RBMOE_NULL_POINTER, "data is NULL");
    const rbmoe_config& c = L->cfg;
    const int E = c.num_experts, d = c.d_model, F = c.d_ff, Fs = L->Fs;
    int want_rows = 0, want_cols = 0;
    char* dst = nullptr;        // destination of the matrix, in weight-dtype elements
    float* sdst = nullptr;      // destination of the scales
    size_t elem_off = 0, scale_off = 0;
    bool is_router = false;
    switch (which) {
        case RBMOE_W_ROUTER:
            want_rows = E; want_cols = d; is_router = true;
            dst = static_cast<char*>(L->router.p);
            break;
        case RBMOE_W_GATE:
        case RBMOE_W_UP:
            want_rows = F; want_cols = d;
            if (expert < 0 || expert >= E) return fail(ctx, RBMOE_INVALID_CONFIG, "expert index out of range");
            elem_off = ((size_t)expert * 2 + (which == RBMOE_W_UP ? 1 : 0)) * F * d;
            scale_off = ((size_t)expert * 2 + (which == RBMOE_W_UP ? 1 : 0)) * F;
            dst = static_cast<char*>(L->wgu.p);
            sdst = static_cast<float*>(L->sgu.p);
            break;
        case RBMOE_W_DOWN:
            want_rows = d; want_cols = F;
            if (expert < 0 || expert >= E) return fail(ctx, RBMOE_INVALID_CONFIG, "expert index out of range");
            elem_off = (size_t)expert * d * F;
            scale_off = (size_t)expert * d;
            dst = static_cast<char*>(L->wd.p);
            sdst = static_cast<float*>(L->sd.p);
            break;
        case RBMOE_W_SHARED_GATE:
        case RBMOE_W_SHARED_UP:
            if (!c.shared_expert) return fail(ctx, RBMOE_INVALID_CONFIG, "the layer has no shared expert");
            want_rows = Fs; want_cols = d;
            elem_off = (size_t)(which == RBMOE_W_SHARED_UP ? 1 : 0) * Fs * d;
            scale_off = (size_t)(which == RBMOE_W_SHARED_UP ? 1 : 0) * Fs;
            dst = static_cast<char*>(L->swgu.p);
            sdst = static_cast<float*>(L->ssgu.p);
            break;
        case RBMOE_W_SHARED_DOWN:
            if (!c.shared_expert) return fail(ctx, RBMOE_INVALID_CONFIG, "the layer has no shared expert");
            want_rows = d; want_cols = Fs;
            dst = static_cast<char*>(L->swd.p);
            sdst = static_cast<float*>(L->ssd.p);
            break;
        default:
            return fail(ctx, RBMOE_INVALID_CONFIG, "unknown weight id");
    }
    if (rows != want_rows || cols != want_cols) {
        char buf[160];
        std::snprintf(buf, sizeof buf, "weight shape [%d, %d] does not match expected [%d, %d]", rows, cols,
                      want_rows, want_cols);
        return fail(ctx, RBMOE_INVALID_INPUT, buf);
    }
    const size_t n = (size_t)rows * cols;
    // The router is f32 whatever the experts' dtype - unless it is given as int8 rows with scales, or the layer
    // was told to quantize it like every other Linear (TransformerLm::quantize, src/transformer.rs:899-910, reaches
    // it through MoeLayer::linears_mut, src/moe.rs:491-500): the layer then routes with the quantized product.
    const bool router_to_i8 = is_router && (dtype == RBMOE_I8 || (L->quantize_router && dtype == RBMOE_F32));
    const int target = is_router ? (router_to_i8 ? RBMOE_I8 : RBMOE_F32) : c.weight_dtype;
    if (router_to_i8 && L->training)
        return fail(ctx, RBMOE_UNSUPPORTED, "the backward pass is not defined for a quantized router");
    HIP_TRY(ctx, hipSetDevice(ctx->device));
    HIP_TRY(ctx, hipStreamSynchronize(ctx->stream));  // no forward may still read the old weights

    std::vector<unsigned char> staged;
    std::vector<float> staged_scales;
    const void* src = data;
    if (dtype == target) {
        if (target == RBMOE_I8) {
            if (!scales) return fail(ctx, RBMOE_NULL_POINTER, "int8 weights need scales");
        }
    } else if (dtype == RBMOE_F32 && target == RBMOE_BF16) {
        staged.resize(n * 2);
        const float* f = static_cast<const float*>(data);
        uint16_t* o = reinterpret_cast<uint16_t*>(staged.data());
        for (size_t i = 0; i < n; ++i) o[i] = host_f32_to_bf16(f[i]);
        src = staged.data();
    } else if (dtype == RBMOE_BF16 && target == RBMOE_F32) {
        staged.resize(n * 4);
        const uint16_t* h = static_cast<const uint16_t*>(data);
        float* o = reinterpret_cast<float*>(staged.data());
        for (size_t i = 0; i < n; ++i) o[i] = host_bf16_to_f32(h[i]);
        src = staged.data();
    } else if (dtype == RBMOE_F32 && target == RBMOE_I8) {
        // Per row: scale = absmax / 127, then
        //   rule 0, the checkpoint writer's (reference src/transformer.rs:512-519, :1839-1847):
        //           q = clamp(round(w / scale)), a zero row stays zero;
        //   rule 1, the in-memory one of Quantized::from_matrix (src/quantized.rs:29-51), which
        //           TransformerLm::quantize applies: q = clamp(round(w * (1 / scale))).
        // `round` is f32::round: halves away from zero.  The two differ where the reciprocal's rounding moves a
        // quotient across a half.
        staged.resize(n);
        staged_scales.resize(rows);
        const float* f = static_cast<const float*>(data);
        int8_t* q = reinterpret_cast<int8_t*>(staged.data());
        for (int r = 0; r < rows; ++r) {
            float absmax = 0.0f;
            for (int cc = 0; cc < cols; ++cc) absmax = std::fmax(absmax, std::fabs(f[(size_t)r * cols + cc]));
            const float scale = absmax / 127.0f;
            staged_scales[r] = scale;
            const float inverse = scale > 0.0f ? 1.0f / scale : 0.0f;
            for (int cc = 0; cc < cols; ++cc) {
                const float w = f[(size_t)r * cols + cc];
                float v = L->quant_rule == 1 ? std::round(w * inverse) : (scale == 0.0f ? 0.0f : std::round(w / scale));
                v = std::fmin(127.0f, std::fmax(-127.0f, v));
                q[(size_t)r * cols + cc] = (int8_t)v;
            }
        }
        src = staged.data();
        scales = staged_scales.data();
    } else {
        return fail(ctx, RBMOE_UNSUPPORTED, "this conversion between weight dtypes is not supported");
    }
    if (is_router) {
        if (router_to_i8) {
            HIP_TRY(ctx, hipMemcpy(L->router_q.p, src, n, hipMemcpyHostToDevice));
            HIP_TRY(ctx, hipMemcpy(L->router_s.p, scales, (size_t)rows * 4, hipMemcpyHostToDevice));
        } else {
            HIP_TRY(ctx, hipMemcpy(L->router.p, src, n * 4, hipMemcpyHostToDevice));
        }
        L->router_q8 = router_to_i8;
        L->weights_set = true;
        return RBMOE_OK;
    }
    const size_t es = dtype_size(target);
    std::vector<unsigned char> packed;
    if (L->use_stream && !is_router) {
        // operand order of the matrix cores, matrix by matrix (same offsets, different inner layout)
        packed.resize(n * es);
        if (target == RBMOE_BF16)
            pack_weight_bf16(static_cast<const uint16_t*>(src), rows, cols, reinterpret_cast<uint16_t*>(packed.data()));
        else
            pack_weight_i8(static_cast<const int8_t*>(src), rows, cols, reinterpret_cast<int8_t*>(packed.data()));
        src = packed.data();
    }
    HIP_TRY(ctx, hipMemcpy(dst + elem_off * es, src, n * es, hipMemcpyHostToDevice));
    if (target == RBMOE_I8)
        HIP_TRY(ctx, hipMemcpy(sdst + scale_off, scales, (size_t)rows * 4, hipMemcpyHostToDevice));
    L->weights_set = true;
    if (L->training && !is_router) {
        // The backward products multiply by the weight itself, not by its transpose (grad_input =
        // grad_output . W, src/param.rs:822-823): keep a transposed copy in the layout the product kernels
        // read.  Gate and up share one matrix [d, 2F] (gate^T in columns [0, F), up^T in [F, 2F)) so that
        // dX = dG . Wg + dU . Wu is one product.
        const bool shared_w = which >= RBMOE_W_SHARED_GATE;
        const bool is_down = which == RBMOE_W_DOWN || which == RBMOE_W_SHARED_DOWN;
        const bool is_up = which == RBMOE_W_UP || which == RBMOE_W_SHARED_UP;
        const int Fw = shared_w ? Fs : F;
        if (target == RBMOE_F32) {
            // plain row-major f32, as the f32 product kernel reads its weights
            const float* f = static_cast<const float*>(src);
            std::vector<float> tr(n);
            for (int r = 0; r < rows; ++r)
                for (int cc = 0; cc < cols; ++cc) tr[(size_t)cc * rows + r] = f[(size_t)r * cols + cc];
            if (is_down) {
                float* tdst = static_cast<float*>(shared_w ? L->swdT.p : L->wdT.p) + (shared_w ? 0 : (size_t)expert * Fw * d);
                HIP_TRY(ctx, hipMemcpy(tdst, tr.data(), n * 4, hipMemcpyHostToDevice));
            } else {
                float* base = static_cast<float*>(shared_w ? L->swguT.p : L->wguT.p) +
                              (shared_w ? 0 : (size_t)expert * d * 2 * Fw) + (is_up ? Fw : 0);
                HIP_TRY(ctx, hipMemcpy2D(base, (size_t)2 * Fw * 4, tr.data(), (size_t)Fw * 4, (size_t)Fw * 4, (size_t)d,
                                         hipMemcpyHostToDevice));
            }
        } else if (!L->use_stream) {
            // plain row-major bf16, as the any-shape product kernel reads its weights
            const uint16_t* h = static_cast<const uint16_t*>(src);
            std::vector<uint16_t> tr(n);
            for (int r = 0; r < rows; ++r)
                for (int cc = 0; cc < cols; ++cc) tr[(size_t)cc * rows + r] = h[(size_t)r * cols + cc];
            if (is_down) {
                uint16_t* tdst = static_cast<uint16_t*>(shared_w ? L->swdT.p : L->wdT.p) + (shared_w ? 0 : (size_t)expert * Fw * d);
                HIP_TRY(ctx, hipMemcpy(tdst, tr.data(), n * 2, hipMemcpyHostToDevice));
            } else {
                uint16_t* base = static_cast<uint16_t*>(shared_w ? L->swguT.p : L->wguT.p) +
                                 (shared_w ? 0 : (size_t)expert * d * 2 * Fw) + (is_up ? Fw : 0);
                HIP_TRY(ctx, hipMemcpy2D(base, (size_t)2 * Fw * 2, tr.data(), (size_t)Fw * 2, (size_t)Fw * 2, (size_t)d,
                                         hipMemcpyHostToDevice));
            }
        } else {
            // packed bf16; column steps of 16 never straddle the two halves of [d, 2F]
            std::vector<uint16_t> plain(n), tr(n), trp(n);
            if (dtype == RBMOE_BF16) {
                std::memcpy(plain.data(), data, n * 2);
            } else {
                const float* f = static_cast<const float*>(data);
                for (size_t i = 0; i < n; ++i) plain[i] = host_f32_to_bf16(f[i]);
            }
            for (int r = 0; r < rows; ++r)
                for (int cc = 0; cc < cols; ++cc) tr[(size_t)cc * rows + r] = plain[(size_t)r * cols + cc];
            pack_weight_bf16(tr.data(), cols, rows, trp.data());  // [cols, rows] matrix
            if (is_down) {
                char* tdst = static_cast<char*>(shared_w ? L->swdT.p : L->wdT.p) + (shared_w ? 0 : (size_t)expert * Fw * d * 2);
                HIP_TRY(ctx, hipMemcpy(tdst, trp.data(), n * 2, hipMemcpyHostToDevice));
            } else {
                // [d, Fw] packed as [d/32][Fw/16][512]; destination [d/32][2Fw/16][512]
                char* base = static_cast<char*>(shared_w ? L->swguT.p : L->wguT.p) +
                             (shared_w ? 0 : (size_t)expert * d * 2 * Fw * 2);
                const size_t half = (size_t)(Fw / 16) * 512;  // elements per row block and half
                for (int rb = 0; rb < d / 32; ++rb)
                    HIP_TRY(ctx, hipMemcpy(base + ((size_t)rb * 2 * half + (is_up ? half : 0)) * 2,
                                           trp.data() + (size_t)rb * half, half * 2, hipMemcpyHostToDevice));
            }
        }
    }
    return RBMOE_OK;
}

}  // extern "C"

namespace {

// The second stream of a context (default priority, like the first) and the events that fork it from and join it
// to the main one: the backward pass runs the router's branch there, the forward pass the shared expert.
int ensure_side_stream(rbmoe_ctx* ctx) {
    if (ctx->side_stream) return RBMOE_OK;
    HIP_TRY(ctx, hipSetDevice(ctx->device));
    // all five or none: a stream without its events would be used as if it were complete
    hipStream_t st = nullptr;
    hipEvent_t ev[4] = {nullptr, nullptr, nullptr, nullptr};
    hipError_t e = hipStreamCreateWithFlags(&st, hipStreamNonBlocking);
    for (int i = 0; i < 4 && e == hipSuccess; ++i) e = hipEventCreateWithFlags(&ev[i], hipEventDisableTiming);
    if (e != hipSuccess) {
        for (hipEvent_t x : ev)
            if (x) (void)hipEventDestroy(x);
        if (st) (void)hipStreamDestroy(st);
        return hip_fail(ctx, e, "creating the context's second stream");
    }
    ctx->side_stream = st;
    ctx->ev_fork = ev[0];
    ctx->ev_fork2 = ev[1];
    ctx->ev_join = ev[2];
    ctx->ev_tables = ev[3];
    return RBMOE_OK;
}

// ints of one chunk table of a training layer's weight-gradient launches (the largest of them)
static size_t wgrad_table_ints(const rbmoe_layer* L) {
    const int E = L->cfg.num_experts;
    return (size_t)std::max(weight_grad_table_ints(E, L->max_S), weight_grad_table_ints(1, L->max_T));
}

Work work_of_layer(const rbmoe_layer* L) {
    Work w;
    w.P = (float*)L->P.p; w.lse = (float*)L->lse.p;
    w.expert_of = (int*)L->expert_of.p; w.gate_of = (float*)L->gate_of.p;
    w.counts = (int*)L->counts.p; w.offsets = (int*)L->offsets.p;
    w.tile_expert = (int*)L->tile_expert.p; w.tile_row0 = (int*)L->tile_row0.p; w.tile_rows = (int*)L->tile_rows.p;
    w.ntiles = (int*)L->ntiles.p; w.losses = (float*)L->losses.p;
    w.perm_slot = (int*)L->perm_slot.p; w.perm_token = (int*)L->perm_token.p; w.inv_pos = (int*)L->inv_pos.p;
    w.h = L->h.p; w.y = L->y.p; w.hs = L->hs.p; w.ys = L->ys.p;
    w.hall = L->hall.p;
    w.expert_tokens = (unsigned int*)L->etok.p;
    w.x16 = L->x16.p;
    w.cmb_counter = (int*)L->cmbcnt.p;
    return w;
}

// The buffers of a decode-shaped forward of T tokens carved out of `base` (pieces of 256 bytes); returns the
// bytes used.  With base == nullptr only the size is computed.
size_t carve_decode_work(const rbmoe_layer* L, int T, unsigned char* base, Work* w) {
    const rbmoe_config& c = L->cfg;
    const size_t E = c.num_experts, d = c.d_model, F = c.d_ff, k = c.experts_per_token, Fs = L->Fs;
    const size_t S = (size_t)T * k, as = L->cast_rows ? 2 : dtype_size(c.act_dtype);
    const size_t tiles = S / kDecodeTileM + E + 1;
    size_t used = 0;
    auto take = [&](size_t bytes) -> void* {
        void* p = base ? base + used : nullptr;
        used += (std::max<size_t>(bytes, 1) + 255) & ~(size_t)255;
        return p;
    };
    Work v;
    // first, at the same place for every call and every layer: the arrival counters of the folded combine, which are
    // zero whenever no call is running (the array starts as zeros and every launch leaves them as it found them)
    v.cmb_counter = (int*)take(kDecodeCombineCounterBytes);
    v.P = (float*)take((size_t)T * E * 4); v.lse = (float*)take((size_t)T * 4);
    v.expert_of = (int*)take(S * 4); v.gate_of = (float*)take(S * 4);
    v.counts = (int*)take(E * 4); v.offsets = (int*)take((E + 1) * 4);
    v.tile_expert = (int*)take(tiles * 4); v.tile_row0 = (int*)take(tiles * 4); v.tile_rows = (int*)take(tiles * 4);
    v.ntiles = (int*)take(8); v.losses = (float*)take(8);
    v.perm_slot = (int*)take(S * 4); v.perm_token = (int*)take(S * 4); v.inv_pos = (int*)take(S * 4);
    v.h = take(S * F * as); v.y = take(S * d * as);
    if ((size_t)T * k >= 2 * E) {  // (the condition of decode_front_ok)
        v.hall = take(E * (size_t)T * F * 2);
        v.expert_tokens = (unsigned int*)take(E * 4);
    }
    if (c.shared_expert) {
        v.hs = take((size_t)T * Fs * as);
        v.ys = take((size_t)T * d * as);
    }
    if (L->cast_rows) v.x16 = take((size_t)T * d * 2);
    if (w) *w = v;
    return used;
}

// `norm_src` (block step): the raw rows; `x` is then the layer's buffer of normed rows, filled here - by the
// small-route kernel itself for a few tokens, by the norm kernel otherwise - before anything reads it.
// `static_scratch` (rbmoe_forward_static): this device's copy of the static scratch array; the call must then be
// decode-shaped, keeps every intermediate result there and touches none of the layer's workspace.
// `timing`: 0 none; 1 an event between the stages (rbmoe_forward_timed); 2 every stage's dispatches carry their own
// start and stop events (rbmoe_forward_kernel_times).
int forward_impl(rbmoe_layer* L, const void* x, int T, int cols, const uint8_t* valid, const float* router_bias,
                 const void* residual, void* out, int timing, const void* norm_src = nullptr,
                 void* static_scratch = nullptr) {
    const bool timed = timing != 0;
    if (!L) return fail(nullptr, RBMOE_NULL_POINTER, "layer is NULL");
    rbmoe_ctx* ctx = L->ctx;
    const rbmoe_config& c = L->cfg;
    const int E = c.num_experts, d = c.d_model, F = c.d_ff, k = c.experts_per_token, Fs = L->Fs;
    // MoeLayer::forward_train's width check (reference src/moe.rs:248-253)
    if (cols != d) {
        char buf[120];
        std::snprintf(buf, sizeof buf, "input length %d does not match expected length %d", cols, d);
        return fail(ctx, RBMOE_INVALID_INPUT, buf);
    }
    if (T < 0) return fail(ctx, RBMOE_INVALID_INPUT, "negative token count");
    if (T > L->max_T) {
        char buf[120];
        std::snprintf(buf, sizeof buf, "%d tokens exceed the layer's max_tokens %d", T, L->max_T);
        return fail(ctx, RBMOE_INVALID_INPUT, buf);
    }
    if (T > 0 && (!x || !out)) return fail(ctx, RBMOE_NULL_POINTER, "x or out is NULL");
    HIP_TRY(ctx, hipSetDevice(ctx->device));
    hipStream_t s = ctx->stream;
    L->last_was_block = false;  // rbmoe_forward_block sets it once this call has succeeded
    const bool abf = c.act_dtype == RBMOE_BF16;
    const bool cast = L->cast_rows;  // f32 rows, bf16 matrix-core products over their bf16 copy
    const WeightKind wk = c.weight_dtype == RBMOE_F32 ? WeightKind::F32
                          : c.weight_dtype == RBMOE_BF16 ? WeightKind::BF16 : WeightKind::I8;
    if (timing == 1 && !L->have_events) {
        for (auto& ev : L->ev) HIP_TRY(ctx, hipEventCreate(&ev));
        L->have_events = true;
    }
    if (timing == 2 && !L->have_ktimers) {
        for (auto& kt : L->ktimer)
            for (auto& ev : kt.ev) HIP_TRY(ctx, hipEventCreate(&ev));
        L->have_ktimers = true;
    }
    struct TimerScope {  // whatever path leaves this function, the thread's launches are plain again
        ~TimerScope() { g_kernel_timer = nullptr; }
    } timer_scope;
    if (timing == 2)
        for (auto& kt : L->ktimer) kt.used = 0;
    // mark(i): stage i - 1 ends here and stage i begins
    auto mark = [&](int i) -> hipError_t {
        if (timing == 2) g_kernel_timer = i < RBMOE_NUM_STAGES - 1 ? &L->ktimer[i] : nullptr;
        return timing == 1 ? hipEventRecord(L->ev[i], s) : hipSuccess;
    };
    HIP_TRY(ctx, mark(0));

    const bool mfma = L->use_stream;
    const bool f32mc = L->use_f32_mc;
    const int tile_m0 = mfma ? stream_tile_m() : (f32mc ? f32_tile_m(T * k, E, std::min(F, d)) : kGenericTileM);
    L->last_tile_m = tile_m0;
    L->kernel_name = mfma ? (wk == WeightKind::I8 ? "mfma_bf16_stream_int8w" : "mfma_bf16_stream")
                          : (f32mc ? "mfma_f32" : "generic");
    // a training layer keeps the gathered rows: the weight gradients of gate and up multiply by them
    const bool gather_in_product = (mfma || f32mc) && !L->explicit_gather && !L->training;

    // whether the single-workgroup routing kernel would stage this call's rows in LDS: only then can it apply the
    // norm and write the bf16 copy of f32 rows
    const bool stages_rows = small_route_stages_rows(x, (const float*)L->router.p, T, d, E, abf) &&
                             (!norm_src || small_route_stages_rows(norm_src, (const float*)L->router.p, T, d, E, abf));
    // (a quantized router has one kernel for its logits, on the large-batch sequence)
    const bool decode_ok = mfma && L->decode_path && !L->training && !L->router_q8 && small_route_ok(T, E, k) &&
                           decode_shape_ok(F, d) &&
                           decode_shape_ok(d, F) &&
                           (!c.shared_expert || (decode_shape_ok(Fs, d) && decode_shape_ok(d, Fs))) &&
                           (!cast || stages_rows);
    const bool norm_in_route = norm_src && decode_ok && stages_rows;
    Work wk_ = work_of_layer(L);
    if (static_scratch) {
        if (!decode_ok) {
            char buf[200];
            std::snprintf(buf, sizeof buf,
                          "rbmoe_forward_static takes decode-shaped calls only: 1 to %d tokens of a layer with bf16 or "
                          "int8 weights on the matrix-core path, not in training mode (got %d tokens)",
                          kSmallRouteMaxTokens, T);
            return fail(ctx, RBMOE_UNSUPPORTED, buf);
        }
        const size_t need = carve_decode_work(L, T, nullptr, nullptr);
        if (need > (size_t)RBMOE_STATIC_SCRATCH_BYTES) {
            char buf[200];
            std::snprintf(buf, sizeof buf, "this call needs %zu bytes of scratch, the static buffer holds %zu", need,
                          (size_t)RBMOE_STATIC_SCRATCH_BYTES);
            return fail(ctx, RBMOE_UNSUPPORTED, buf);
        }
        // Nothing of it is cleared: every word a kernel of this call reads was written by an earlier kernel of
        // the same call (the tile-table entries past *ntiles, which the product kernels fetch and drop, may be
        // a previous call's).
        carve_decode_work(L, T, static_cast<unsigned char*>(static_scratch), &wk_);
    }
    // the rows the expert products read
    const void* const xe = cast ? wk_.x16 : x;
    if (norm_src && !norm_in_route)
        HIP_TRY(ctx, launch_rmsnorm(norm_src, (const float*)L->norm_w.p, L->norm_eps, T, d, L->xn.p, abf, s));

    // ---- a few tokens: route in one workgroup, then stream the touched weights once -------
    if (decode_ok) {
        L->kernel_name = wk == WeightKind::I8 ? "mfma_bf16_decode_int8w" : "mfma_bf16_decode";
        SmallRouteArgs sr{};
        sr.x = x; sr.wr = (const float*)L->router.p; sr.bias = router_bias; sr.valid = valid;
        if (norm_in_route) {
            sr.x = norm_src; sr.norm_w = (const float*)L->norm_w.p; sr.norm_eps = L->norm_eps; sr.xn_out = L->xn.p;
        }
        if (cast) sr.rows16 = wk_.x16;
        // the routing beside the gate/up products, in one launch: bf16 rows as they are (no norm to apply first)
        const bool front = L->decode_front && !norm_src && !cast && wk_.hall != nullptr &&
                           decode_front_ok(x, (const float*)L->router.p, T, d, E, k);
        sr.T = T; sr.d = d; sr.E = E; sr.k = k;
        sr.w_aux = c.aux_loss_weight; sr.w_z = c.router_z_loss_weight;
        sr.tile_m = kDecodeTileM;
        sr.P = wk_.P; sr.lse = wk_.lse;
        sr.expert_of = wk_.expert_of; sr.gate_of = wk_.gate_of;
        sr.counts = wk_.counts; sr.offsets = wk_.offsets;
        sr.tile_expert = wk_.tile_expert; sr.tile_row0 = wk_.tile_row0; sr.tile_rows = wk_.tile_rows;
        sr.ntiles = wk_.ntiles; sr.losses = wk_.losses;
        sr.perm_slot = wk_.perm_slot; sr.perm_token = wk_.perm_token; sr.inv_pos = wk_.inv_pos;
        for (auto& r : L->replay) r = nullptr;
        if (!front) {
            HIP_TRY(ctx, launch_route_small(sr, abf, s));
            L->replay[RBMOE_STAGE_ROUTER] = [=](hipStream_t st) { return launch_route_small(sr, abf, st); };
        }
        HIP_TRY(ctx, mark(1));
        HIP_TRY(ctx, mark(2));
        HIP_TRY(ctx, mark(3));

        DecodeGemmArgs d1{};
        d1.a = xe; d1.row_index = wk_.perm_token;
        d1.w = L->wgu.p; d1.w_expert_stride = (size_t)2 * F * d;
        d1.scales = wk == WeightKind::I8 ? (const float*)L->sgu.p : nullptr; d1.s_expert_stride = (size_t)2 * F;
        d1.N = F; d1.K = d;
        d1.tile_expert = wk_.tile_expert; d1.tile_row0 = wk_.tile_row0;
        d1.tile_rows = wk_.tile_rows; d1.ntiles = wk_.ntiles;
        d1.max_tiles = (T * k) / kDecodeTileM + E;
        d1.out = wk_.h;
        d1.swiglu = 1;
        if (c.shared_expert) {
            d1.a_shared = xe; d1.w_shared = L->swgu.p;
            d1.scales_shared = wk == WeightKind::I8 ? (const float*)L->ssgu.p : nullptr;
            d1.N_shared = Fs; d1.K_shared = d; d1.T_shared = T; d1.out_shared = wk_.hs;
        }
        if (front) {
            d1.row_index = nullptr;
            d1.out = wk_.hall;
            sr.expert_tokens = wk_.expert_tokens;
            HIP_TRY(ctx, launch_decode_front(sr, d1, wk, s));
            L->replay[RBMOE_STAGE_GATE_UP] = [=](hipStream_t st) { return launch_decode_front(sr, d1, wk, st); };
        } else {
            HIP_TRY(ctx, launch_decode_gemm(d1, wk, s));
            L->replay[RBMOE_STAGE_GATE_UP] = [=](hipStream_t st) { return launch_decode_gemm(d1, wk, st); };
        }
        HIP_TRY(ctx, mark(4));

        DecodeGemmArgs d2 = d1;
        d2.a = wk_.h; d2.row_index = nullptr;
        if (front) {  // the routed rows are picked out of the per-expert hidden rows: row token of expert e
            d2.a = wk_.hall; d2.row_index = wk_.perm_token; d2.a_expert_rows = T;
        }
        d2.w = L->wd.p; d2.w_expert_stride = (size_t)d * F;
        d2.scales = wk == WeightKind::I8 ? (const float*)L->sd.p : nullptr; d2.s_expert_stride = (size_t)d;
        d2.N = d; d2.K = F;
        d2.out = wk_.y;
        d2.swiglu = 0;
        if (c.shared_expert) {
            d2.a_shared = wk_.hs; d2.w_shared = L->swd.p;
            d2.scales_shared = wk == WeightKind::I8 ? (const float*)L->ssd.p : nullptr;
            d2.N_shared = d; d2.K_shared = Fs; d2.out_shared = wk_.ys;
        }
        // the combine inside the same launch: the last workgroup of every block of 32 output columns to finish
        // sums that block (same order, same roundings as combine_vec_kernel)
        const bool fold = L->decode_fold && d / 32 <= kDecodeCombineMaxBlocks && wk_.cmb_counter != nullptr;
        if (fold) {
            d2.cmb_counter = wk_.cmb_counter;
            d2.cmb_inv_pos = wk_.inv_pos; d2.cmb_gate_of = wk_.gate_of;
            d2.cmb_residual = residual; d2.cmb_out = out;
            d2.cmb_T = T; d2.cmb_k = k; d2.cmb_f32 = abf ? 0 : 1;
        }
        // behind the routing-beside-the-products launch every expert's rows are known by its token bits: the down
        // launch then has one row of workgroups per expert, whose weights go out before anything of the routing is read
        if (front && fold && L->decode_down_by_expert && wk_.expert_tokens != nullptr && decode_down_by_expert_ok(d2, E, T, k)) {
            const unsigned int* const etok = wk_.expert_tokens;
            const int* const offs = wk_.offsets;
            HIP_TRY(ctx, launch_decode_down_by_expert(d2, etok, offs, E, wk, s));
            L->replay[RBMOE_STAGE_DOWN] = [=](hipStream_t st) { return launch_decode_down_by_expert(d2, etok, offs, E, wk, st); };
        } else {
            HIP_TRY(ctx, launch_decode_gemm(d2, wk, s));
            L->replay[RBMOE_STAGE_DOWN] = [=](hipStream_t st) { return launch_decode_gemm(d2, wk, st); };
        }
        HIP_TRY(ctx, mark(5));
        HIP_TRY(ctx, mark(6));
        if (!fold) {
            CombineArgs cd{wk_.y, c.shared_expert ? wk_.ys : nullptr, residual, wk_.inv_pos, wk_.gate_of, T, d, k, out};
            cd.rows_bf16 = cast;
            HIP_TRY(ctx, launch_combine(cd, abf, s));
            L->replay[RBMOE_STAGE_COMBINE] = [=](hipStream_t st) { return launch_combine(cd, abf, st); };
        }
        HIP_TRY(ctx, mark(7));
        L->last_T = T;
        L->last = wk_;
        L->last_front = front;
        L->kernel_name = front ? (wk == WeightKind::I8 ? "mfma_bf16_decode_front_int8w" : "mfma_bf16_decode_front")
                               : L->kernel_name;
        return RBMOE_OK;
    }

    if (L->training && T > 0)  // MoeCache keeps the input (src/moe.rs:133-135)
        HIP_TRY(ctx, hipMemcpyAsync(L->xc.p, x, (size_t)T * d * dtype_size(c.act_dtype), hipMemcpyDeviceToDevice, s));

    for (auto& r : L->replay) r = nullptr;
    auto run_on = [=](const GroupedArgs& g, hipStream_t st) -> hipError_t {
        if (mfma) return launch_grouped_stream(g, wk, st);
        if (f32mc) return launch_grouped_f32(g, st);
        return launch_grouped_generic(g, abf, wk, kGenericTileM, st);
    };
    auto run = [&](const GroupedArgs& g, bool) -> hipError_t { return run_on(g, s); };
    // The shared expert (src/moe.rs:313-319) takes every row and needs nothing of the routing: with a second stream
    // its two products run beside the routing kernels, which are bound by the vector units and by latency and
    // leave the matrix cores idle.  (Not when the stages are timed one by one, and not over f32 rows, whose bf16
    // copy the logits kernel has yet to write.)
    auto shared_expert = [&](hipStream_t st) -> hipError_t {
        GroupedArgs s1{};
        s1.a = xe;
        s1.w = L->swgu.p;
        s1.scales = wk == WeightKind::I8 ? (const float*)L->ssgu.p : nullptr;
        s1.N = Fs;
        s1.K = d;
        s1.dense_rows = T;
        s1.out = L->hs.p;
        s1.swiglu = true;
        s1.group_m = L->group_m;
        if (L->training) s1.gu_out = L->gus.p;
        hipError_t e = run_on(s1, st);
        if (e != hipSuccess) return e;
        GroupedArgs s2 = s1;
        s2.a = L->hs.p;
        s2.w = L->swd.p;
        s2.scales = wk == WeightKind::I8 ? (const float*)L->ssd.p : nullptr;
        s2.gu_out = nullptr;
        s2.N = d;
        s2.K = Fs;
        s2.out = L->ys.p;
        s2.swiglu = false;
        if (L->group_m == 0) s2.group_m = 4;
        return run_on(s2, st);
    };
    struct JoinGuard {  // an error between fork and join must not leave the side stream forked (a capture could not end)
        rbmoe_ctx* ctx;
        hipStream_t main;
        bool armed = false;
        ~JoinGuard() {
            if (armed) (void)hipStreamWaitEvent(main, ctx->ev_join, 0);
        }
    } join_guard{ctx, s};
    bool shared_forked = false;
    if (c.shared_expert && T >= 1024 && !timed && !cast && L->shared_beside && (mfma || f32mc) &&
        ensure_side_stream(ctx) == RBMOE_OK) {
        HIP_TRY(ctx, hipEventRecord(ctx->ev_fork, s));
        HIP_TRY(ctx, hipStreamWaitEvent(ctx->side_stream, ctx->ev_fork, 0));
        const hipError_t e = shared_expert(ctx->side_stream);
        (void)hipEventRecord(ctx->ev_join, ctx->side_stream);  // recorded whatever happened: the join below always works
        join_guard.armed = true;
        shared_forked = true;
        if (e != hipSuccess) return hip_fail(ctx, e, "shared expert on the side stream");
    }

    RouterArgs ra{x, (const float*)L->router.p, router_bias, valid, T, d, E, k,
                  (float*)L->P.p, (float*)L->lse.p, (int*)L->expert_of.p, (float*)L->gate_of.p,
                  (int*)L->rank_in_block.p, (int*)L->blockcnt.p, (float*)L->partial.p};
    if (cast) ra.rows16 = L->x16.p;
    ra.allow_fused = L->fused_router;
    if (L->router_q8) {
        ra.wq = (const int8_t*)L->router_q.p;
        ra.wscale = (const float*)L->router_s.p;
        if (cast) {  // the quantized router's kernel does not write the bf16 copy of f32 rows on its way
            ra.rows16 = nullptr;
            HIP_TRY(ctx, launch_cast_rows_bf16((const float*)x, L->x16.p, (long long)T * d, s));
        }
    }
    HIP_TRY(ctx, launch_router(ra, abf, s));
    L->replay[RBMOE_STAGE_ROUTER] = [=](hipStream_t st) { return launch_router(ra, abf, st); };
    HIP_TRY(ctx, mark(1));

    HIP_TRY(ctx, mark(2));  // an interval with no work in it: the cost of one pair of event records

    DispatchArgs da{};
    da.x = xe;
    da.expert_of = (const int*)L->expert_of.p;
    da.rank_in_block = (const int*)L->rank_in_block.p;
    da.blockcnt = (const int*)L->blockcnt.p;
    da.partial = (const float*)L->partial.p;
    da.blockbase = (int*)L->blockbase.p;
    da.T = T; da.d = d; da.E = E; da.k = k;
    da.w_aux = c.aux_loss_weight; da.w_z = c.router_z_loss_weight;
    da.tile_m = tile_m0;
    da.counts = (int*)L->counts.p; da.offsets = (int*)L->offsets.p;
    da.tile_expert = (int*)L->tile_expert.p; da.tile_row0 = (int*)L->tile_row0.p; da.tile_rows = (int*)L->tile_rows.p;
    da.ntiles = (int*)L->ntiles.p; da.losses = (float*)L->losses.p;
    da.perm_slot = (int*)L->perm_slot.p; da.perm_token = (int*)L->perm_token.p; da.inv_pos = (int*)L->inv_pos.p;
    da.xg = gather_in_product ? nullptr : L->xg.p;
    HIP_TRY(ctx, launch_dispatch(da, abf || cast, s));
    {
        const bool rows_bf16 = abf || cast;
        L->replay[RBMOE_STAGE_DISPATCH] = [=](hipStream_t st) { return launch_dispatch(da, rows_bf16, st); };
    }
    HIP_TRY(ctx, mark(3));

    GroupedArgs g1{};
    g1.a = gather_in_product ? xe : L->xg.p;
    g1.row_index = gather_in_product ? (const int*)L->perm_token.p : nullptr;
    g1.w = L->wgu.p;
    g1.w_expert_stride = (size_t)2 * F * d;
    g1.scales = wk == WeightKind::I8 ? (const float*)L->sgu.p : nullptr;
    g1.s_expert_stride = (size_t)2 * F;
    g1.N = F;
    g1.K = d;
    g1.tile_expert = (const int*)L->tile_expert.p;
    g1.tile_row0 = (const int*)L->tile_row0.p;
    g1.tile_rows = (const int*)L->tile_rows.p;
    g1.ntiles = (const int*)L->ntiles.p;
    g1.max_tiles = T > 0 ? (T * k) / tile_m0 + E : 0;
    g1.tile_m = tile_m0;
    g1.dense_rows = -1;
    g1.out = L->h.p;
    g1.swiglu = true;
    g1.group_m = L->group_m;
    if (L->training) g1.gu_out = L->gu.p;
    HIP_TRY(ctx, run(g1, true));
    L->replay[RBMOE_STAGE_GATE_UP] = [=](hipStream_t st) { return run_on(g1, st); };
    HIP_TRY(ctx, mark(4));

    GroupedArgs g2 = g1;
    g2.a = L->h.p;
    g2.gu_out = nullptr;
    g2.row_index = nullptr;
    g2.w = L->wd.p;
    g2.w_expert_stride = (size_t)d * F;
    g2.scales = wk == WeightKind::I8 ? (const float*)L->sd.p : nullptr;
    g2.s_expert_stride = (size_t)d;
    g2.N = d;
    g2.K = F;
    g2.out = L->y.p;
    g2.swiglu = false;
    // M-tiles that walk the column tiles together on one XCD: what they share must fit its 4 MiB L2 beside the
    // weights - eight tiles' token rows for the gate/up product (launch_grouped_stream's default), four tiles' hidden
    // rows, which are wider, for the down product (measured HBM-side traffic: 270 against 301 MB with groups of 8
    // against 4 for gate/up, 147 against 166 MB with 4 against 8 for down)
    if (L->group_m == 0) g2.group_m = 4;
    HIP_TRY(ctx, run(g2, false));
    L->replay[RBMOE_STAGE_DOWN] = [=](hipStream_t st) { return run_on(g2, st); };
    HIP_TRY(ctx, mark(5));

    if (c.shared_expert && T > 0 && !shared_forked) HIP_TRY(ctx, shared_expert(s));
    if (shared_forked) {
        HIP_TRY(ctx, hipStreamWaitEvent(s, ctx->ev_join, 0));
        join_guard.armed = false;
    }
    HIP_TRY(ctx, mark(6));

    CombineArgs ca{L->y.p, c.shared_expert ? L->ys.p : nullptr, residual, (const int*)L->inv_pos.p,
                   (const float*)L->gate_of.p, T, d, k, out};
    ca.rows_bf16 = cast;
    HIP_TRY(ctx, launch_combine(ca, abf, s));
    L->replay[RBMOE_STAGE_COMBINE] = [=](hipStream_t st) { return launch_combine(ca, abf, st); };
    HIP_TRY(ctx, mark(7));
    L->last_T = T;
    L->last = wk_;
    L->last_front = false;
    return RBMOE_OK;
}

// Allocates and clears the buffers of `p` for a layer that already exists: the budget is checked before
// anything is allocated, and a failure part-way frees what this call had allocated, so that the layer is left as
// it was and the call can simply be made again.
int allocate_plan(rbmoe_layer* L, Plan& p, const char* what) {
    rbmoe_ctx* ctx = L->ctx;
    if (ctx->budget_bytes && ctx->allocated + p.total > ctx->budget_bytes) {
        char buf[200];
        std::snprintf(buf, sizeof buf, "memory budget exceeded: estimated %zu MiB exceeds budget %zu MiB",
                      (ctx->allocated + p.total + (1 << 20) - 1) >> 20, ctx->budget_bytes >> 20);
        return fail(ctx, RBMOE_MEMORY_BUDGET, buf);
    }
    size_t done = 0;
    hipError_t e = hipSetDevice(ctx->device);
    while (e == hipSuccess && done < p.items.size()) {
        auto& it = p.items[done];
        void* q = nullptr;
        e = hipMalloc(&q, it.second);
        if (e != hipSuccess) break;
        it.first->p = q;
        it.first->bytes = it.second;
        ctx->allocated += it.second;
        L->all.push_back(it.first);
        ++done;
        e = hipMemsetAsync(q, 0, it.second, ctx->stream);
    }
    if (e == hipSuccess) e = hipStreamSynchronize(ctx->stream);
    if (e == hipSuccess) return RBMOE_OK;
    (void)hipGetLastError();
    (void)hipStreamSynchronize(ctx->stream);
    for (size_t i = 0; i < done; ++i) {
        Buf* b = p.items[i].first;
        (void)hipFree(b->p);
        if (ctx->allocated >= b->bytes) ctx->allocated -= b->bytes;
        b->p = nullptr;
        b->bytes = 0;
        for (size_t j = L->all.size(); j-- > 0;)
            if (L->all[j] == b) {
                L->all.erase(L->all.begin() + (long)j);
                break;
            }
    }
    if (e == hipErrorOutOfMemory)
        return fail(ctx, RBMOE_OUT_OF_MEMORY, std::string("out of memory while allocating ") + what);
    return hip_fail(ctx, e, what);
}

// Buffers of the backward pass through the norm: allocated by whichever of rbmoe_set_feed_forward_norm and
// rbmoe_layer_enable_training comes second.
int ensure_block_training_buffers(rbmoe_layer* L) {
    if (!L->training || !L->norm_w.p || L->xraw.p) return RBMOE_OK;
    const rbmoe_config& c = L->cfg;
    const size_t T = L->max_T, d = c.d_model, as = dtype_size(c.act_dtype);
    Plan p;
    p.add(&L->xraw, T * d * as);
    p.add(&L->dxn, T * d * as);
    p.add(&L->inv_rms, T * 4);
    p.add(&L->norm_partial, (size_t)rmsnorm_grad_tiles((int)T) * d * 4);
    p.add(&L->g_norm, d * 4);
    return allocate_plan(L, p, "the norm's backward buffers");
}

}  // namespace

extern "C" {

int rbmoe_forward(rbmoe_layer* L, const void* x, int32_t T, int32_t cols, const uint8_t* valid,
                  const float* router_bias, const void* residual, void* out) {
    return forward_impl(L, x, T, cols, valid, router_bias, residual, out, 0);
}

int rbmoe_forward_static(rbmoe_layer* L, const void* x, int32_t T, int32_t cols, const uint8_t* valid,
                         const float* router_bias, const void* residual, void* out) {
    if (!L) return fail(nullptr, RBMOE_NULL_POINTER, "layer is NULL");
    if (!L->ctx->static_scratch) return fail(L->ctx, RBMOE_DEVICE_ERROR, "the static scratch buffer was not resolved");
    return forward_impl(L, x, T, cols, valid, router_bias, residual, out, 0, nullptr, L->ctx->static_scratch);
}

int rbmoe_forward_timed(rbmoe_layer* L, const void* x, int32_t T, int32_t cols, const uint8_t* valid,
                        const float* router_bias, const void* residual, void* out, float* ms) {
    if (!ms) return fail(L ? L->ctx : nullptr, RBMOE_NULL_POINTER, "ms is NULL");
    int rc = forward_impl(L, x, T, cols, valid, router_bias, residual, out, 1);
    if (rc != RBMOE_OK) return rc;
    rbmoe_ctx* ctx = L->ctx;
    HIP_TRY(ctx, hipStreamSynchronize(ctx->stream));
    for (int i = 0; i < RBMOE_NUM_STAGES - 1; ++i)
        HIP_TRY(ctx, hipEventElapsedTime(&ms[i], L->ev[i], L->ev[i + 1]));
    HIP_TRY(ctx, hipEventElapsedTime(&ms[RBMOE_STAGE_TOTAL], L->ev[0], L->ev[RBMOE_NUM_STAGES - 1]));
    return RBMOE_OK;
}

int rbmoe_forward_kernel_times(rbmoe_layer* L, const void* x, int32_t T, int32_t cols, const uint8_t* valid,
                               const float* router_bias, const void* residual, void* out, float* ms) {
    if (!ms) return fail(L ? L->ctx : nullptr, RBMOE_NULL_POINTER, "ms is NULL");
    int rc = forward_impl(L, x, T, cols, valid, router_bias, residual, out, 2);
    if (rc != RBMOE_OK) return rc;
    rbmoe_ctx* ctx = L->ctx;
    HIP_TRY(ctx, hipStreamSynchronize(ctx->stream));
    float total = 0.0f;
    for (int i = 0; i < RBMOE_NUM_STAGES - 1; ++i) {
        ms[i] = 0.0f;
        for (int u = 0; u < L->ktimer[i].used; ++u) {
            float one = 0.0f;
            HIP_TRY(ctx, hipEventElapsedTime(&one, L->ktimer[i].ev[2 * u], L->ktimer[i].ev[2 * u + 1]));
            ms[i] += one;
        }
        total += ms[i];
    }
    ms[RBMOE_STAGE_TOTAL] = total;
    return RBMOE_OK;
}

int rbmoe_replay_stage(rbmoe_layer* L, int32_t stage, int32_t launches, float* ms_per_launch) {
    if (!L) return fail(nullptr, RBMOE_NULL_POINTER, "layer is NULL");
    rbmoe_ctx* ctx = L->ctx;
    if (stage < 0 || stage >= RBMOE_NUM_STAGES || launches <= 0)
        return fail(ctx, RBMOE_INVALID_INPUT, "stage out of range or launches not positive");
    if (L->last_T < 0) return fail(ctx, RBMOE_INVALID_INPUT, "no forward pass has run yet");
    if (!L->replay[stage]) return fail(ctx, RBMOE_UNSUPPORTED, "the last forward had no launch of its own for this stage");
    HIP_TRY(ctx, hipSetDevice(ctx->device));
    hipStream_t s = ctx->stream;
    if (!ms_per_launch) {  // enqueue only: the caller times a sequence of its own
        for (int i = 0; i < launches; ++i) HIP_TRY(ctx, L->replay[stage](s));
        return RBMOE_OK;
    }
    if (!L->have_events) {
        for (auto& ev : L->ev) HIP_TRY(ctx, hipEventCreate(&ev));
        L->have_events = true;
    }
    HIP_TRY(ctx, L->replay[stage](s));  // warm-up: the stage's operands are back in the caches it usually finds them in
    HIP_TRY(ctx, hipEventRecord(L->ev[0], s));
    for (int i = 0; i < launches; ++i) HIP_TRY(ctx, L->replay[stage](s));
    HIP_TRY(ctx, hipEventRecord(L->ev[1], s));
    HIP_TRY(ctx, hipStreamSynchronize(s));
    float ms = 0.0f;
    HIP_TRY(ctx, hipEventElapsedTime(&ms, L->ev[0], L->ev[1]));
    *ms_per_launch = ms / (float)launches;
    return RBMOE_OK;
}

int rbmoe_forward_host(rbmoe_layer* L, const void* x, int32_t T, int32_t cols, const uint8_t* valid,
                       const float* router_bias, const void* residual, void* out) {
    if (!L) return fail(nullptr, RBMOE_NULL_POINTER, "layer is NULL");
    rbmoe_ctx* ctx = L->ctx;
    const rbmoe_config& c = L->cfg;
    if (cols != c.d_model) {
        char buf[120];
        std::snprintf(buf, sizeof buf, "input length %d does not match expected length %d", cols, c.d_model);
        return fail(ctx, RBMOE_INVALID_INPUT, buf);
    }
    if (T < 0 || T > L->max_T) return fail(ctx, RBMOE_INVALID_INPUT, "token count outside [0, max_tokens]");
    if (T > 0 && (!x || !out)) return fail(ctx, RBMOE_NULL_POINTER, "x or out is NULL");
    HIP_TRY(ctx, hipSetDevice(ctx->device));
    const size_t as = dtype_size(c.act_dtype);
    const size_t nbytes = (size_t)T * c.d_model * as;
    hipStream_t s = ctx->stream;
    if (T > 0) {
        HIP_TRY(ctx, hipMemcpyAsync(L->st_x.p, x, nbytes, hipMemcpyHostToDevice, s));
        if (valid) HIP_TRY(ctx, hipMemcpyAsync(L->st_valid.p, valid, (size_t)T, hipMemcpyHostToDevice, s));
        if (residual) HIP_TRY(ctx, hipMemcpyAsync(L->st_res.p, residual, nbytes, hipMemcpyHostToDevice, s));
    }
    if (router_bias)
        HIP_TRY(ctx, hipMemcpyAsync(L->st_bias.p, router_bias, (size_t)c.num_experts * 4, hipMemcpyHostToDevice, s));
    int rc = forward_impl(L, L->st_x.p, T, cols, valid ? (const uint8_t*)L->st_valid.p : nullptr,
                          router_bias ? (const float*)L->st_bias.p : nullptr, residual ? L->st_res.p : nullptr,
                          L->st_out.p, 0);
    if (rc != RBMOE_OK) return rc;
    if (T > 0) HIP_TRY(ctx, hipMemcpyAsync(out, L->st_out.p, nbytes, hipMemcpyDeviceToHost, s));
    HIP_TRY(ctx, hipStreamSynchronize(s));
    return RBMOE_OK;
}

// ---------------------------------------------------------------------------
// The block's steps either side of the layer: RmsNorm::forward in front
// (src/norm.rs:41-61, src/transformer_block.rs:216), the residual add behind
// (src/transformer_block.rs:221-222).
// ---------------------------------------------------------------------------
int rbmoe_set_feed_forward_norm(rbmoe_layer* L, const float* weight, int32_t cols, float eps) {
    if (!L) return fail(nullptr, RBMOE_NULL_POINTER, "layer is NULL");
    rbmoe_ctx* ctx = L->ctx;
    const rbmoe_config& c = L->cfg;
    if (!weight) return fail(ctx, RBMOE_NULL_POINTER, "weight is NULL");
    if (cols != c.d_model) {
        char buf[120];
        std::snprintf(buf, sizeof buf, "norm weight length %d does not match expected length %d", cols, c.d_model);
        return fail(ctx, RBMOE_INVALID_INPUT, buf);
    }
    HIP_TRY(ctx, hipSetDevice(ctx->device));
    if (!L->norm_w.p) {
        Plan p;
        p.add(&L->xn, (size_t)L->max_T * c.d_model * dtype_size(c.act_dtype));
        p.add(&L->norm_w, (size_t)c.d_model * 4);
        if (const int rc = allocate_plan(L, p, "the normed rows")) return rc;
    }
    HIP_TRY(ctx, hipStreamSynchronize(ctx->stream));  // no forward may still read the old weight
    HIP_TRY(ctx, hipMemcpy(L->norm_w.p, weight, (size_t)c.d_model * 4, hipMemcpyHostToDevice));
    L->norm_eps = eps;
    L->norm_set = true;
    return ensure_block_training_buffers(L);
}

int rbmoe_forward_block(rbmoe_layer* L, const void* x, int32_t T, int32_t cols, const uint8_t* valid,
                        const float* router_bias, void* out) {
    if (!L) return fail(nullptr, RBMOE_NULL_POINTER, "layer is NULL");
    rbmoe_ctx* ctx = L->ctx;
    if (!L->norm_set) return fail(ctx, RBMOE_INVALID_CONFIG, "the feed-forward norm has not been set");
    if (cols != L->cfg.d_model) {
        char buf[120];
        std::snprintf(buf, sizeof buf, "input length %d does not match expected length %d", cols, L->cfg.d_model);
        return fail(ctx, RBMOE_INVALID_INPUT, buf);
    }
    if (T < 0 || T > L->max_T) return fail(ctx, RBMOE_INVALID_INPUT, "token count outside [0, max_tokens]");
    if (T > 0 && (!x || !out)) return fail(ctx, RBMOE_NULL_POINTER, "x or out is NULL");
    HIP_TRY(ctx, hipSetDevice(ctx->device));
    if (L->training && T > 0)  // TransformerBlockCache keeps the residual (src/transformer_block.rs:224-232)
        HIP_TRY(ctx, hipMemcpyAsync(L->xraw.p, x, (size_t)T * cols * dtype_size(L->cfg.act_dtype),
                                    hipMemcpyDeviceToDevice, ctx->stream));
    const int rc = forward_impl(L, L->xn.p, T, cols, valid, router_bias, x, out, 0, x);
    if (rc == RBMOE_OK) L->last_was_block = true;
    return rc;
}

int rbmoe_forward_block_host(rbmoe_layer* L, const void* x, int32_t T, int32_t cols, const uint8_t* valid,
                             const float* router_bias, void* out) {
    if (!L) return fail(nullptr, RBMOE_NULL_POINTER, "layer is NULL");
    rbmoe_ctx* ctx = L->ctx;
    const rbmoe_config& c = L->cfg;
    if (!L->norm_set) return fail(ctx, RBMOE_INVALID_CONFIG, "the feed-forward norm has not been set");
    if (cols != c.d_model) {
        char buf[120];
        std::snprintf(buf, sizeof buf, "input length %d does not match expected length %d", cols, c.d_model);
        return fail(ctx, RBMOE_INVALID_INPUT, buf);
    }
    if (T < 0 || T > L->max_T) return fail(ctx, RBMOE_INVALID_INPUT, "token count outside [0, max_tokens]");
    if (T > 0 && (!x || !out)) return fail(ctx, RBMOE_NULL_POINTER, "x or out is NULL");
    HIP_TRY(ctx, hipSetDevice(ctx->device));
    const size_t nbytes = (size_t)T * c.d_model * dtype_size(c.act_dtype);
    hipStream_t s = ctx->stream;
    if (T > 0) {
        HIP_TRY(ctx, hipMemcpyAsync(L->st_x.p, x, nbytes, hipMemcpyHostToDevice, s));
        if (valid) HIP_TRY(ctx, hipMemcpyAsync(L->st_valid.p, valid, (size_t)T, hipMemcpyHostToDevice, s));
    }
    if (router_bias)
        HIP_TRY(ctx, hipMemcpyAsync(L->st_bias.p, router_bias, (size_t)c.num_experts * 4, hipMemcpyHostToDevice, s));
    int rc = rbmoe_forward_block(L, L->st_x.p, T, cols, valid ? (const uint8_t*)L->st_valid.p : nullptr,
                                 router_bias ? (const float*)L->st_bias.p : nullptr, L->st_out.p);
    if (rc != RBMOE_OK) return rc;
    if (T > 0) HIP_TRY(ctx, hipMemcpyAsync(out, L->st_out.p, nbytes, hipMemcpyDeviceToHost, s));
    HIP_TRY(ctx, hipStreamSynchronize(s));
    return RBMOE_OK;
}

// ---------------------------------------------------------------------------
// Training: MoeLayer::backward (reference src/moe.rs:348-489).
// ---------------------------------------------------------------------------
int rbmoe_layer_enable_training(rbmoe_layer* L) {
    if (!L) return fail(nullptr, RBMOE_NULL_POINTER, "layer is NULL");
    rbmoe_ctx* ctx = L->ctx;
    if (L->training) return RBMOE_OK;
    const rbmoe_config& c = L->cfg;
    if (c.weight_dtype == RBMOE_I8)  // as in the reference: quantized experts are inference-only (src/ffn.rs:87-93)
        return fail(ctx, RBMOE_UNSUPPORTED, "the backward pass is not defined for int8 weights");
    if (L->weights_set)
        return fail(ctx, RBMOE_INVALID_CONFIG, "enable training before the weights are set");
    if (L->quantize_router)
        return fail(ctx, RBMOE_UNSUPPORTED, "the backward pass is not defined for a quantized router");
    // (f32 rows over bf16 weights - the reference's own mixed-precision shape, src/gpu_model.rs:2146-2153 - stay on
    // the matrix cores in both directions: the products read the bf16 copy of the rows that the forward writes
    // anyway and a bf16 copy of the upstream gradient that the backward pass writes first; the router's branch,
    // the norm and the sums that end in the caller's buffers stay f32)
    const bool bf16_layer = L->use_stream && c.weight_dtype == RBMOE_BF16;
    if (L->max_T > router_grad_max_tokens()) {  // found here, not in the middle of a backward pass
        char buf[160];
        std::snprintf(buf, sizeof buf, "the backward pass takes at most %d tokens a call, the layer was created for %d",
                      router_grad_max_tokens(), L->max_T);
        return fail(ctx, RBMOE_UNSUPPORTED, buf);
    }
    const size_t E = c.num_experts, d = c.d_model, F = c.d_ff, Fs = L->Fs, T = L->max_T, S = L->max_S;
    if (bf16_layer) {
        if (!stream_shape_ok((int)d, (int)(2 * F)) || (c.shared_expert && !stream_shape_ok((int)d, (int)(2 * Fs))))
            return fail(ctx, RBMOE_UNSUPPORTED, "expert width not supported by the backward products");
        // 32-bit byte offsets into the widest operand of the backward products: [S, 2F] bf16
        if (std::max(S * 2 * F, T * 2 * Fs) * 2 >= ((size_t)1 << 32))
            return fail(ctx, RBMOE_UNSUPPORTED, "max_tokens x expert width too large for the backward products");
    } else if (L->use_f32_mc &&
               (!f32_shape_ok((int)d, (int)(2 * F)) || (c.shared_expert && !f32_shape_ok((int)d, (int)(2 * Fs))))) {
        return fail(ctx, RBMOE_UNSUPPORTED, "expert width not supported by the backward products");
    }
    // (any other layer - odd widths, mixed dtypes - takes the any-shape kernels in both directions)
    const size_t ws = dtype_size(c.weight_dtype);  // bytes per element of the transposed weight copies
    const size_t as = dtype_size(c.act_dtype);
    const size_t ps = L->cast_rows ? 2 : as;       // bytes per element of the rows the products read and write
    Plan p;
    p.add(&L->xc, T * d * as);
    if (L->cast_rows) p.add(&L->g16, T * d * 2);
    p.add(&L->gu, S * 2 * F * ps);
    p.add(&L->dy, S * d * ps);
    p.add(&L->dgu, S * 2 * F * ps);
    p.add(&L->dxg, S * d * ps);
    p.add(&L->grad_gates, S * 4);
    p.add(&L->ones, S * 4);
    p.add(&L->dlogits, T * E * 4);
    p.add(&L->dxr, T * d * as);
    p.add(&L->rpartial, (size_t)router_grad_chunks((int)T) * E * d * 4);
    p.add(&L->g_router, E * d * 4);
    p.add(&L->g_gu, E * 2 * F * d * 4);
    p.add(&L->g_down, E * d * F * 4);
    p.add(&L->wdT, E * F * d * ws);
    p.add(&L->wguT, E * d * 2 * F * ws);
    // (four tables: down and gate/up gradients of the routed experts and of the shared one)
    p.add(&L->wg_chunks, (size_t)4 * wgrad_table_ints(L) * 4);
    // How the weight gradients treat an expert far above the average share (and the shared expert, whose one
    // group of rows is always cut): in a fixed order by default (RBMOE_OPT_WGRAD_MODE for f32 atomics or no cut).
    if (L->wgrad_split == WgradSplit::Ordered) {
        const bool wbf = c.act_dtype == RBMOE_BF16 || L->cast_rows;
        // sized for every token count up to max_tokens: a smaller batch can need more partial matrices than the
        // largest one, because the cut limit follows the row count with a floor and a rounding
        const int k = c.experts_per_token;
        size_t need = std::max(weight_grad_partial_bytes_upto((int)d, (int)F, (int)E, false, (int)T, k, wbf),
                               weight_grad_partial_bytes_upto((int)(2 * F), (int)d, (int)E, false, (int)T, k, wbf));
        if (c.shared_expert)
            need = std::max(need, std::max(weight_grad_partial_bytes_upto((int)d, (int)Fs, 1, true, (int)T, 1, wbf),
                                           weight_grad_partial_bytes_upto((int)(2 * Fs), (int)d, 1, true, (int)T, 1, wbf)));
        p.add(&L->wg_partial, need);
    }
    p.add(&L->st_gout, T * d * as);
    p.add(&L->st_gin, T * d * as);
    if (c.shared_expert) {
        p.add(&L->gus, T * 2 * Fs * ps);
        p.add(&L->dgus, T * 2 * Fs * ps);
        p.add(&L->dxs, T * d * ps);
        p.add(&L->g_sgu, 2 * Fs * d * 4);
        p.add(&L->g_sdown, d * Fs * 4);
        p.add(&L->swdT, Fs * d * ws);
        p.add(&L->swguT, d * 2 * Fs * ws);
    }
    // (the second stream first: a failure there must not leave buffers behind that a second attempt would allocate again)
    if (L->shared_beside)
        if (const int rc = ensure_side_stream(ctx)) return rc;
    if (const int rc = allocate_plan(L, p, "the training buffers")) return rc;
    HIP_TRY(ctx, launch_fill_f32((float*)L->ones.p, 1.0f, (long long)S, ctx->stream));
    HIP_TRY(ctx, hipStreamSynchronize(ctx->stream));
    L->side_branch = L->shared_beside;
    L->training = true;
    L->grads_clear = true;
    return ensure_block_training_buffers(L);
}

int rbmoe_layer_set_option(rbmoe_layer* L, int32_t option, int32_t value) {
    if (!L) return fail(nullptr, RBMOE_NULL_POINTER, "layer is NULL");
    rbmoe_ctx* ctx = L->ctx;
    switch (option) {
        case RBMOE_OPT_FORCE_GENERIC:
            // the kernel set decides how the weights are laid out on the device
            if (L->weights_set || L->training)
                return fail(ctx, RBMOE_INVALID_CONFIG, "choose the kernel set before weights are set or training is enabled");
            L->force_generic = value != 0;
            choose_kernel_sets(L);
            return RBMOE_OK;
        case RBMOE_OPT_EXPLICIT_GATHER: L->explicit_gather = value != 0; return RBMOE_OK;
        case RBMOE_OPT_GROUP_M:
            if (value < 0) return fail(ctx, RBMOE_INVALID_CONFIG, "the group size must not be negative");
            L->group_m = value;
            return RBMOE_OK;
        case RBMOE_OPT_DECODE_PATH: L->decode_path = value != 0; return RBMOE_OK;
        case RBMOE_OPT_DECODE_FRONT: L->decode_front = value != 0; return RBMOE_OK;
        case RBMOE_OPT_FUSED_ROUTER: L->fused_router = value != 0; return RBMOE_OK;
        case RBMOE_OPT_DECODE_COMBINE_FOLD: L->decode_fold = value != 0; return RBMOE_OK;
        case RBMOE_OPT_DECODE_DOWN_BY_EXPERT: L->decode_down_by_expert = value != 0; return RBMOE_OK;
        case RBMOE_OPT_SIDE_STREAM:
            if (value != 0 && L->training)
                if (const int rc = ensure_side_stream(ctx)) return rc;
            L->shared_beside = value != 0;
            L->side_branch = value != 0;
            return RBMOE_OK;
        case RBMOE_OPT_WGRAD_MODE:
            if (value < 0 || value > 2) return fail(ctx, RBMOE_INVALID_CONFIG, "weight-gradient mode must be 0, 1 or 2");
            L->wgrad_split = value == 0 ? WgradSplit::Ordered : value == 1 ? WgradSplit::Atomic : WgradSplit::None;
            return RBMOE_OK;
        case RBMOE_OPT_WGRAD_GENERIC: L->wgrad_generic = value != 0; return RBMOE_OK;
        case RBMOE_OPT_QUANT_RULE:
            if (value != 0 && value != 1) return fail(ctx, RBMOE_INVALID_CONFIG, "the quantisation rule is 0 or 1");
            L->quant_rule = value;
            return RBMOE_OK;
        case RBMOE_OPT_QUANTIZE_ROUTER:
            if (value != 0 && L->training)
                return fail(ctx, RBMOE_UNSUPPORTED, "the backward pass is not defined for a quantized router");
            L->quantize_router = value != 0;
            return RBMOE_OK;
    }
    return fail(ctx, RBMOE_INVALID_CONFIG, "unknown option");
}

int rbmoe_zero_grads(rbmoe_layer* L) {
    if (!L) return fail(nullptr, RBMOE_NULL_POINTER, "layer is NULL");
    rbmoe_ctx* ctx = L->ctx;
    if (!L->training) return fail(ctx, RBMOE_INVALID_CONFIG, "training is not enabled on this layer");
    // The expert matrices (hundreds of MB) are not touched: they count as zero from here on, and the next
    // backward pass writes them instead of adding to them.  The router's gradient is small and is cleared.
    HIP_TRY(ctx, hipSetDevice(ctx->device));
    // (a fill kernel, not a memset: a caller may capture a training step in a graph)
    HIP_TRY(ctx, launch_fill_f32((float*)L->g_router.p, 0.0f, (long long)(L->g_router.bytes / 4), ctx->stream));
    if (L->g_norm.p) HIP_TRY(ctx, launch_fill_f32((float*)L->g_norm.p, 0.0f, (long long)(L->g_norm.bytes / 4), ctx->stream));
    L->grads_clear = true;
    return RBMOE_OK;
}

// The backward entry points differentiate the LAST forward, whose shape the reference takes from the cached input
// (src/moe.rs:349-350).  Here the cache is the layer's own state, so the caller states the shape of its buffers
// and a mismatch is refused before any of their bytes is read or written.
static int backward_shape_problem(rbmoe_layer* L, int32_t tokens, int32_t cols) {
    rbmoe_ctx* ctx = L->ctx;
    char buf[160];
    if (cols != L->cfg.d_model) {
        std::snprintf(buf, sizeof buf, "gradient length %d does not match expected length %d", cols, L->cfg.d_model);
        return fail(ctx, RBMOE_INVALID_INPUT, buf);
    }
    if (tokens != L->last_T) {
        std::snprintf(buf, sizeof buf, "gradient rows %d do not match the %d rows of the last forward pass", tokens,
                      L->last_T);
        return fail(ctx, RBMOE_INVALID_INPUT, buf);
    }
    return RBMOE_OK;
}

int rbmoe_backward(rbmoe_layer* L, const void* grad_output, int32_t tokens, int32_t cols, void* grad_input) {
    if (!L) return fail(nullptr, RBMOE_NULL_POINTER, "layer is NULL");
    rbmoe_ctx* ctx = L->ctx;
    if (!L->training) return fail(ctx, RBMOE_INVALID_CONFIG, "training is not enabled on this layer");
    if (L->last_T < 0) return fail(ctx, RBMOE_INVALID_INPUT, "no forward pass has run yet");
    if (const int rc = backward_shape_problem(L, tokens, cols)) return rc;
    const rbmoe_config& c = L->cfg;
    const int E = c.num_experts, d = c.d_model, F = c.d_ff, k = c.experts_per_token, Fs = L->Fs, T = L->last_T;
    if (T == 0) return RBMOE_OK;
    if (!grad_output || !grad_input) return fail(ctx, RBMOE_NULL_POINTER, "grad_output or grad_input is NULL");
    HIP_TRY(ctx, hipSetDevice(ctx->device));
    hipStream_t s = ctx->stream;
    const bool xbf = c.act_dtype == RBMOE_BF16;       // the caller's rows and gradients
    const bool cast = L->cast_rows;                   // ... are f32, the products' rows bf16
    const bool abf = xbf || cast;                     // the rows of the expert products
    const int S = T * k;
    const int* offsets = (const int*)L->offsets.p;
    const int* counts = (const int*)L->counts.p;
    // what the expert branch reads of the upstream gradient: the caller's rows, or their bf16 copy
    const void* gout = grad_output;
    if (cast) {
        HIP_TRY(ctx, launch_cast_rows_bf16((const float*)grad_output, L->g16.p, (long long)T * d, s));
        gout = L->g16.p;
    }

    // upstream of every expert: gate * dOut[token]; gate gradient: dOut[token] . Y[row]
    // (grad_gates of unrouted slots stays unwritten: the only reader skips padding rows)
    HIP_TRY(ctx, launch_scale_rows(gout, L->y.p, (const int*)L->perm_slot.p, (const int*)L->perm_token.p,
                                   (const float*)L->gate_of.p, offsets, E, d, S, L->dy.p, (float*)L->grad_gates.p, abf,
                                   s));
    // The router's branch needs nothing but the gate gradients from here on and is a handful of small launches
    // that leave most of the chip idle: it runs on the side stream, beside the products below, which meet
    // again at the final sum.  Gates -> probabilities -> logits with the two auxiliary losses
    // (src/moe.rs:421-478), then the router's weight and input gradients.
    const bool side = L->side_branch && ctx->side_stream != nullptr;
    const hipStream_t rs = side ? ctx->side_stream : s;
    if (side) {
        HIP_TRY(ctx, hipEventRecord(ctx->ev_fork, s));
        HIP_TRY(ctx, hipStreamWaitEvent(rs, ctx->ev_fork, 0));
    }
    // grad_input = sum over a token's slots of its expert rows + shared + router
    CombineArgs ca{L->dxg.p, c.shared_expert ? L->dxs.p : nullptr, L->dxr.p, (const int*)L->inv_pos.p,
                   (const float*)L->ones.p, T, d, k, grad_input};
    ca.rows_bf16 = cast;
    const bool combine_on_side = side && !c.shared_expert;
    const bool tables_early = side && !L->wgrad_generic;
    // From here to the join the side stream hangs off the main one: an error in between must not leave it forked
    // (a stream capture in progress could then never end), so the rest runs as one unit that is always joined.
    auto forked = [&]() -> int {
    if (tables_early) {
        // the chunk tables of the weight-gradient launches depend on nothing but the forward's counts and offsets:
        // they are worked out here, on the side stream, instead of in front of each product on the main one
        auto table = [&](int which, int M, int N, int groups, int dense_rows, int total_rows) -> hipError_t {
            if (!weight_grad_shape_ok(M, N, abf)) return hipSuccess;
            return launch_weight_grad(nullptr, M, nullptr, N, counts, offsets, groups, dense_rows, total_rows, L->wgrad_split,
                                      L->grads_clear, (int*)L->wg_chunks.p + (size_t)which * wgrad_table_ints(L),
                                      (float*)L->wg_partial.p, L->wg_partial.bytes, nullptr, 0, abf, rs, WgradPart::TableOnly);
        };
        HIP_TRY(ctx, table(0, d, F, E, -1, S));
        HIP_TRY(ctx, table(1, 2 * F, d, E, -1, S));
        if (c.shared_expert) {
            HIP_TRY(ctx, table(2, d, Fs, 1, T, T));
            HIP_TRY(ctx, table(3, 2 * Fs, d, 1, T, T));
        }
        HIP_TRY(ctx, hipEventRecord(ctx->ev_tables, rs));
    }
    HIP_TRY(ctx, launch_route_backward((const float*)L->P.p, (const float*)L->lse.p, (const int*)L->expert_of.p,
                                       (const float*)L->grad_gates.p, counts, offsets, T, E, k, c.aux_loss_weight,
                                       c.router_z_loss_weight, (float*)L->dlogits.p, rs));
    HIP_TRY(ctx, launch_router_grad((const float*)L->dlogits.p, L->xc.p, (const float*)L->router.p, T, d, E,
                                    (float*)L->rpartial.p, (float*)L->g_router.p, L->dxr.p, xbf, rs));

    // SwiGlu::backward over the routed rows (src/ffn.rs:87-120)
    GroupedArgs g{};
    g.tile_expert = (const int*)L->tile_expert.p;
    g.tile_row0 = (const int*)L->tile_row0.p;
    g.tile_rows = (const int*)L->tile_rows.p;
    g.ntiles = (const int*)L->ntiles.p;
    g.max_tiles = S / L->last_tile_m + E;  // the tile table of the last forward
    g.tile_m = L->last_tile_m;
    g.dense_rows = -1;
    g.swiglu = false;
    g.group_m = L->group_m;
    GroupedArgs gh = g;  // grad_hidden = dY . Wdown
    gh.a = L->dy.p; gh.w = L->wdT.p; gh.w_expert_stride = (size_t)F * d; gh.N = F; gh.K = d;
    gh.swiglu_grad_gu = L->gu.p; gh.gu_out = L->dgu.p;  // the hidden gradient goes straight through SwiGLU's backward
    const WeightKind wk = c.weight_dtype == RBMOE_F32 ? WeightKind::F32 : WeightKind::BF16;
    auto prod_on = [&](const GroupedArgs& a, hipStream_t st) -> hipError_t {
        if (L->use_stream) return launch_grouped_stream(a, WeightKind::BF16, st);
        if (L->use_f32_mc) return launch_grouped_f32(a, st);
        return launch_grouped_generic(a, abf, wk, kGenericTileM, st);
    };
    auto prod = [&](const GroupedArgs& a) -> hipError_t { return prod_on(a, s); };
    HIP_TRY(ctx, prod(gh));
    GroupedArgs gx = g;  // grad_input rows = dG . Wgate + dU . Wup
    gx.a = L->dgu.p; gx.w = L->wguT.p; gx.w_expert_stride = (size_t)d * 2 * F; gx.N = d; gx.K = 2 * F; gx.out = L->dxg.p;
    if (side) {
        // the input-gradient product follows the router's branch on the side stream, beside the weight gradients
        // (it needs dG | dU, which the launch above has just written)
        HIP_TRY(ctx, hipEventRecord(ctx->ev_fork2, s));
        HIP_TRY(ctx, hipStreamWaitEvent(rs, ctx->ev_fork2, 0));
        HIP_TRY(ctx, prod_on(gx, rs));
        // without a shared expert everything the final sum reads is written on the side stream: it runs there too,
        // beside the weight gradients
        if (combine_on_side) HIP_TRY(ctx, launch_combine(ca, xbf, rs));
        HIP_TRY(ctx, hipEventRecord(ctx->ev_join, rs));
    } else {
        HIP_TRY(ctx, prod(gx));
    }
    // weight gradients (src/param.rs:819-821): down += dY^T . H; (gate | up) += (dG | dU)^T . X[token]
    auto wgrad = [&](int table, const void* a, int M, const void* b, const int* b_rows, int N, int groups,
                     int dense_rows, int total_rows, float* out, size_t stride) -> hipError_t {
        if (!L->wgrad_generic && !b_rows && weight_grad_shape_ok(M, N, abf))
            return launch_weight_grad(a, M, b, N, counts, offsets, groups, dense_rows, total_rows,
                                      L->wgrad_split, L->grads_clear, (int*)L->wg_chunks.p + (size_t)table * wgrad_table_ints(L),
                                      (float*)L->wg_partial.p, L->wg_partial.bytes, out, stride, abf, s,
                                      tables_early ? WgradPart::ProductOnly : WgradPart::Both);
        if (L->grads_clear) {
            const hipError_t e = launch_fill_f32(out, 0.0f, (long long)((size_t)groups * (stride ? stride : (size_t)M * N)), s);
            if (e != hipSuccess) return e;
        }
        return launch_grouped_tn(a, M, b, b_rows, N, counts, offsets, groups, dense_rows, out, stride, abf, s);
    };
    if (tables_early) HIP_TRY(ctx, hipStreamWaitEvent(s, ctx->ev_tables, 0));
    HIP_TRY(ctx, wgrad(0, L->dy.p, d, L->h.p, nullptr, F, E, -1, S, (float*)L->g_down.p, (size_t)d * F));
    HIP_TRY(ctx, wgrad(1, L->dgu.p, 2 * F, L->xg.p, nullptr, d, E, -1, S, (float*)L->g_gu.p, (size_t)2 * F * d));
    // shared expert over every row (src/moe.rs:356-361)
    if (c.shared_expert) {
        GroupedArgs sh = g;
        sh.dense_rows = T;
        sh.a = gout; sh.w = L->swdT.p; sh.w_expert_stride = 0; sh.N = Fs; sh.K = d;
        sh.swiglu_grad_gu = L->gus.p; sh.gu_out = L->dgus.p;
        HIP_TRY(ctx, prod(sh));
        GroupedArgs sx = g;
        sx.dense_rows = T; sx.w_expert_stride = 0;
        sx.a = L->dgus.p; sx.w = L->swguT.p; sx.N = d; sx.K = 2 * Fs; sx.out = L->dxs.p;
        HIP_TRY(ctx, prod(sx));
        HIP_TRY(ctx, wgrad(2, gout, d, L->hs.p, nullptr, Fs, 1, T, T, (float*)L->g_sdown.p, 0));
        HIP_TRY(ctx, wgrad(3, L->dgus.p, 2 * Fs, cast ? L->x16.p : L->xc.p, nullptr, d, 1, T, T, (float*)L->g_sgu.p, 0));
    }
    // grad_input = sum over a token's slots of its expert rows + shared + router
    if (side) HIP_TRY(ctx, hipStreamWaitEvent(s, ctx->ev_join, 0));
    return RBMOE_OK;
    };
    const int rc = forked();
    if (rc != RBMOE_OK) {
        if (side) {  // rejoin whatever the side stream got to
            (void)hipEventRecord(ctx->ev_join, rs);
            (void)hipStreamWaitEvent(s, ctx->ev_join, 0);
        }
        return rc;
    }
    if (!combine_on_side) HIP_TRY(ctx, launch_combine(ca, xbf, s));
    L->grads_clear = false;
    return RBMOE_OK;
}

int rbmoe_backward_host(rbmoe_layer* L, const void* grad_output, int32_t tokens, int32_t cols, void* grad_input) {
    if (!L) return fail(nullptr, RBMOE_NULL_POINTER, "layer is NULL");
    rbmoe_ctx* ctx = L->ctx;
    if (!L->training) return fail(ctx, RBMOE_INVALID_CONFIG, "training is not enabled on this layer");
    if (L->last_T < 0) return fail(ctx, RBMOE_INVALID_INPUT, "no forward pass has run yet");
    if (const int rc = backward_shape_problem(L, tokens, cols)) return rc;  // before any byte of the buffers is touched
    const int T = L->last_T;
    if (T == 0) return RBMOE_OK;
    if (!grad_output || !grad_input) return fail(ctx, RBMOE_NULL_POINTER, "grad_output or grad_input is NULL");
    const size_t nbytes = (size_t)T * L->cfg.d_model * dtype_size(L->cfg.act_dtype);
    HIP_TRY(ctx, hipSetDevice(ctx->device));
    HIP_TRY(ctx, hipMemcpyAsync(L->st_gout.p, grad_output, nbytes, hipMemcpyHostToDevice, ctx->stream));
    int rc = rbmoe_backward(L, L->st_gout.p, tokens, cols, L->st_gin.p);
    if (rc != RBMOE_OK) return rc;
    HIP_TRY(ctx, hipMemcpyAsync(grad_input, L->st_gin.p, nbytes, hipMemcpyDeviceToHost, ctx->stream));
    HIP_TRY(ctx, hipStreamSynchronize(ctx->stream));
    return RBMOE_OK;
}

int rbmoe_backward_block(rbmoe_layer* L, const void* grad_output, int32_t tokens, int32_t cols, void* grad_input) {
    if (!L) return fail(nullptr, RBMOE_NULL_POINTER, "layer is NULL");
    rbmoe_ctx* ctx = L->ctx;
    if (!L->training) return fail(ctx, RBMOE_INVALID_CONFIG, "training is not enabled on this layer");
    if (!L->norm_set) return fail(ctx, RBMOE_INVALID_CONFIG, "the feed-forward norm has not been set");
    if (L->last_T < 0 || !L->last_was_block)
        return fail(ctx, RBMOE_INVALID_INPUT, "the last forward pass was not rbmoe_forward_block");
    if (const int rc = backward_shape_problem(L, tokens, cols)) return rc;
    const int T = L->last_T, d = L->cfg.d_model;
    if (T == 0) return RBMOE_OK;
    if (!grad_output || !grad_input) return fail(ctx, RBMOE_NULL_POINTER, "grad_output or grad_input is NULL");
    // grad_projected = feed_forward.backward(cache, grad_output)  (src/transformer_block.rs:257)
    const int rc = rbmoe_backward(L, grad_output, tokens, cols, L->dxn.p);
    if (rc != RBMOE_OK) return rc;
    // grad_residual = feed_forward_norm.backward(residual, grad_projected) + grad_output  (:258-263)
    HIP_TRY(ctx, launch_rmsnorm_backward(L->xraw.p, L->dxn.p, (const float*)L->norm_w.p, L->norm_eps, grad_output, T, d,
                                         grad_input, (float*)L->inv_rms.p, (float*)L->norm_partial.p,
                                         (float*)L->g_norm.p, L->cfg.act_dtype == RBMOE_BF16, ctx->stream));
    return RBMOE_OK;
}

int rbmoe_backward_block_host(rbmoe_layer* L, const void* grad_output, int32_t tokens, int32_t cols,
                              void* grad_input) {
    if (!L) return fail(nullptr, RBMOE_NULL_POINTER, "layer is NULL");
    rbmoe_ctx* ctx = L->ctx;
    if (!L->training) return fail(ctx, RBMOE_INVALID_CONFIG, "training is not enabled on this layer");
    if (!L->norm_set) return fail(ctx, RBMOE_INVALID_CONFIG, "the feed-forward norm has not been set");
    if (L->last_T < 0 || !L->last_was_block)
        return fail(ctx, RBMOE_INVALID_INPUT, "the last forward pass was not rbmoe_forward_block");
    if (const int rc = backward_shape_problem(L, tokens, cols)) return rc;  // before any byte of the buffers is touched
    const int T = L->last_T;
    if (T == 0) return RBMOE_OK;
    if (!grad_output || !grad_input) return fail(ctx, RBMOE_NULL_POINTER, "grad_output or grad_input is NULL");
    const size_t nbytes = (size_t)T * L->cfg.d_model * dtype_size(L->cfg.act_dtype);
    HIP_TRY(ctx, hipSetDevice(ctx->device));
    HIP_TRY(ctx, hipMemcpyAsync(L->st_gout.p, grad_output, nbytes, hipMemcpyHostToDevice, ctx->stream));
    const int rc = rbmoe_backward_block(L, L->st_gout.p, tokens, cols, L->st_gin.p);
    if (rc != RBMOE_OK) return rc;
    HIP_TRY(ctx, hipMemcpyAsync(grad_input, L->st_gin.p, nbytes, hipMemcpyDeviceToHost, ctx->stream));
    HIP_TRY(ctx, hipStreamSynchronize(ctx->stream));
    return RBMOE_OK;
}

int rbmoe_get_weight_grad(rbmoe_layer* L, int32_t which, int32_t expert, float* host, int32_t rows, int32_t cols) {
    if (!L) return fail(nullptr, RBMOE_NULL_POINTER, "layer is NULL");
    rbmoe_ctx* ctx = L->ctx;
    if (!L->training) return fail(ctx, RBMOE_INVALID_CONFIG, "training is not enabled on this layer");
    if (!host) return fail(ctx, RBMOE_NULL_POINTER, "host buffer is NULL");
    const rbmoe_config& c = L->cfg;
    const size_t E = c.num_experts, d = c.d_model, F = c.d_ff, Fs = L->Fs;
    const float* src = nullptr;
    size_t want_rows = 0, want_cols = 0;
    const bool bad_expert = expert < 0 || (size_t)expert >= E;
    switch (which) {
        case RBMOE_W_ROUTER: src = (const float*)L->g_router.p; want_rows = E; want_cols = d; break;
        case RBMOE_W_GATE:
        case RBMOE_W_UP:
            if (bad_expert) return fail(ctx, RBMOE_INVALID_CONFIG, "expert index out of range");
            src = (const float*)L->g_gu.p + ((size_t)expert * 2 + (which == RBMOE_W_UP ? 1 : 0)) * F * d;
            want_rows = F; want_cols = d;
            break;
        case RBMOE_W_DOWN:
            if (bad_expert) return fail(ctx, RBMOE_INVALID_CONFIG, "expert index out of range");
            src = (const float*)L->g_down.p + (size_t)expert * d * F;
            want_rows = d; want_cols = F;
            break;
        case RBMOE_W_SHARED_GATE:
        case RBMOE_W_SHARED_UP:
            if (!c.shared_expert) return fail(ctx, RBMOE_INVALID_CONFIG, "the layer has no shared expert");
            src = (const float*)L->g_sgu.p + (size_t)(which == RBMOE_W_SHARED_UP ? 1 : 0) * Fs * d;
            want_rows = Fs; want_cols = d;
            break;
        case RBMOE_W_SHARED_DOWN:
            if (!c.shared_expert) return fail(ctx, RBMOE_INVALID_CONFIG, "the layer has no shared expert");
            src = (const float*)L->g_sdown.p;
            want_rows = d; want_cols = Fs;
            break;
        case RBMOE_W_NORM:
            if (!L->g_norm.p) return fail(ctx, RBMOE_INVALID_CONFIG, "the feed-forward norm has not been set");
            src = (const float*)L->g_norm.p;
            want_rows = 1; want_cols = d;
            break;
        default:
            return fail(ctx, RBMOE_INVALID_CONFIG, "unknown weight id");
    }
    if ((size_t)rows != want_rows || (size_t)cols != want_cols)
        return fail(ctx, RBMOE_INVALID_INPUT, "gradient shape does not match the weight");
    if (L->grads_clear && which != RBMOE_W_ROUTER && which != RBMOE_W_NORM) {  // cleared and not written since
        std::memset(host, 0, want_rows * want_cols * 4);
        return RBMOE_OK;
    }
    HIP_TRY(ctx, hipStreamSynchronize(ctx->stream));
    HIP_TRY(ctx, hipMemcpy(host, src, want_rows * want_cols * 4, hipMemcpyDeviceToHost));
    return RBMOE_OK;
}

int rbmoe_get_losses(rbmoe_layer* L, float* aux_loss, float* z_loss) {
    if (!L) return fail(nullptr, RBMOE_NULL_POINTER, "layer is NULL");
    rbmoe_ctx* ctx = L->ctx;
    if (L->last_T < 0) return fail(ctx, RBMOE_INVALID_INPUT, "no forward pass has run yet");
    float v[2] = {0.f, 0.f};
    HIP_TRY(ctx, hipStreamSynchronize(ctx->stream));
    HIP_TRY(ctx, hipMemcpy(v, L->last.losses, 8, hipMemcpyDeviceToHost));
    if (aux_loss) *aux_loss = v[0];
    if (z_loss) *z_loss = v[1];
    return RBMOE_OK;
}

int rbmoe_get_routing(rbmoe_layer* L, rbmoe_routing* r) {
    if (!L || !r) return fail(L ? L->ctx : nullptr, RBMOE_NULL_POINTER, "layer or routing is NULL");
    rbmoe_ctx* ctx = L->ctx;
    if (L->last_T < 0) return fail(ctx, RBMOE_INVALID_INPUT, "no forward pass has run yet");
    const int T = L->last_T, E = L->cfg.num_experts, k = L->cfg.experts_per_token;
    const size_t S = (size_t)T * k;
    HIP_TRY(ctx, hipStreamSynchronize(ctx->stream));
    const Work& w = L->last;
    if (r->counts) HIP_TRY(ctx, hipMemcpy(r->counts, w.counts, (size_t)E * 4, hipMemcpyDeviceToHost));
    if (r->offsets) HIP_TRY(ctx, hipMemcpy(r->offsets, w.offsets, (size_t)(E + 1) * 4, hipMemcpyDeviceToHost));
    if (S == 0) return RBMOE_OK;
    if (r->expert_of) HIP_TRY(ctx, hipMemcpy(r->expert_of, w.expert_of, S * 4, hipMemcpyDeviceToHost));
    if (r->gate_of) HIP_TRY(ctx, hipMemcpy(r->gate_of, w.gate_of, S * 4, hipMemcpyDeviceToHost));
    if (r->perm_slot) HIP_TRY(ctx, hipMemcpy(r->perm_slot, w.perm_slot, S * 4, hipMemcpyDeviceToHost));
    if (r->perm_token) HIP_TRY(ctx, hipMemcpy(r->perm_token, w.perm_token, S * 4, hipMemcpyDeviceToHost));
    if (r->probabilities)
        HIP_TRY(ctx, hipMemcpy(r->probabilities, w.P, (size_t)T * E * 4, hipMemcpyDeviceToHost));
    if (r->log_sum_exp) HIP_TRY(ctx, hipMemcpy(r->log_sum_exp, w.lse, (size_t)T * 4, hipMemcpyDeviceToHost));
    return RBMOE_OK;
}

int rbmoe_get_expert_rows(rbmoe_layer* L, float* hidden, float* expert_out) {
    if (!L) return fail(nullptr, RBMOE_NULL_POINTER, "layer is NULL");
    rbmoe_ctx* ctx = L->ctx;
    if (L->last_T < 0) return fail(ctx, RBMOE_INVALID_INPUT, "no forward pass has run yet");
    const int E = L->cfg.num_experts, d = L->cfg.d_model, F = L->cfg.d_ff;
    HIP_TRY(ctx, hipStreamSynchronize(ctx->stream));
    int R = 0;
    HIP_TRY(ctx, hipMemcpy(&R, L->last.offsets + E, 4, hipMemcpyDeviceToHost));
    const bool abf = L->cfg.act_dtype == RBMOE_BF16 || L->cast_rows;  // the rows of a cast_rows layer are bf16
    auto fetch = [&](float* dst, const void* src, size_t n) -> int {
        if (!dst || n == 0) return RBMOE_OK;
        if (!abf) {
            HIP_TRY(ctx, hipMemcpy(dst, src, n * 4, hipMemcpyDeviceToHost));
            return RBMOE_OK;
        }
        std::vector<uint16_t> tmp(n);
        HIP_TRY(ctx, hipMemcpy(tmp.data(), src, n * 2, hipMemcpyDeviceToHost));
        for (size_t i = 0; i < n; ++i) dst[i] = host_bf16_to_f32(tmp[i]);
        return RBMOE_OK;
    };
    int rc = RBMOE_OK;
    if (L->last_front && hidden && R > 0) {
        // the hidden rows lie per expert over all the call's rows: pick the routed ones, in permuted order
        const int T = L->last_T;
        std::vector<float> all((size_t)E * T * F);
        std::vector<int> offs(E + 1), ptok(R);
        rc = fetch(all.data(), L->last.hall, all.size());
        if (rc != RBMOE_OK) return rc;
        HIP_TRY(ctx, hipMemcpy(offs.data(), L->last.offsets, (size_t)(E + 1) * 4, hipMemcpyDeviceToHost));
        HIP_TRY(ctx, hipMemcpy(ptok.data(), L->last.perm_token, (size_t)R * 4, hipMemcpyDeviceToHost));
        for (int e = 0; e < E; ++e)
            for (int pos = offs[e]; pos < offs[e + 1]; ++pos)
                std::memcpy(hidden + (size_t)pos * F, all.data() + ((size_t)e * T + ptok[pos]) * F, (size_t)F * 4);
    } else {
        rc = fetch(hidden, L->last.h, (size_t)R * F);
    }
    if (rc != RBMOE_OK) return rc;
    return fetch(expert_out, L->last.y, (size_t)R * d);
}

const char* rbmoe_expert_kernel_name(const rbmoe_layer* L) { return L ? L->kernel_name : "none"; }

int rbmoe_device_alloc(rbmoe_ctx* ctx, size_t bytes, void** out) {
    if (!ctx || !out) return fail(ctx, RBMOE_NULL_POINTER, "ctx or out is NULL");
    HIP_TRY(ctx, hipSetDevice(ctx->device));
    HIP_TRY(ctx, hipMalloc(out, bytes ? bytes : 1));
    return RBMOE_OK;
}

int rbmoe_device_free(rbmoe_ctx* ctx, void* ptr) {
    if (!ctx) return fail(nullptr, RBMOE_NULL_POINTER, "ctx is NULL");
    if (ptr) HIP_TRY(ctx, hipFree(ptr));
    return RBMOE_OK;
}

int rbmoe_copy_to_device(rbmoe_ctx* ctx, void* dst, const void* src, size_t bytes) {
    if (!ctx) return fail(nullptr, RBMOE_NULL_POINTER, "ctx is NULL");
    if (bytes == 0) return RBMOE_OK;
    if (!dst || !src) return fail(ctx, RBMOE_NULL_POINTER, "dst or src is NULL");
    HIP_TRY(ctx, hipMemcpyAsync(dst, src, bytes, hipMemcpyHostToDevice, ctx->stream));
    HIP_TRY(ctx, hipStreamSynchronize(ctx->stream));
    return RBMOE_OK;
}

int rbmoe_copy_to_host(rbmoe_ctx* ctx, void* dst, const void* src, size_t bytes) {
    if (!ctx) return fail(nullptr, RBMOE_NULL_POINTER, "ctx is NULL");
    if (bytes == 0) return RBMOE_OK;
    if (!dst || !src) return fail(ctx, RBMOE_NULL_POINTER, "dst or src is NULL");
    HIP_TRY(ctx, hipMemcpyAsync(dst, src, bytes, hipMemcpyDeviceToHost, ctx->stream));
    HIP_TRY(ctx, hipStreamSynchronize(ctx->stream));
    return RBMOE_OK;
}

// Test hook (not part of rbmoe.h): the partial matrices an ordered weight-gradient launch over `tokens` tokens cuts
// out, and how many a buffer sized for `max_tokens` holds.
int rbmoe_internal_weight_grad_slots(int32_t M, int32_t N, int32_t groups, int32_t dense, int32_t tokens,
                                     int32_t rows_per_token, int32_t bf16, int32_t max_tokens, int64_t* needed,
                                     int64_t* held) {
    if (!needed || !held) return RBMOE_NULL_POINTER;
    const size_t one = (size_t)M * N * sizeof(float);
    const int rows = dense ? tokens : tokens * rows_per_token;
    *needed = (int64_t)(weight_grad_partial_bytes(M, N, groups, dense ? rows : -1, rows, bf16 != 0) / one);
    *held = (int64_t)(weight_grad_partial_bytes_upto(M, N, groups, dense != 0, max_tokens, rows_per_token, bf16 != 0) / one);
    return RBMOE_OK;
}

int rbmoe_copy_device(rbmoe_ctx* ctx, void* dst, const void* src, size_t bytes) {
    if (!ctx) return fail(nullptr, RBMOE_NULL_POINTER, "ctx is NULL");
    if (bytes == 0) return RBMOE_OK;
    if (!dst || !src) return fail(ctx, RBMOE_NULL_POINTER, "dst or src is NULL");
    HIP_TRY(ctx, hipMemcpyAsync(dst, src, bytes, hipMemcpyDeviceToDevice, ctx->stream));
    HIP_TRY(ctx, hipStreamSynchronize(ctx->stream));
    return RBMOE_OK;
}

}  // extern "C"
