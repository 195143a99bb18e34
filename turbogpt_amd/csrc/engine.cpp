// Engine behind the tg_* C ABI: owns every device buffer, and runs the training step as a
// sequence of kernel launches on one HIP stream.  Host-side counterpart of the reference's
// cuda/runtime.cu + cuda/engine_state.cu (resource ownership, transfers, entry points) and of the
// op sequencing that its persistent kernel does on the device (cuda/trainer.cuh:103-125,
// cuda/model.cuh:8-99).  All arithmetic is in the tgk_* kernels; this file only sequences them.
#include "common.h"
#include "../../include/tg_model.h"
#include "../../include/tgk_kernels.h"
#include <algorithm>
#include <climits>
#include <cmath>
#include <cstring>
#include <vector>

namespace {

constexpr int MaxLaunchSteps = 4096; // cuda/types.cuh:10
constexpr int NormPartials = 1024;
constexpr int MaxInFlight = 16; // batches in flight, each with its own stream and saved activations

struct LayerBuffers {
    bf16_t *n1, *qkv, *o, *mid, *n2, *u, *a;
    float *lse;
};

void ok(int status) {
    if (status < 0)
        throw std::runtime_error(tg_last_error);
}
// one operator launch, attributed to a TG_CLASS_* for tg_profile_step
#define OP(cls, call)                 \
    do {                              \
        Scope profile_scope(this, cls); \
        ok(call);                     \
    } while (0)

// optim.h:18-44
StepRates onecycle_point(const OneCycle &s, int step) {
    if (s.total_steps < 1 || step < 0 || step >= s.total_steps ||
        !(s.warmup_fraction > 0 && s.warmup_fraction < 1) ||
        !(s.initial_lr_fraction > 0 && s.initial_lr_fraction < 1) ||
        !(s.final_lr_fraction > 0 && s.final_lr_fraction <= s.initial_lr_fraction) ||
        !(s.low_momentum >= 0 && s.low_momentum < 1) ||
        !(s.high_momentum >= s.low_momentum && s.high_momentum < 1))
        throw std::runtime_error("Invalid OneCycle schedule or step");
    const double warmup_steps = s.warmup_fraction * s.total_steps - 1;
    if (warmup_steps == 0)
        throw std::runtime_error("OneCycle warmup must span at least two steps");
    const bool warming = step <= warmup_steps;
    const double fraction =
        warming ? step / warmup_steps : (step - warmup_steps) / (s.total_steps - 1 - warmup_steps);
    const double c = 0.5 * (1 + std::cos(3.14159265358979323846 * fraction));
    const auto between = [c](double from, double to) { return to + (from - to) * c; };
    return {float(warming ? between(s.initial_lr_fraction, 1.0) : between(1.0, s.final_lr_fraction)),
            float(warming ? between(s.high_momentum, s.low_momentum)
                          : between(s.low_momentum, s.high_momentum))};
}

} // namespace

// Everything one batch in flight owns: its stream, its tokens, its saved activations and its gradient.
// A synchronous engine has one slot on the engine's stream; inflight = K gives K slots on K streams
// (the worker teams of cuda/pipeline.cuh:52-92).
struct Slot {
    hipStream_t stream = nullptr;
    hipEvent_t ready = nullptr; // the gradient of the slot's latest step is complete
    uint8_t *input = nullptr, *target = nullptr;
    float *token_losses = nullptr, *gradient = nullptr;
    std::vector<bf16_t *> x; // x[l] = input of block l; x[depth] = output of the last block
    std::vector<LayerBuffers> layers;
    bf16_t *nf = nullptr, *logits = nullptr, *dh = nullptr, *t1 = nullptr, *du = nullptr, *dqkv = nullptr;
    bf16_t *dh_mid = nullptr; // the gradient between a block's two halves, when the block's weight gradients are batched
    // When all weight gradients of a step go out as one launch behind the backward pass, every block keeps the four
    // output gradients that launch reads: g_x[l] = gradient of the loss by x[l] (g_x[l + 1] enters block l), g_mid[l]
    // by the block's middle, g_u[l] by the MLP pre-activation, g_qkv[l] by the packed projections.
    std::vector<bf16_t *> g_x, g_mid, g_u, g_qkv;
    std::vector<TgkWgradJob> wgrad_jobs;
    void *wgrad_table = nullptr;
    bf16_t *onehot = nullptr; // [tokens][256]: the token table's gradient is one more product of that launch
    // ... and the kernels that write the gradient leave the sums of its squares here (cuda/trainer.cuh:35-46): the
    // launch above for the matrices, one more small launch for the ranges in `norm_ranges` (every other tensor)
    float *norms = nullptr;
    int list_norms = 0, range_norms = 0;
    void *norm_ranges = nullptr;
    void *workspace = nullptr;
    // LayerNorm parameter gradients: every LayerNorm backward of a step leaves its per-block partial sums in a
    // block of its own here and one launch at the end of the backward pass folds all 2 * depth + 1 of them
    uint8_t *ln_partials = nullptr;
    void *ln_targets = nullptr; // device array of {dgamma, dbeta} pointers into `gradient`, in fold order
};
// One immutable copy of the weights: a batch reads a single version from its first kernel to its last
// (cuda/pipeline.cuh:36-38).  inflight = K keeps K + 1 of them in a ring; a synchronous engine one.
struct Version {
    uint16_t *hi = nullptr, *lo = nullptr;
    uint16_t *t = nullptr;     // every matrix of hi transposed ([In][Out]), same offsets (wide model only)
    hipEvent_t done = nullptr; // the optimizer step that wrote this version has finished
};

struct Engine {
    TgModelConfig config{};
    TgParameterLayout layout{};
    hipStream_t stream = nullptr;
    std::vector<void *> allocations;
    size_t allocated_bytes = 0;
    int compute_units = 0;
    bool width16 = false; // the reference's own network, created from the plain Config

    std::vector<Slot> slots;
    std::vector<Version> versions;
    void *transpose_jobs = nullptr;
    int transpose_count = 0, transpose_tiles = 0;
    float *momentum = nullptr, *variance = nullptr;
    float *norm_partials = nullptr, *loss_history = nullptr;
    int64_t *segment_starts = nullptr;
    uint8_t *segment_flags = nullptr;
    int segments = 0;
    uint8_t *data = nullptr;
    int64_t data_size = 0;
    float *logits_f32 = nullptr;
    size_t workspace_bytes = 0;
    bool batched_wgrad = false; // a block's four weight gradients in one launch (shapes permitting)
    bool list_wgrad = false;    // every weight gradient of a step in one launch (widths that are multiples of 256)

    std::vector<StepRates> schedule;
    uint64_t step = 0;
    uint64_t floor = 0; // oldest weight version that exists: the step at the last tg_set_weights / _set_optimizer_state
    int last_train_steps = 0;
    std::vector<int> version_trace; // weight version each step of the last tg_train read
    uint64_t total_staleness = 0;
    int max_staleness = 0;

    // optional per-class timing of one step (tg_profile_step): event pairs around every launch
    struct Span {
        int cls;
        hipEvent_t start, stop;
    };
    bool profiling = false;
    std::vector<Span> spans;
    std::vector<hipEvent_t> event_pool;
    hipEvent_t event() {
        if (event_pool.empty()) {
            hipEvent_t fresh;
            check_hip(hipEventCreate(&fresh));
            return fresh;
        }
        hipEvent_t pooled = event_pool.back();
        event_pool.pop_back();
        return pooled;
    }
    struct Scope {
        Engine *e;
        size_t index = 0;
        Scope(Engine *engine, int cls) : e(engine) { // profiling exists for synchronous engines: one stream
            if (!e->profiling)
                return;
            index = e->spans.size();
            e->spans.push_back({cls, e->event(), e->event()});
            check_hip(hipEventRecord(e->spans[index].start, e->stream));
        }
        ~Scope() {
            if (e->profiling)
                (void)hipEventRecord(e->spans[index].stop, e->stream);
        }
    };

    int tokens() const { return config.base.batch * config.base.context; }

    template <class T> void allocate(T *&ptr, size_t n, bool zero = true) { // cuda/engine_internal.h:17-27
        void *raw = nullptr;
        check_hip(hipMalloc(&raw, n * sizeof(T)), "allocation: ");
        ptr = static_cast<T *>(raw);
        allocations.push_back(raw);
        allocated_bytes += n * sizeof(T);
        if (zero)
            check_hip(hipMemsetAsync(raw, 0, n * sizeof(T), stream));
    }
    void use_device() const { check_hip(hipSetDevice(config.base.device)); }
    void sync() const { // every stream: the engine is quiescent afterwards
        for (const Slot &slot : slots)
            if (slot.stream && slot.stream != stream)
                check_hip(hipStreamSynchronize(slot.stream));
        check_hip(hipStreamSynchronize(stream));
    }
    Version &current() { return versions[step % versions.size()]; }
    template <class T> void upload(T *device, const T *host, size_t n) {
        check_hip(hipMemcpyAsync(device, host, n * sizeof(T), hipMemcpyHostToDevice, stream));
    }
    template <class T> void download(T *host, const T *device, size_t n) {
        check_hip(hipMemcpyAsync(host, device, n * sizeof(T), hipMemcpyDeviceToHost, stream));
    }
    ~Engine() { // cuda/engine_internal.h:28-37
        (void)hipSetDevice(config.base.device);
        for (Slot &slot : slots)
            if (slot.stream && slot.stream != stream)
                (void)hipStreamSynchronize(slot.stream);
        if (stream)
            (void)hipStreamSynchronize(stream);
        for (void *allocation : allocations)
            (void)hipFree(allocation);
        for (Slot &slot : slots) {
            if (slot.ready)
                (void)hipEventDestroy(slot.ready);
            if (slot.stream && slot.stream != stream)
                (void)hipStreamDestroy(slot.stream);
        }
        for (Version &version : versions)
            if (version.done)
                (void)hipEventDestroy(version.done);
        for (Span &span : spans) {
            (void)hipEventDestroy(span.start);
            (void)hipEventDestroy(span.stop);
        }
        for (hipEvent_t pooled : event_pool)
            (void)hipEventDestroy(pooled);
        if (stream)
            (void)hipStreamDestroy(stream);
    }

    // input gradients and the head's forward projection read the transposed weights: call after every change of a
    // version's hi half
    void refresh_transposed(const Version &v) {
        if (width16)
            return;
        ok(tgk_transpose_batch(stream, v.hi, v.t, transpose_jobs, transpose_count, transpose_tiles));
    }

    // cuda/model.cuh:8-59.  evaluate: logits stay logits; otherwise they are replaced by dlogits.
    // On the slot's stream, with one weight version, from the slot's tokens.
    void forward(Slot &s, const Version &v, bool with_gradient, float *logits_out) {
        const Config &c = config.base;
        hipStream_t stream = s.stream;
        const uint8_t *tokens_in = s.input, *targets = s.target;
        float *token_losses = s.token_losses;
        if (width16) {
            OP(TG_CLASS_OTHER, tgk_w16_forward(stream, c.depth, c.batch, c.context, v.hi, v.lo, tokens_in, targets,
                                               s.workspace, token_losses, logits_out, with_gradient ? 1 : 0));
            return;
        }
        const auto w = [&](int64_t offset) { return v.hi + offset; };
        const auto wl = [&](int64_t offset) { return v.lo + offset; };
        const auto wt = [&](int64_t offset) { return v.t + offset; };
        std::vector<bf16_t *> &x = s.x;
        std::vector<LayerBuffers> &layers = s.layers;
        bf16_t *nf = s.nf, *logits = s.logits;
        const int M = tokens(), d = config.d_model, F = config.ffn, V = config.vocab, T = c.context;
        const float scale = 1.0f / std::sqrt(float(d / config.heads));
        OP(TG_CLASS_OTHER, tgk_embed_fwd(stream, M, T, d, tokens_in, w(layout.embedding), w(layout.positions), x[0]));
        for (int l = 0; l < c.depth; ++l) {
            const TgLayerParameters &p = layout.layers[l];
            LayerBuffers &b = layers[l];
            OP(TG_CLASS_LAYERNORM_FWD, tgk_layernorm_fwd(stream, M, d, x[l], w(p.ln1_g), wl(p.ln1_g), w(p.ln1_b), wl(p.ln1_b), b.n1,
                                 config.ln_eps));
            OP(TG_CLASS_GEMM_FWD, tgk_gemm_fwd(stream, M, 3 * d, d, b.n1, d, w(p.qkv), d, b.qkv, 3 * d, nullptr, 0, nullptr, 0));
            OP(TG_CLASS_ATTN_FWD, tgk_attn_fwd(stream, c.batch, config.heads, T, d / config.heads, b.qkv, b.qkv + d, b.qkv + 2 * d,
                            3 * d, b.o, d, b.lse, scale));
            OP(TG_CLASS_GEMM_FWD, tgk_gemm_fwd(stream, M, d, d, b.o, d, w(p.attn_out), d, b.mid, d, x[l], d, nullptr, 0));
            OP(TG_CLASS_LAYERNORM_FWD, tgk_layernorm_fwd(stream, M, d, b.mid, w(p.ln2_g), wl(p.ln2_g), w(p.ln2_b), wl(p.ln2_b), b.n2,
                                 config.ln_eps));
            OP(TG_CLASS_GEMM_FWD_GELU, tgk_gemm_fwd(stream, M, F, d, b.n2, d, w(p.mlp_up), d, b.u, F, nullptr, 0, b.a, F));
            OP(TG_CLASS_GEMM_FWD, tgk_gemm_fwd(stream, M, d, F, b.a, F, w(p.mlp_down), F, x[l + 1], d, b.mid, d, nullptr, 0));
        }
        OP(TG_CLASS_LAYERNORM_FWD, tgk_layernorm_fwd(stream, M, d, x[c.depth], w(layout.lnf_g), wl(layout.lnf_g), w(layout.lnf_b),
                             wl(layout.lnf_b), nf, config.ln_eps));
        OP(TG_CLASS_HEAD, tgk_gemm_fwd_t(stream, M, V, d, nf, d, wt(layout.head), V, logits, V, nullptr, 0, nullptr, 0));
        OP(TG_CLASS_OTHER, tgk_cross_entropy(stream, M, V, logits, targets, token_losses, logits_out, 1.0f / float(M),
                             with_gradient ? 1 : 0));
    }

    // cuda/model.cuh:61-99.  Every element of `gradient` is overwritten: nothing needs zeroing.
    void backward(Slot &s, const Version &v) {
        const Config &c = config.base;
        hipStream_t stream = s.stream;
        const uint8_t *tokens_in = s.input;
        float *gradient = s.gradient;
        void *workspace = s.workspace;
        if (width16) {
            OP(TG_CLASS_OTHER, tgk_w16_backward(stream, c.depth, c.batch, c.context, v.hi, v.lo, tokens_in, workspace,
                                                gradient));
            return;
        }
        const auto w = [&](int64_t offset) { return v.hi + offset; };
        const auto wl = [&](int64_t offset) { return v.lo + offset; };
        const auto wt = [&](int64_t offset) { return v.t + offset; };
        std::vector<bf16_t *> &x = s.x;
        std::vector<LayerBuffers> &layers = s.layers;
        bf16_t *nf = s.nf, *logits = s.logits, *dh = s.dh, *t1 = s.t1, *du = s.du, *dqkv = s.dqkv;
        const int M = tokens(), d = config.d_model, F = config.ffn, V = config.vocab, T = c.context;
        const float scale = 1.0f / std::sqrt(float(d / config.heads));
        float *g = gradient;
        // LayerNorm j of the fold: 0 = final, 1 + 2 l = block l's second, 2 + 2 l = its first
        const size_t ln_stride = tgk_layernorm_bwd_workspace(M, d);
        const auto ln_rows = [&](int job, const bf16_t *input, const bf16_t *dy, int64_t gamma, const bf16_t *residual,
                                 bf16_t *dx) {
            return tgk_layernorm_bwd_rows(stream, M, d, input, dy, w(gamma), wl(gamma), residual, dx, config.ln_eps,
                                          s.ln_partials + size_t(job) * ln_stride, ln_stride);
        };
        if (list_wgrad) {
            // No weight gradient in the loop: every block leaves its output gradients in buffers of its own and one
            // launch at the end computes all 4 * depth + 2 products (the head's included - its operands are dlogits,
            // still in `logits`, and nf - and the token table's, one-hot^T times the gradient entering the first block).
            OP(TG_CLASS_HEAD, tgk_gemm_dgrad_t(stream, M, V, d, logits, V, wt(layout.head), V, t1, d, nullptr, 0));
            OP(TG_CLASS_LAYERNORM_BWD, ln_rows(0, x[c.depth], t1, layout.lnf_g, nullptr, s.g_x[c.depth]));
            for (int l = c.depth - 1; l >= 0; --l) {
                const TgLayerParameters &p = layout.layers[l];
                LayerBuffers &b = layers[l];
                bf16_t *in = s.g_x[l + 1], *mid = s.g_mid[l], *gu = s.g_u[l], *gqkv = s.g_qkv[l];
                OP(TG_CLASS_GEMM_DGRAD_GELU, tgk_gemm_dgrad_t(stream, M, d, F, in, d, wt(p.mlp_down), d, gu, F, b.u, F));
                OP(TG_CLASS_GEMM_DGRAD, tgk_gemm_dgrad_t(stream, M, F, d, gu, F, wt(p.mlp_up), F, t1, d, nullptr, 0));
                OP(TG_CLASS_LAYERNORM_BWD, ln_rows(1 + 2 * l, b.mid, t1, p.ln2_g, in, mid));
                OP(TG_CLASS_GEMM_DGRAD, tgk_gemm_dgrad_t(stream, M, d, d, mid, d, wt(p.attn_out), d, t1, d, nullptr, 0));
                OP(TG_CLASS_ATTN_BWD, tgk_attn_bwd(stream, c.batch, config.heads, T, d / config.heads, b.qkv, b.qkv + d,
                                                   b.qkv + 2 * d, 3 * d, b.o, d, b.lse, t1, d, gqkv, gqkv + d, gqkv + 2 * d,
                                                   3 * d, scale, workspace, workspace_bytes));
                OP(TG_CLASS_GEMM_DGRAD, tgk_gemm_dgrad_t(stream, M, 3 * d, d, gqkv, 3 * d, wt(p.qkv), 3 * d, t1, d, nullptr, 0));
                OP(TG_CLASS_LAYERNORM_BWD, ln_rows(2 + 2 * l, x[l], t1, p.ln1_g, mid, s.g_x[l]));
            }
            OP(TG_CLASS_LAYERNORM_BWD, tgk_layernorm_bwd_fold(stream, M, d, 2 * c.depth + 1, s.ln_partials, ln_stride, s.ln_targets, 0));
            OP(TG_CLASS_OTHER, tgk_embed_bwd_onehot(stream, c.batch, T, d, tokens_in, s.g_x[0], s.onehot, g + layout.positions, 0));
            const bool norms = c.clip > 0;
            OP(TG_CLASS_GEMM_WGRAD, tgk_gemm_wgrad_list(stream, M, int(s.wgrad_jobs.size()), s.wgrad_jobs.data(), s.wgrad_table, 0,
                                                        workspace, workspace_bytes, norms ? s.norms : nullptr));
            if (norms)
                OP(TG_CLASS_OPTIMIZER, tgk_sumsq_segments(stream, g, s.norm_ranges, s.range_norms, s.norms + s.list_norms));
            return;
        }
        OP(TG_CLASS_HEAD, tgk_gemm_wgrad(stream, M, V, d, logits, V, nf, d, g + layout.head, d, 0, workspace, workspace_bytes));
        OP(TG_CLASS_HEAD, tgk_gemm_dgrad_t(stream, M, V, d, logits, V, wt(layout.head), V, t1, d, nullptr, 0));
        OP(TG_CLASS_LAYERNORM_BWD, ln_rows(0, x[c.depth], t1, layout.lnf_g, nullptr, dh));
        for (int l = c.depth - 1; l >= 0; --l) {
            const TgLayerParameters &p = layout.layers[l];
            LayerBuffers &b = layers[l];
            if (batched_wgrad) {
                // The four weight gradients wait until all their operands exist (after the attention backward) and
                // go out as one launch; for that the gradient entering the block (dh) survives the block's first
                // half: LayerNorm 2 writes its sum with dh into dh_mid.
                bf16_t *mid = s.dh_mid;
                OP(TG_CLASS_GEMM_DGRAD_GELU, tgk_gemm_dgrad_t(stream, M, d, F, dh, d, wt(p.mlp_down), d, du, F, b.u, F));
                OP(TG_CLASS_GEMM_DGRAD, tgk_gemm_dgrad_t(stream, M, F, d, du, F, wt(p.mlp_up), F, t1, d, nullptr, 0));
                OP(TG_CLASS_LAYERNORM_BWD, ln_rows(1 + 2 * l, b.mid, t1, p.ln2_g, dh, mid));
                OP(TG_CLASS_GEMM_DGRAD, tgk_gemm_dgrad_t(stream, M, d, d, mid, d, wt(p.attn_out), d, t1, d, nullptr, 0));
                OP(TG_CLASS_ATTN_BWD, tgk_attn_bwd(stream, c.batch, config.heads, T, d / config.heads, b.qkv, b.qkv + d,
                                                   b.qkv + 2 * d, 3 * d, b.o, d, b.lse, t1, d, dqkv, dqkv + d, dqkv + 2 * d,
                                                   3 * d, scale, workspace, workspace_bytes));
                const TgkWgradJob jobs[4] = {{d, F, dh, d, b.a, F, g + p.mlp_down, F},
                                             {F, d, du, F, b.n2, d, g + p.mlp_up, d},
                                             {d, d, mid, d, b.o, d, g + p.attn_out, d},
                                             {3 * d, d, dqkv, 3 * d, b.n1, d, g + p.qkv, d}};
                OP(TG_CLASS_GEMM_WGRAD, tgk_gemm_wgrad_batch(stream, M, 4, jobs, 0, workspace, workspace_bytes));
                OP(TG_CLASS_GEMM_DGRAD, tgk_gemm_dgrad_t(stream, M, 3 * d, d, dqkv, 3 * d, wt(p.qkv), 3 * d, t1, d, nullptr, 0));
                OP(TG_CLASS_LAYERNORM_BWD, ln_rows(2 + 2 * l, x[l], t1, p.ln1_g, mid, dh));
                continue;
            }
            OP(TG_CLASS_GEMM_WGRAD, tgk_gemm_wgrad(stream, M, d, F, dh, d, b.a, F, g + p.mlp_down, F, 0, workspace, workspace_bytes));
            OP(TG_CLASS_GEMM_DGRAD_GELU, tgk_gemm_dgrad_t(stream, M, d, F, dh, d, wt(p.mlp_down), d, du, F, b.u, F));
            OP(TG_CLASS_GEMM_WGRAD, tgk_gemm_wgrad(stream, M, F, d, du, F, b.n2, d, g + p.mlp_up, d, 0, workspace, workspace_bytes));
            OP(TG_CLASS_GEMM_DGRAD, tgk_gemm_dgrad_t(stream, M, F, d, du, F, wt(p.mlp_up), F, t1, d, nullptr, 0));
            OP(TG_CLASS_LAYERNORM_BWD, ln_rows(1 + 2 * l, b.mid, t1, p.ln2_g, dh, dh));
            OP(TG_CLASS_GEMM_WGRAD, tgk_gemm_wgrad(stream, M, d, d, dh, d, b.o, d, g + p.attn_out, d, 0, workspace, workspace_bytes));
            OP(TG_CLASS_GEMM_DGRAD, tgk_gemm_dgrad_t(stream, M, d, d, dh, d, wt(p.attn_out), d, t1, d, nullptr, 0));
            OP(TG_CLASS_ATTN_BWD, tgk_attn_bwd(stream, c.batch, config.heads, T, d / config.heads, b.qkv, b.qkv + d, b.qkv + 2 * d,
                            3 * d, b.o, d, b.lse, t1, d, dqkv, dqkv + d, dqkv + 2 * d, 3 * d, scale, workspace,
                            workspace_bytes));
            OP(TG_CLASS_GEMM_WGRAD, tgk_gemm_wgrad(stream, M, 3 * d, d, dqkv, 3 * d, b.n1, d, g + p.qkv, d, 0, workspace,
                              workspace_bytes));
            OP(TG_CLASS_GEMM_DGRAD, tgk_gemm_dgrad_t(stream, M, 3 * d, d, dqkv, 3 * d, wt(p.qkv), 3 * d, t1, d, nullptr, 0));
            OP(TG_CLASS_LAYERNORM_BWD, ln_rows(2 + 2 * l, x[l], t1, p.ln1_g, dh, dh));
        }
        OP(TG_CLASS_LAYERNORM_BWD, tgk_layernorm_bwd_fold(stream, M, d, 2 * c.depth + 1, s.ln_partials, ln_stride, s.ln_targets, 0));
        OP(TG_CLASS_OTHER, tgk_embed_bwd(stream, c.batch, T, d, V, tokens_in, dh, g + layout.embedding, g + layout.positions, 0,
                                         workspace, workspace_bytes));
    }

    // cuda/optim.cuh:66-106 for optimizer step `at` (0-based), on the engine's stream: gradient -> the weights of
    // version `to` (which already hold the previous version's values)
    // `from`: the slot whose backward pass has just written `gradient`, when it left the sums of squares with it
    void optimize(uint64_t at, const float *gradient, Version &to, const Slot *from = nullptr) {
        const Config &c = config.base;
        uint16_t *weight_hi = to.hi, *weight_lo = to.lo, *weight_t = to.t;
        float lr = c.learning_rate, beta1 = c.beta1, muon_lr = c.muon_lr, muon_momentum = c.momentum;
        if (!schedule.empty()) { // cuda/optim.cuh:81-88: one point drives both learning rates and both momenta
            lr *= schedule[at].multiplier;
            muon_lr *= schedule[at].multiplier;
            beta1 = muon_momentum = schedule[at].momentum;
        }
        const bool fused = from && from->norms && list_wgrad;
        if (c.clip > 0 && !fused)
            OP(TG_CLASS_OPTIMIZER, tgk_sumsq_partials(stream, gradient, size_t(layout.count), norm_partials, NormPartials));
        OP(TG_CLASS_OPTIMIZER, tgk_adamw(stream, size_t(layout.count), weight_hi, weight_lo, momentum, variance, gradient,
                     fused ? from->norms : norm_partials, fused ? from->list_norms + from->range_norms : NormPartials,
                     segment_starts, segment_flags, segments, lr, beta1, c.beta2, c.epsilon, c.weight_decay, c.clip, at));
        if (width16) { // the hidden matrices, which the AdamW segments skip (cuda/optim.cuh:107-118)
            OP(TG_CLASS_OPTIMIZER, tgk_w16_muon(stream, c.depth, weight_hi, weight_lo, momentum, gradient, norm_partials,
                                                NormPartials, c.clip, muon_lr, muon_momentum, c.weight_decay, c.ns_steps));
            return;
        }
        OP(TG_CLASS_OPTIMIZER, tgk_transpose_batch(stream, weight_hi, weight_t, transpose_jobs, transpose_count,
                                                   transpose_tiles));
    }
    // batch `at`: sample, forward, loss row, backward, on one slot with one weight version
    void batch_gradient(Slot &s, const Version &v, uint64_t at, float *history_row) {
        const Config &c = config.base;
        hipStream_t stream = s.stream;
        OP(TG_CLASS_OTHER, tgk_sample_batch(stream, data, data_size, c.seed, at, c.batch, c.context, s.input, s.target));
        forward(s, v, true, nullptr);
        OP(TG_CLASS_OTHER, tgk_position_means(stream, s.token_losses, c.batch, c.context, history_row));
        backward(s, v);
    }
    // One training step.  Synchronous engine: everything in order on the one stream, weights updated in place
    // (cuda/trainer.cuh:109-124).  inflight = K (cuda/pipeline.cuh:40-126 as streams and events): batch `at`
    // runs on slot at % K with the oldest version the ring still guarantees, max(floor, at - K + 1), so it
    // only waits for optimizer step at - K (which also freed the slot's gradient); the optimizer step waits for
    // the batch, copies version `at` into ring place at + 1 and updates it there.  The choice is made on the
    // host, so a run is reproducible; the staleness bound at - K + 1 <= version <= at is the reference's.
    void train_step(uint64_t at, float *history_row, int *trace) {
        const uint64_t K = slots.size(), ring = versions.size();
        if (K == 1) {
            batch_gradient(slots[0], versions[0], at, history_row);
            optimize(at, slots[0].gradient, versions[0], &slots[0]);
            *trace = int(at);
            return;
        }
        Slot &s = slots[at % K];
        const uint64_t read = std::max(floor, at + 1 >= K ? at + 1 - K : 0);
        check_hip(hipStreamWaitEvent(s.stream, versions[read % ring].done, 0));
        batch_gradient(s, versions[read % ring], at, history_row);
        check_hip(hipEventRecord(s.ready, s.stream));
        Version &from = versions[at % ring], &to = versions[(at + 1) % ring];
        check_hip(hipStreamWaitEvent(stream, s.ready, 0));
        const size_t bytes = size_t(layout.count) * 2;
        check_hip(hipMemcpyAsync(to.hi, from.hi, bytes, hipMemcpyDeviceToDevice, stream));
        check_hip(hipMemcpyAsync(to.lo, from.lo, bytes, hipMemcpyDeviceToDevice, stream));
        optimize(at, s.gradient, to, &s);
        check_hip(hipEventRecord(to.done, stream));
        *trace = int(read);
        total_staleness += at - read;
        max_staleness = std::max(max_staleness, int(at - read));
    }

    void read_losses(float *out) { // cuda/runtime.cu:279-290
        const Config &c = config.base;
        std::vector<float> losses(static_cast<size_t>(tokens()));
        download(losses.data(), slots[0].token_losses, losses.size());
        sync();
        for (int p = 0; p < c.context; ++p) {
            double sum = 0;
            for (int b = 0; b < c.batch; ++b)
                sum += losses[size_t(b) * c.context + p];
            out[p] = float(sum / c.batch);
        }
    }
};

namespace {

void validate(const TgModelConfig &m) {
    const Config &c = m.base;
    if (c.depth < 1 || c.depth > TG_MAX_DEPTH)
        throw std::runtime_error("Supported: depth 1..64");
    if (m.vocab != 256)
        throw std::runtime_error("Supported: vocabulary 256 (byte tokens)");
    if (m.d_model < 128 || m.d_model % 128 || m.d_model > 2048)
        throw std::runtime_error("Supported: d_model a multiple of 128, at most 2048");
    if (m.heads * 64 != m.d_model)
        throw std::runtime_error("Supported: head_dim 64 (heads = d_model / 64)");
    if (m.ffn < 128 || m.ffn % 128)
        throw std::runtime_error("Supported: ffn a multiple of 128");
    if (c.context < 128 || c.context % 128)
        throw std::runtime_error("Supported: context a multiple of 128");
    if (c.batch < 1 || int64_t(c.batch) * c.context > (int64_t(1) << 24))
        throw std::runtime_error("Supported: batch >= 1 with batch*context <= 2^24 tokens");
    if (c.inflight < 1 || c.inflight > MaxInFlight)
        throw std::runtime_error("inflight must be 1.." + std::to_string(MaxInFlight));
    if (!(m.ln_eps > 0))
        throw std::runtime_error("ln_eps must be positive");
}

// Streams, events and the buffers every model kind needs per slot and per weight version.
void build_slots(Engine *e, int inflight, bool transposed_copies) {
    const size_t P = size_t(e->layout.count), M = size_t(e->tokens());
    e->slots.resize(size_t(inflight));
    e->versions.resize(inflight > 1 ? size_t(inflight) + 1 : 1);
    for (Slot &slot : e->slots) {
        if (inflight > 1) {
            check_hip(hipStreamCreate(&slot.stream)); // default priority
            check_hip(hipEventCreateWithFlags(&slot.ready, hipEventDisableTiming));
        } else {
            slot.stream = e->stream;
        }
        e->allocate(slot.input, M);
        e->allocate(slot.target, M);
        e->allocate(slot.token_losses, M);
        e->allocate(slot.gradient, P);
    }
    for (Version &version : e->versions) {
        e->allocate(version.hi, P);
        e->allocate(version.lo, P);
        if (transposed_copies)
            e->allocate(version.t, P);
        if (inflight > 1)
            check_hip(hipEventCreateWithFlags(&version.done, hipEventDisableTiming));
    }
}

void build_transpose_jobs(Engine *e) {
    struct Job {
        int64_t offset;
        int rows, cols, first_tile, pad;
    };
    std::vector<Job> jobs;
    int tiles = 0;
    const auto add = [&](int64_t offset, int rows, int cols) {
        jobs.push_back({offset, rows, cols, tiles, 0});
        tiles += (rows / 64) * (cols / 64);
    };
    const TgParameterLayout &p = e->layout;
    const int d = e->config.d_model, F = e->config.ffn, V = e->config.vocab;
    for (int l = 0; l < e->config.base.depth; ++l) {
        const TgLayerParameters &b = p.layers[l];
        add(b.qkv, 3 * d, d);
        add(b.attn_out, d, d);
        add(b.mlp_up, F, d);
        add(b.mlp_down, d, F);
    }
    add(p.head, V, d);
    Job *device = nullptr;
    e->allocate(device, jobs.size(), false);
    e->upload(device, jobs.data(), jobs.size());
    e->sync();
    e->transpose_jobs = device;
    e->transpose_count = int(jobs.size());
    e->transpose_tiles = tiles;
}

void build_segments(Engine *e) {
    // weight-decay groups: block matrices and head decay, everything else does not
    std::vector<int64_t> starts;
    std::vector<uint8_t> flags;
    const auto add = [&](int64_t start, bool decay) {
        if (!flags.empty() && flags.back() == uint8_t(decay))
            return;
        starts.push_back(start);
        flags.push_back(uint8_t(decay));
    };
    const TgParameterLayout &p = e->layout;
    add(p.embedding, false);
    for (int l = 0; l < e->config.base.depth; ++l) {
        const TgLayerParameters &b = p.layers[l];
        add(b.ln1_g, false);
        add(b.qkv, true);
        add(b.ln2_g, false);
        add(b.mlp_up, true);
    }
    add(p.lnf_g, false);
    add(p.head, true);
    e->segments = int(starts.size());
    e->allocate(e->segment_starts, starts.size(), false);
    e->allocate(e->segment_flags, flags.size(), false);
    e->upload(e->segment_starts, starts.data(), starts.size());
    e->upload(e->segment_flags, flags.data(), flags.size());
    e->sync(); // the host vectors go out of scope
}

} // namespace

// cuda/runtime.cu:62-155: the reference's own width-16 network (config.h:4)
TG_API Engine *tg_create(const Config *c) {
    Engine *e = nullptr;
    try {
        if (!c)
            throw std::runtime_error("Missing configuration");
        if ((c->context != 4 && c->context != 8) || (c->depth != 4 && c->depth != 8) || c->batch < 4 ||
            c->batch * c->context % 16)
            throw std::runtime_error("Supported: depth 4/8, context 4/8, batch at least 4 with "
                                     "batch*context divisible by 16");
        if (c->inflight < 1 || c->inflight > MaxInFlight)
            throw std::runtime_error("inflight must be 1.." + std::to_string(MaxInFlight));
        if (c->inflight > 1 && c->blocks)
            throw std::runtime_error("model.blocks applies to synchronous training only");
        if (c->ns_steps < 1 || c->ns_steps > 10)
            throw std::runtime_error("ns_steps must be 1..10");
        int devices = 0;
        check_hip(hipGetDeviceCount(&devices), "device query: ");
        if (c->device < 0 || c->device >= devices)
            throw std::runtime_error("No such device");
        check_hip(hipSetDevice(c->device));
        hipDeviceProp_t prop{};
        check_hip(hipGetDeviceProperties(&prop, c->device));
        if (std::strncmp(prop.gcnArchName, "gfx950", 6) != 0)
            throw std::runtime_error(std::string("Requires an MI355X-class device (gfx950), found ") +
                                     prop.gcnArchName);
        e = new Engine;
        e->width16 = true;
        e->config.base = *c;
        e->config.d_model = 16, e->config.heads = 4, e->config.vocab = 256, e->config.ffn = 48;
        e->config.ln_eps = 1e-6f;
        e->layout.count = tgk_w16_parameter_count(c->depth);
        e->compute_units = prop.multiProcessorCount;
        check_hip(hipStreamCreate(&e->stream));
        const size_t P = size_t(e->layout.count);
        build_slots(e, c->inflight, false);
        e->allocate(e->momentum, P);
        e->allocate(e->variance, P);
        e->allocate(e->norm_partials, NormPartials);
        e->allocate(e->loss_history, size_t(MaxLaunchSteps) * c->context);
        // AdamW owns the embedding, the RMSNorm scales and the head (decayed); Muon the hidden matrices
        // (cuda/optim.cuh:5-15).  Flat order per layer (model.h:20-31): scale 16, qkv 768, attention 256, scale 16,
        // gate 768, up 768, down 768.
        std::vector<int64_t> starts;
        std::vector<uint8_t> flags;
        int64_t at = 0;
        const auto add = [&](int64_t size, uint8_t flag) {
            if (flags.empty() || flags.back() != flag) {
                starts.push_back(at);
                flags.push_back(flag);
            }
            at += size;
        };
        add(256 * 16, 0);
        for (int l = 0; l < c->depth; ++l) {
            add(16, 0);
            add(48 * 16 + 16 * 16, 2);
            add(16, 0);
            add(3 * 48 * 16, 2);
        }
        add(16, 0);
        add(256 * 16, 1);
        if (at != int64_t(P))
            throw std::runtime_error("internal: width-16 segment table does not cover the parameters");
        e->segments = int(starts.size());
        e->allocate(e->segment_starts, starts.size(), false);
        e->allocate(e->segment_flags, flags.size(), false);
        e->upload(e->segment_starts, starts.data(), starts.size());
        e->upload(e->segment_flags, flags.data(), flags.size());
        e->workspace_bytes = tgk_w16_workspace(c->depth, c->batch, c->context);
        for (Slot &slot : e->slots) {
            uint8_t *ws = nullptr;
            e->allocate(ws, e->workspace_bytes, false);
            slot.workspace = ws;
        }
        e->sync();
        return e;
    } catch (const std::exception &error) {
        tg_last_error = error.what();
        delete e;
        return nullptr;
    }
}

TG_API Engine *tg_create_ex(const TgModelConfig *model) {
    Engine *e = nullptr;
    try {
        if (!model)
            throw std::runtime_error("Missing configuration");
        validate(*model);
        int devices = 0;
        check_hip(hipGetDeviceCount(&devices), "device query: ");
        if (model->base.device < 0 || model->base.device >= devices)
            throw std::runtime_error("No such device");
        check_hip(hipSetDevice(model->base.device));
        hipDeviceProp_t prop{};
        check_hip(hipGetDeviceProperties(&prop, model->base.device));
        if (std::strncmp(prop.gcnArchName, "gfx950", 6) != 0)
            throw std::runtime_error(std::string("Requires an MI355X-class device (gfx950), found ") +
                                     prop.gcnArchName);
        e = new Engine;
        e->config = *model;
        e->layout = tg_parameter_layout(model);
        e->compute_units = prop.multiProcessorCount;
        if (e->layout.count > INT_MAX)
            throw std::runtime_error("Parameter count exceeds signed 32-bit indexing");
        check_hip(hipStreamCreate(&e->stream));

        const Config &c = model->base;
        const size_t P = size_t(e->layout.count), M = size_t(e->tokens()), d = size_t(model->d_model);
        const size_t F = size_t(model->ffn), V = size_t(model->vocab);
        build_slots(e, c.inflight, true);
        e->allocate(e->momentum, P);
        e->allocate(e->variance, P);
        e->allocate(e->norm_partials, NormPartials);
        e->allocate(e->loss_history, size_t(MaxLaunchSteps) * c.context);
        build_segments(e);
        build_transpose_jobs(e);
        for (Slot &slot : e->slots) {
            slot.x.resize(c.depth + 1);
            slot.layers.resize(c.depth);
            for (int l = 0; l <= c.depth; ++l)
                e->allocate(slot.x[l], M * d, false);
            for (int l = 0; l < c.depth; ++l) {
                LayerBuffers &b = slot.layers[l];
                e->allocate(b.n1, M * d, false);
                e->allocate(b.qkv, M * 3 * d, false);
                e->allocate(b.o, M * d, false);
                e->allocate(b.lse, size_t(c.batch) * model->heads * c.context, false);
                e->allocate(b.mid, M * d, false);
                e->allocate(b.n2, M * d, false);
                e->allocate(b.u, M * F, false);
                e->allocate(b.a, M * F, false);
            }
            e->allocate(slot.nf, M * d, false);
            e->allocate(slot.logits, M * V, false);
            e->allocate(slot.dh, M * d, false);
            e->allocate(slot.t1, M * d, false);
            e->allocate(slot.du, M * F, false);
            e->allocate(slot.dqkv, M * 3 * d, false);
        }
        const TgkWgradJob block_jobs[4] = {{int(d), int(F), nullptr, int(d), nullptr, int(F), nullptr, int(F)},
                                           {int(F), int(d), nullptr, int(F), nullptr, int(d), nullptr, int(d)},
                                           {int(d), int(d), nullptr, int(d), nullptr, int(d), nullptr, int(d)},
                                           {int(3 * d), int(d), nullptr, int(3 * d), nullptr, int(d), nullptr, int(d)}};
        size_t batch_need = tgk_gemm_wgrad_batch_workspace(int(M), 4, block_jobs);
        // One launch for all weight gradients where the shapes allow it (every width a multiple of 256)
        size_t table_bytes = 0;
        for (Slot &slot : e->slots) {
            std::vector<TgkWgradJob> &jobs = slot.wgrad_jobs;
            for (int l = 0; l < c.depth; ++l)
                for (int j = 0; j < 4; ++j)
                    jobs.push_back(block_jobs[j]);
            jobs.push_back({int(V), int(d), nullptr, int(V), nullptr, int(d), nullptr, int(d)}); // the head
            jobs.push_back({int(V), int(d), nullptr, int(V), nullptr, int(d), nullptr, int(d)}); // the token table
            table_bytes = tgk_gemm_wgrad_list_table_bytes(int(M), int(jobs.size()), jobs.data());
        }
        e->list_wgrad = table_bytes > 0;
        if (e->list_wgrad) {
            batch_need = 0;
            for (Slot &slot : e->slots) {
                slot.g_x.resize(c.depth + 1), slot.g_mid.resize(c.depth), slot.g_u.resize(c.depth), slot.g_qkv.resize(c.depth);
                for (int l = 0; l <= c.depth; ++l)
                    e->allocate(slot.g_x[l], M * d, false);
                for (int l = 0; l < c.depth; ++l) {
                    e->allocate(slot.g_mid[l], M * d, false);
                    e->allocate(slot.g_u[l], M * F, false);
                    e->allocate(slot.g_qkv[l], M * 3 * d, false);
                    const TgLayerParameters &p = e->layout.layers[l];
                    const LayerBuffers &b = slot.layers[l];
                    float *g = slot.gradient;
                    TgkWgradJob *jobs = slot.wgrad_jobs.data() + 4 * l;
                    jobs[0].dY = slot.g_x[l + 1], jobs[0].X = b.a, jobs[0].dW = g + p.mlp_down;
                    jobs[1].dY = slot.g_u[l], jobs[1].X = b.n2, jobs[1].dW = g + p.mlp_up;
                    jobs[2].dY = slot.g_mid[l], jobs[2].X = b.o, jobs[2].dW = g + p.attn_out;
                    jobs[3].dY = slot.g_qkv[l], jobs[3].X = b.n1, jobs[3].dW = g + p.qkv;
                }
                TgkWgradJob &head = slot.wgrad_jobs[4 * c.depth], &table_job = slot.wgrad_jobs[4 * c.depth + 1];
                head.dY = slot.logits, head.X = slot.nf, head.dW = slot.gradient + e->layout.head;
                e->allocate(slot.onehot, M * V, false);
                table_job.dY = slot.onehot, table_job.X = slot.g_x[0], table_job.dW = slot.gradient + e->layout.embedding;
                uint8_t *table = nullptr;
                e->allocate(table, table_bytes, false);
                slot.wgrad_table = table;
                ok(tgk_gemm_wgrad_list_prepare(int(M), int(slot.wgrad_jobs.size()), slot.wgrad_jobs.data(), table, table_bytes));
                // the tensors no matrix product writes, in ranges of at most 8192 elements; with the matrices they
                // must cover the flat gradient exactly
                struct Range {
                    int64_t start, length;
                };
                std::vector<Range> ranges;
                int64_t covered = 2 * int64_t(V) * d; // the head and the token table
                const auto cover = [&](int64_t start, int64_t length) {
                    covered += length;
                    for (int64_t at = 0; at < length; at += 8192)
                        ranges.push_back({start + at, std::min<int64_t>(8192, length - at)});
                };
                cover(e->layout.positions, int64_t(c.context) * d);
                for (int l = 0; l < c.depth; ++l) {
                    const TgLayerParameters &p = e->layout.layers[l];
                    cover(p.ln1_g, d), cover(p.ln1_b, d), cover(p.ln2_g, d), cover(p.ln2_b, d);
                    covered += 4 * int64_t(d) * d + 2 * int64_t(F) * d;
                }
                cover(e->layout.lnf_g, d), cover(e->layout.lnf_b, d);
                if (covered != e->layout.count)
                    throw std::runtime_error("engine: gradient norm ranges do not cover the parameters");
                slot.list_norms = tgk_gemm_wgrad_list_sumsq_count(int(M), int(slot.wgrad_jobs.size()), slot.wgrad_jobs.data());
                slot.range_norms = int(ranges.size());
                if (slot.list_norms <= 0 || slot.list_norms + slot.range_norms > 4096)
                    throw std::runtime_error("engine: too many gradient norm partials");
                e->allocate(slot.norms, size_t(slot.list_norms + slot.range_norms), false);
                uint8_t *device_ranges = nullptr;
                e->allocate(device_ranges, ranges.size() * sizeof(Range), false);
                check_hip(hipMemcpy(device_ranges, ranges.data(), ranges.size() * sizeof(Range), hipMemcpyHostToDevice),
                          "norm ranges: ");
                slot.norm_ranges = device_ranges;
                batch_need = std::max(batch_need, tgk_gemm_wgrad_list_workspace(int(M), int(slot.wgrad_jobs.size()), slot.wgrad_jobs.data()));
            }
        }
        e->batched_wgrad = !e->list_wgrad && batch_need > 0;
        if (e->batched_wgrad)
            for (Slot &slot : e->slots)
                e->allocate(slot.dh_mid, M * d, false);
        size_t need = std::max(batch_need, tgk_attn_bwd_workspace(c.batch, model->heads, c.context));
        need = std::max(need, tgk_layernorm_bwd_workspace(int(M), int(d)));
        need = std::max(need, tgk_embed_bwd_workspace(int(M), int(d)));
        need = std::max(need, tgk_gemm_wgrad_workspace(int(M), int(V), int(d)));
        need = std::max(need, tgk_gemm_wgrad_workspace(int(M), int(d), int(F)));
        need = std::max(need, tgk_gemm_wgrad_workspace(int(M), int(F), int(d)));
        need = std::max(need, tgk_gemm_wgrad_workspace(int(M), int(d), int(d)));
        need = std::max(need, tgk_gemm_wgrad_workspace(int(M), int(3 * d), int(d)));
        e->workspace_bytes = need;
        const int norms = 2 * c.depth + 1;
        const size_t ln_stride = tgk_layernorm_bwd_workspace(int(M), int(d));
        for (Slot &slot : e->slots) {
            uint8_t *ws = nullptr;
            e->allocate(ws, need, false);
            slot.workspace = ws;
            e->allocate(slot.ln_partials, size_t(norms) * ln_stride, false);
            std::vector<float *> targets(size_t(2 * norms));
            targets[0] = slot.gradient + e->layout.lnf_g, targets[1] = slot.gradient + e->layout.lnf_b;
            for (int l = 0; l < c.depth; ++l) {
                const TgLayerParameters &p = e->layout.layers[l];
                targets[size_t(2 * (1 + 2 * l))] = slot.gradient + p.ln2_g, targets[size_t(2 * (1 + 2 * l) + 1)] = slot.gradient + p.ln2_b;
                targets[size_t(2 * (2 + 2 * l))] = slot.gradient + p.ln1_g, targets[size_t(2 * (2 + 2 * l) + 1)] = slot.gradient + p.ln1_b;
            }
            uint8_t *table = nullptr;
            e->allocate(table, targets.size() * sizeof(float *), false);
            check_hip(hipMemcpy(table, targets.data(), targets.size() * sizeof(float *), hipMemcpyHostToDevice));
            slot.ln_targets = table;
        }
        e->sync();
        return e;
    } catch (const std::exception &error) {
        tg_last_error = error.what();
        delete e;
        return nullptr;
    }
}

TG_API void tg_destroy(Engine *e) {
    delete e;
}
TG_API int tg_parameter_count(Engine *e) {
    return int(e->layout.count);
}
TG_API int tg_blocks(Engine *e) {
    return e->compute_units;
}
TG_API int tg_shared_bytes(Engine *) {
    return 3 * (128 + 192) * 64 + 4 * 4096; // the 128x192 GEMM: three 32-k stages plus the epilogue's fp32 staging tiles
}
TG_API int tg_synchronize(Engine *e) {
    return guarded([&] {
        e->use_device();
        e->sync();
    });
}
TG_API int tg_memory(Engine *e, double *used_gb) {
    return guarded([&] {
        if (!used_gb)
            throw std::runtime_error("Missing memory output");
        *used_gb = double(e->allocated_bytes) / (1024.0 * 1024.0 * 1024.0);
    });
}

// cuda/engine_state.cu:7-35
TG_API int tg_set_weights(Engine *e, const float *weights) {
    return guarded([&] {
        if (!weights)
            throw std::runtime_error("Missing weights");
        e->use_device();
        const size_t n = size_t(e->layout.count);
        std::vector<uint16_t> high(n), low(n);
        for (size_t i = 0; i < n; ++i) {
            uint32_t bits;
            std::memcpy(&bits, weights + i, 4);
            high[i] = uint16_t(bits >> 16);
            low[i] = uint16_t(bits);
        }
        e->sync(); // nothing may still read the version that is overwritten
        e->step = 0;
        e->floor = 0;
        e->total_staleness = 0, e->max_staleness = 0;
        Version &v = e->current();
        e->upload(v.hi, high.data(), n);
        e->upload(v.lo, low.data(), n);
        check_hip(hipMemsetAsync(e->momentum, 0, n * 4, e->stream));
        check_hip(hipMemsetAsync(e->variance, 0, n * 4, e->stream));
        e->refresh_transposed(v);
        e->sync();
    });
}
// cuda/engine_state.cu:36-55
TG_API int tg_get_weights(Engine *e, float *weights) {
    return guarded([&] {
        if (!weights)
            throw std::runtime_error("Missing weights output");
        e->use_device();
        const size_t n = size_t(e->layout.count);
        std::vector<uint16_t> high(n), low(n);
        e->sync();
        e->download(high.data(), e->current().hi, n);
        e->download(low.data(), e->current().lo, n);
        e->sync();
        for (size_t i = 0; i < n; ++i) {
            const uint32_t bits = (uint32_t(high[i]) << 16) | low[i];
            std::memcpy(weights + i, &bits, 4);
        }
    });
}
TG_API int tg_get_optimizer_state(Engine *e, float *momentum, float *variance, uint64_t *step) {
    return guarded([&] {
        if (!momentum || !variance || !step)
            throw std::runtime_error("Missing optimizer state output");
        e->use_device();
        e->sync();
        e->download(momentum, e->momentum, size_t(e->layout.count));
        e->download(variance, e->variance, size_t(e->layout.count));
        e->sync();
        *step = e->step;
    });
}
TG_API int tg_set_optimizer_state(Engine *e, const float *momentum, const float *variance, uint64_t step) {
    return guarded([&] {
        if (!momentum || !variance)
            throw std::runtime_error("Missing optimizer state input");
        e->use_device();
        e->sync();
        // the weights keep their values but become version `step`: move them to that place of the ring
        Version &from = e->current();
        Version &to = e->versions[step % e->versions.size()];
        if (&from != &to) {
            const size_t bytes = size_t(e->layout.count) * 2;
            check_hip(hipMemcpyAsync(to.hi, from.hi, bytes, hipMemcpyDeviceToDevice, e->stream));
            check_hip(hipMemcpyAsync(to.lo, from.lo, bytes, hipMemcpyDeviceToDevice, e->stream));
            if (to.t)
                check_hip(hipMemcpyAsync(to.t, from.t, bytes, hipMemcpyDeviceToDevice, e->stream));
        }
        e->upload(e->momentum, momentum, size_t(e->layout.count));
        e->upload(e->variance, variance, size_t(e->layout.count));
        e->step = step;
        e->floor = step;
        e->sync();
    });
}

TG_API int tg_onecycle_point(const OneCycle *schedule, int step, StepRates *rates) {
    return guarded([&] {
        if (!schedule || !rates)
            throw std::runtime_error("Missing schedule or output");
        *rates = onecycle_point(*schedule, step);
    });
}
// cuda/runtime.cu:42-61; the table stays on the host because the host issues every optimizer launch
TG_API int tg_set_onecycle(Engine *e, const OneCycle *schedule) {
    return guarded([&] {
        if (!schedule)
            throw std::runtime_error("Missing schedule");
        if (!e->schedule.empty() || e->step)
            throw std::runtime_error("Set OneCycle once, before training");
        onecycle_point(*schedule, 0); // validate before allocating
        std::vector<StepRates> rates(size_t(schedule->total_steps));
        for (int step = 0; step < schedule->total_steps; ++step)
            rates[size_t(step)] = onecycle_point(*schedule, step);
        e->schedule = std::move(rates);
    });
}

// cuda/runtime.cu:190-206
TG_API int tg_set_data(Engine *e, const uint8_t *bytes, int64_t size) {
    return guarded([&] {
        e->use_device();
        const int64_t low = std::max(8, e->config.base.context);
        if (!bytes || size <= low)
            throw std::runtime_error("Dataset needs at least " + std::to_string(low + 1) + " bytes");
        if (e->data)
            throw std::runtime_error("Dataset already loaded");
        e->allocate(e->data, size_t(size), false);
        e->data_size = size;
        e->upload(e->data, bytes, size_t(size));
        e->sync();
    });
}

// cuda/runtime.cu:213-242 with the step loop of cuda/trainer.cuh:109-124 unrolled into launches
TG_API int tg_train(Engine *e, int steps) {
    return guarded([&] {
        if (!e->data || steps < 1 || steps > MaxLaunchSteps)
            throw std::runtime_error("Load data first; each invocation permits 1.." +
                                     std::to_string(MaxLaunchSteps) + " steps");
        if (e->step + uint64_t(steps) > uint64_t(INT_MAX))
            throw std::runtime_error("Training step count exceeds signed 32-bit indexing");
        if (!e->schedule.empty() && e->step + uint64_t(steps) > e->schedule.size())
            throw std::runtime_error("Training would exceed the OneCycle schedule");
        e->use_device();
        e->version_trace.assign(size_t(steps), 0);
        for (int i = 0; i < steps; ++i)
            e->train_step(e->step + uint64_t(i), e->loss_history + size_t(i) * e->config.base.context,
                          &e->version_trace[size_t(i)]);
        e->last_train_steps = steps;
        e->step += uint64_t(steps);
    });
}
// cuda/engine_state.cu:76-92
TG_API int tg_get_training_losses(Engine *e, float *losses, int count) {
    return guarded([&] {
        if (!losses && count)
            throw std::runtime_error("Missing training loss output");
        if (count < 0 || count > e->last_train_steps)
            throw std::runtime_error("Training loss count exceeds the last launch");
        e->use_device();
        e->sync(); // the rows are written on the slots' streams
        e->download(losses, e->loss_history, size_t(count) * e->config.base.context);
        e->sync();
    });
}
// cuda/runtime.cu:243-262: the weight version each step of the last tg_train read (a synchronous engine
// trains step s on version s)
TG_API int tg_training_versions(Engine *e, int *out, int count) {
    return guarded([&] {
        if (count < 0 || count > e->last_train_steps || (!out && count))
            throw std::runtime_error("Version trace exceeds last training launch");
        for (int i = 0; i < count; ++i)
            out[i] = e->version_trace[size_t(i)];
    });
}
// cuda/runtime.cu:263-278
TG_API int tg_pipeline_stats(Engine *e, double *mean, int *maximum) {
    return guarded([&] {
        if (!mean || !maximum)
            throw std::runtime_error("Missing pipeline statistics output");
        *mean = e->step ? double(e->total_staleness) / double(e->step) : 0;
        *maximum = e->max_staleness;
    });
}

// cuda/runtime.cu:291-320
TG_API int tg_batch(Engine *e, const uint8_t *x, const uint8_t *y, float *logits, float *gradient,
                    float *loss) {
    return guarded([&] {
        if (!x || !y || !logits || !loss)
            throw std::runtime_error("Missing batch input or output");
        e->use_device();
        const size_t M = size_t(e->tokens()), V = size_t(e->config.vocab);
        if (!e->logits_f32)
            e->allocate(e->logits_f32, M * V, false);
        e->sync(); // fixed batches run on slot 0 with the newest weights, after everything in flight
        Slot &slot = e->slots[0];
        check_hip(hipMemcpyAsync(slot.input, x, M, hipMemcpyHostToDevice, slot.stream));
        check_hip(hipMemcpyAsync(slot.target, y, M, hipMemcpyHostToDevice, slot.stream));
        e->forward(slot, e->current(), gradient != nullptr, e->logits_f32);
        if (gradient)
            e->backward(slot, e->current());
        check_hip(hipStreamSynchronize(slot.stream));
        e->download(logits, e->logits_f32, M * V);
        if (gradient)
            e->download(gradient, slot.gradient, size_t(e->layout.count));
        e->read_losses(loss);
    });
}
// cuda/runtime.cu:322-351
TG_API int tg_predict(Engine *e, const uint8_t *context, float *logits) {
    return guarded([&] {
        if (!context || !logits)
            throw std::runtime_error("Missing prediction input or output");
        e->use_device();
        const Config &c = e->config.base;
        const size_t M = size_t(e->tokens()), V = size_t(e->config.vocab);
        if (!e->logits_f32)
            e->allocate(e->logits_f32, M * V, false);
        std::vector<uint8_t> input(M), target(M, 0);
        for (int b = 0; b < c.batch; ++b)
            std::copy(context, context + c.context, input.begin() + size_t(b) * c.context);
        e->sync();
        Slot &slot = e->slots[0];
        check_hip(hipMemcpyAsync(slot.input, input.data(), M, hipMemcpyHostToDevice, slot.stream));
        check_hip(hipMemcpyAsync(slot.target, target.data(), M, hipMemcpyHostToDevice, slot.stream));
        e->forward(slot, e->current(), false, e->logits_f32);
        check_hip(hipStreamSynchronize(slot.stream));
        e->download(logits, e->logits_f32 + size_t(c.context - 1) * V, V);
        e->sync();
    });
}
// cuda/runtime.cu:352-371
TG_API int tg_optimizer_test(Engine *e, const float *gradient, int steps) {
    return guarded([&] {
        if (!gradient)
            throw std::runtime_error("Missing gradient");
        if (e->slots.size() > 1)
            throw std::runtime_error("Optimizer oracle requires synchronous configuration");
        if (steps < 1 || steps > 64)
            throw std::runtime_error("steps must be 1..64");
        if (!e->schedule.empty() && e->step + uint64_t(steps) > e->schedule.size())
            throw std::runtime_error("Optimizer test would exceed the OneCycle schedule");
        e->use_device();
        e->upload(e->slots[0].gradient, gradient, size_t(e->layout.count));
        for (int i = 0; i < steps; ++i)
            e->optimize(e->step + uint64_t(i), e->slots[0].gradient, e->versions[0]);
        e->step += uint64_t(steps);
        e->sync();
    });
}

// Not in the reference.  One training step exactly like tg_train(engine, 1), with a HIP event pair
// around every operator launch on the engine's stream; returns the summed milliseconds and the
// number of launches per TG_CLASS_*.  Synchronises.
TG_API int tg_profile_step(Engine *e, float *class_ms, int *class_launches, int classes) {
    return guarded([&] {
        if (!class_ms || !class_launches || classes < TG_CLASSES)
            throw std::runtime_error("tg_profile_step needs room for TG_CLASSES entries");
        if (!e->data)
            throw std::runtime_error("Load data first");
        if (e->slots.size() > 1)
            throw std::runtime_error("tg_profile_step requires synchronous configuration (inflight 1)");
        if (!e->schedule.empty() && e->step + 1 > e->schedule.size())
            throw std::runtime_error("Training would exceed the OneCycle schedule");
        e->use_device();
        e->version_trace.assign(1, 0);
        e->profiling = true;
        try {
            e->train_step(e->step, e->loss_history, e->version_trace.data());
        } catch (...) {
            e->profiling = false;
            throw;
        }
        e->profiling = false;
        e->last_train_steps = 1;
        e->step += 1;
        e->sync();
        std::fill(class_ms, class_ms + classes, 0.f);
        std::fill(class_launches, class_launches + classes, 0);
        for (Engine::Span &span : e->spans) {
            float ms = 0.f;
            check_hip(hipEventElapsedTime(&ms, span.start, span.stop));
            class_ms[span.cls] += ms;
            class_launches[span.cls] += 1;
            e->event_pool.push_back(span.start);
            e->event_pool.push_back(span.stop);
        }
        e->spans.clear();
    });
}
