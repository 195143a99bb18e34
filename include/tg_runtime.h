/*
 * tg_* : the engine-level C ABI.  Same names, argument meaning, status convention and POD layouts
 * as the reference's runtime.h:13-42 (lostmsu/TurboGPT), so host code written against the
 * reference (trainer.cpp, sampling.cpp, report.cpp, tests/bridge.py) binds to this library
 * unchanged.  One addition: tg_create_ex, because the reference's Config has no field for the
 * model width (config.h:4 hard-codes width 16, 4 heads, vocabulary 256).
 *
 * Conventions (cuda/runtime.cu, cuda/engine_state.cu): int status 0 = ok, < 0 = error with the
 * message in tg_error() (thread local, valid until the next failing call on the same thread);
 * no exception crosses the boundary; all pointers are caller-owned HOST memory copied
 * synchronously, except that tg_train only enqueues work; an Engine is used from one thread at a
 * time; several engines may coexist.
 */
#ifndef TG_RUNTIME_H
#define TG_RUNTIME_H
#include <stdint.h>

#ifdef __cplusplus
#define TG_API extern "C" __attribute__((visibility("default")))
#else
#define TG_API __attribute__((visibility("default")))
#endif

/* config.h:5-13 - 72 bytes, mirrored by tests/bridge.py:7-15 */
typedef struct Config {
    int depth, context, batch, device;
    int blocks, ns_steps;
    float learning_rate, muon_lr;
    float beta1, beta2, momentum;
    float weight_decay, epsilon, clip;
    uint64_t seed;
    int inflight; /* 1: synchronous; 2..16: that many batches in flight on versioned, stale weights */
} Config;

/* The model shape the reference has no room for.  Byte-level GPT: pre-LayerNorm blocks,
 * softmax attention with head_dim 64, GELU MLP, learned absolute positions. */
typedef struct TgModelConfig {
    Config base;   /* depth, context, batch, device, optimizer constants, seed */
    int d_model;   /* multiple of 128 */
    int heads;     /* d_model / 64 */
    int vocab;     /* 256 */
    int ffn;       /* MLP hidden width, multiple of 128 (4*d_model in the target configs) */
    float ln_eps;  /* LayerNorm epsilon (1e-5) */
    int reserved[3];
} TgModelConfig;

/* optim.h:6-16 */
typedef struct OneCycle {
    int total_steps;
    double warmup_fraction, initial_lr_fraction, final_lr_fraction, low_momentum, high_momentum;
} OneCycle;
typedef struct StepRates {
    float multiplier, momentum;
} StepRates;

typedef struct Engine Engine;

TG_API const char *tg_error(void);                                   /* runtime.h:14 */
/* runtime.h:15, cuda/runtime.cu:62-155: the reference's own width-16 network (RMSNorm, partial RoPE,
 * arg-max attention, SwiGLU; AdamW + Muon), with the reference's limits: depth 4/8, context 4/8, batch >= 4,
 * batch*context divisible by 16, ns_steps 1..10, inflight 1..16.  Flat weight order: model.h:12-37. */
TG_API Engine *tg_create(const Config *config);
/* Validates the shape, allocates every device buffer once (weights hi/lo, m, v, gradient, saved
 * activations, workspaces, loss history); NULL on failure (cuda/runtime.cu:62-155). */
TG_API Engine *tg_create_ex(const TgModelConfig *config);
TG_API void tg_destroy(Engine *engine);                              /* runtime.h:16 */
TG_API int tg_parameter_count(Engine *engine);                       /* runtime.h:17 */
TG_API int tg_blocks(Engine *engine);                                /* runtime.h:18: compute units used */
TG_API int tg_shared_bytes(Engine *engine);                          /* runtime.h:19: largest LDS footprint */
TG_API int tg_set_weights(Engine *engine, const float *weights);     /* runtime.h:20; zeroes m, v, step */
TG_API int tg_get_weights(Engine *engine, float *weights);           /* runtime.h:21; exact fp32 (hi|lo) */
TG_API int tg_get_optimizer_state(Engine *engine, float *momentum, float *variance, uint64_t *step);
TG_API int tg_set_optimizer_state(Engine *engine, const float *momentum, const float *variance,
                                  uint64_t step);
TG_API int tg_memory(Engine *engine, double *used_gb);               /* runtime.h:25 */
TG_API int tg_set_data(Engine *engine, const uint8_t *bytes, int64_t size); /* once; size > max(8, context) */
TG_API int tg_train(Engine *engine, int steps);                      /* 1..4096, enqueues and returns */
TG_API int tg_get_training_losses(Engine *engine, float *per_position, int count); /* synchronises */
TG_API int tg_training_versions(Engine *engine, int *versions, int count);
TG_API int tg_pipeline_stats(Engine *engine, double *mean_staleness, int *max_staleness);
TG_API int tg_onecycle_point(const OneCycle *schedule, int step, StepRates *rates); /* optim.h:18-44 */
TG_API int tg_set_onecycle(Engine *engine, const OneCycle *schedule); /* once, before training */
/* Fixed batch -> logits [B*T*vocab] fp32, flat gradient [P] (NULL = evaluate only), per-position
 * mean loss [context] (cuda/runtime.cu:291-320). */
TG_API int tg_batch(Engine *engine, const uint8_t *x, const uint8_t *y, float *logits, float *gradients,
                    float *per_position);
TG_API int tg_predict(Engine *engine, const uint8_t *context, float *logits); /* last position, [vocab] */
TG_API int tg_optimizer_test(Engine *engine, const float *gradients, int steps); /* 1..64 */
TG_API int tg_synchronize(Engine *engine);

/* Not in the reference: measurement aid.  Runs one training step exactly like tg_train(engine, 1)
 * with a HIP event pair around every operator launch on the engine's stream, and returns summed
 * milliseconds and launch counts per operator class.  Synchronises. */
enum {
    TG_CLASS_GEMM_FWD = 0,   /* block projections forward with a plain or residual epilogue (QKV, attention-out, MLP-down) */
    TG_CLASS_GEMM_DGRAD = 1, /* input gradients with a plain epilogue (MLP-up, attention-out, QKV) */
    TG_CLASS_GEMM_WGRAD = 2, /* the weight gradients, partial-sum folds included */
    TG_CLASS_ATTN_FWD = 3,
    TG_CLASS_ATTN_BWD = 4,
    TG_CLASS_LAYERNORM_FWD = 5,
    TG_CLASS_LAYERNORM_BWD = 6,
    TG_CLASS_HEAD = 7,       /* vocabulary projection: forward, dgrad, wgrad */
    TG_CLASS_OTHER = 8,      /* sampling, embedding, cross-entropy, loss means */
    TG_CLASS_OPTIMIZER = 9,  /* gradient norm + AdamW */
    TG_CLASS_GEMM_FWD_GELU = 10,   /* MLP-up forward: two outputs, pre-activation and GELU */
    TG_CLASS_GEMM_DGRAD_GELU = 11, /* MLP-down input gradient times GELU' of the saved pre-activation */
    TG_CLASSES = 12
};
TG_API int tg_profile_step(Engine *engine, float *class_ms, int *class_launches, int classes);

#ifdef __cplusplus
static_assert(sizeof(Config) == 72, "Config must keep the reference layout");
static_assert(sizeof(OneCycle) == 48 && sizeof(StepRates) == 8, "schedule PODs must keep the reference layout");
#endif
#endif
