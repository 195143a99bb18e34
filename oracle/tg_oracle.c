/*
 * TEST INFRASTRUCTURE ONLY -- CPU restatement (fp32, optional bf16 rounding points) of the
 * training-step hot path.  Nothing in the shipped library links or calls this file; it is the
 * checker the HIP path is compared against, and the host-core baseline that the benchmark
 * times next to the GPU.
 *
 * What it follows in the reference (lostmsu/TurboGPT), file:line under the reference root:
 *   hash_u64                      utils.h:13-18 (SplitMix64 finaliser)
 *   hi/lo fp32 weight split       cuda/ops.cuh:6-14, cuda/engine_state.cu:15-25,46-49
 *   forward GEMM  Y = X W^T (+res) cuda/mma.cuh:77-103   (W is [Out][In] row major, bf16 RN store,
 *                                                         residual added in bf16)
 *   dgrad         dX = dY W        cuda/ops.cuh:30-55,115
 *   wgrad         dW = dY^T X      cuda/ops.cuh:83-109    (fp32 result, optional accumulate)
 *   op order, saved activations,
 *   bf16 rounding points, CE and
 *   dlogits/(B*T) scaling          cuda/model.cuh:8-99, tests/reference.py:50-81
 *   AdamW arithmetic               cuda/optim.cuh:67-106  (clip, bias correction with current beta1)
 *   weight-decay groups            cuda/optim.cuh:5-15    (matrices and head only)
 *   batch sampling                 cuda/dataset.cuh:7-34
 *   per-position loss means        cuda/trainer.cuh:79-100, cuda/runtime.cu:279-290
 *   OneCycle                       optim.h:18-44
 *
 * What the reference does not contain and is therefore restated from the published
 * mathematics (pinned by the closed-form / finite-difference / library checks in tests/):
 *   softmax causal attention with saved log-sum-exp and its analytic backward,
 *   LayerNorm (biased variance, eps inside the sqrt) forward/backward,
 *   GELU (exact erf form) forward/backward, learned absolute positions.
 *
 * Pin status: every function below is covered by tests/test_oracle_*.py against numpy fp64
 * closed forms, finite differences, or torch CPU fp64 library routines (none is "parity
 * unpinned").
 */
#include <math.h>
#include <stdint.h>
#include <stdlib.h>
#include <string.h>

#ifdef _OPENMP
#include <omp.h>
#endif

#define ORC_API __attribute__((visibility("default")))

/* ------------------------------------------------------------------------------------------
 * scalars
 * ---------------------------------------------------------------------------------------- */

/* utils.h:13-18 */
ORC_API uint64_t orc_hash_u64(uint64_t x) {
    x += 0x9e3779b97f4a7c15ULL;
    x = (x ^ (x >> 30)) * 0xbf58476d1ce4e5b9ULL;
    x = (x ^ (x >> 27)) * 0x94d049bb133111ebULL;
    return x ^ (x >> 31);
}

static inline uint32_t f2u(float f) {
    uint32_t u;
    memcpy(&u, &f, 4);
    return u;
}
static inline float u2f(uint32_t u) {
    float f;
    memcpy(&f, &u, 4);
    return f;
}

/* round-to-nearest-even to bf16, returned as fp32 (the store rounding of cuda/mma.cuh:95) */
ORC_API float orc_bf16_round(float f) {
    uint32_t u = f2u(f);
    if ((u & 0x7f800000u) == 0x7f800000u) /* inf / nan: keep, quiet the nan */
        return u2f((u & 0xffff0000u) | ((u & 0xffffu) ? 0x00400000u : 0u));
    u += 0x7fffu + ((u >> 16) & 1u);
    return u2f(u & 0xffff0000u);
}
/* high half of the fp32 master: the compute weight (cuda/ops.cuh:10-14, engine_state.cu:18-19) */
ORC_API float orc_bf16_trunc(float f) {
    return u2f(f2u(f) & 0xffff0000u);
}
ORC_API void orc_bf16_round_array(float *x, int64_t n) {
    for (int64_t i = 0; i < n; ++i)
        x[i] = orc_bf16_round(x[i]);
}
ORC_API void orc_bf16_trunc_array(float *x, int64_t n) {
    for (int64_t i = 0; i < n; ++i)
        x[i] = orc_bf16_trunc(x[i]);
}
/* cuda/engine_state.cu:15-20 and :46-49 */
ORC_API void orc_split_hilo(const float *w, uint16_t *hi, uint16_t *lo, int64_t n) {
    for (int64_t i = 0; i < n; ++i) {
        uint32_t b = f2u(w[i]);
        hi[i] = (uint16_t)(b >> 16);
        lo[i] = (uint16_t)b;
    }
}
ORC_API void orc_join_hilo(const uint16_t *hi, const uint16_t *lo, float *w, int64_t n) {
    for (int64_t i = 0; i < n; ++i)
        w[i] = u2f(((uint32_t)hi[i] << 16) | lo[i]);
}

static inline float rb(float x, int emulate) {
    return emulate ? orc_bf16_round(x) : x;
}

/* ------------------------------------------------------------------------------------------
 * counter-based synthetic inputs: element i of stream `seed` depends only on (seed, i)
 * ---------------------------------------------------------------------------------------- */
static inline double unit_open(uint64_t h) { /* (0,1] */
    return ((double)(h >> 11) + 1.0) * (1.0 / 9007199254740992.0);
}
ORC_API void orc_fill_normal(float *out, int64_t n, uint64_t seed, float scale) {
    const uint64_t base = seed << 40;
#pragma omp parallel for schedule(static)
    for (int64_t i = 0; i < n; ++i) {
        double u1 = unit_open(orc_hash_u64(base + 2 * (uint64_t)i));
        double u2 = unit_open(orc_hash_u64(base + 2 * (uint64_t)i + 1));
        out[i] = (float)(sqrt(-2.0 * log(u1)) * cos(6.283185307179586476925 * u2)) * scale;
    }
}
ORC_API void orc_fill_uniform_bytes(uint8_t *out, int64_t n, uint64_t seed) {
    const uint64_t base = seed << 40;
    for (int64_t i = 0; i < n; ++i)
        out[i] = (uint8_t)(orc_hash_u64(base + (uint64_t)i) >> 56);
}
/* Zipf(s) over 256 symbols, p(k) ~ (k+1)^-s, inverse CDF on the counter stream */
ORC_API void orc_fill_zipf_bytes(uint8_t *out, int64_t n, uint64_t seed, double s) {
    double cdf[256], total = 0;
    for (int k = 0; k < 256; ++k) {
        total += pow((double)(k + 1), -s);
        cdf[k] = total;
    }
    const uint64_t base = seed << 40;
    for (int64_t i = 0; i < n; ++i) {
        double u = unit_open(orc_hash_u64(base + (uint64_t)i)) * total;
        int lo = 0, hi = 255;
        while (lo < hi) {
            int mid = (lo + hi) / 2;
            if (cdf[mid] >= u)
                hi = mid;
            else
                lo = mid + 1;
        }
        out[i] = (uint8_t)lo;
    }
}

/* ------------------------------------------------------------------------------------------
 * GEMM family.  X [M][K], W [N][K], Y/dY [M][N], all row major with explicit leading
 * dimensions; fp32 accumulate.  `emulate` rounds stores to bf16 as the device path does.
 * ---------------------------------------------------------------------------------------- */

/* cuda/mma.cuh:77-103: y = RN(sum_k x w) ; if residual: y = RN(y + residual) */
ORC_API void orc_gemm_fwd(int M, int N, int K, const float *X, int ldx, const float *W, int ldw,
                          float *Y, int ldy, const float *residual, int ldr, int emulate) {
#pragma omp parallel for schedule(static)
    for (int i = 0; i < M; ++i) {
        const float *x = X + (size_t)i * ldx;
        for (int j = 0; j < N; ++j) {
            const float *w = W + (size_t)j * ldw;
            float acc = 0;
#pragma omp simd reduction(+ : acc)
            for (int k = 0; k < K; ++k)
                acc += x[k] * w[k];
            acc = rb(acc, emulate);
            if (residual)
                acc = rb(acc + residual[(size_t)i * ldr + j], emulate);
            Y[(size_t)i * ldy + j] = acc;
        }
    }
}

/* cuda/ops.cuh:115 (matmul dY[32 x out] . W[out x in]) then cast_result :51-55 */
ORC_API void orc_gemm_dgrad(int M, int N, int K, const float *dY, int lddy, const float *W, int ldw,
                            float *dX, int lddx, int emulate) {
#pragma omp parallel
    {
        float *row = (float *)malloc(sizeof(float) * (size_t)K);
#pragma omp for schedule(static)
        for (int i = 0; i < M; ++i) {
            memset(row, 0, sizeof(float) * (size_t)K);
            for (int j = 0; j < N; ++j) {
                const float g = dY[(size_t)i * lddy + j];
                const float *w = W + (size_t)j * ldw;
#pragma omp simd
                for (int k = 0; k < K; ++k)
                    row[k] += g * w[k];
            }
            for (int k = 0; k < K; ++k)
                dX[(size_t)i * lddx + k] = rb(row[k], emulate);
        }
        free(row);
    }
}

/* cuda/ops.cuh:83-109: G[o][i] (=|+=) sum_t dY[t][o] X[t][i], fp32, never rounded */
ORC_API void orc_gemm_wgrad(int M, int N, int K, const float *dY, int lddy, const float *X, int ldx,
                            float *dW, int lddw, int accumulate) {
#pragma omp parallel
    {
        float *row = (float *)malloc(sizeof(float) * (size_t)K);
#pragma omp for schedule(static)
        for (int j = 0; j < N; ++j) {
            memset(row, 0, sizeof(float) * (size_t)K);
            for (int t = 0; t < M; ++t) {
                const float g = dY[(size_t)t * lddy + j];
                const float *x = X + (size_t)t * ldx;
#pragma omp simd
                for (int k = 0; k < K; ++k)
                    row[k] += g * x[k];
            }
            float *out = dW + (size_t)j * lddw;
            for (int k = 0; k < K; ++k)
                out[k] = accumulate ? out[k] + row[k] : row[k];
        }
        free(row);
    }
}

/* ------------------------------------------------------------------------------------------
 * causal softmax attention on the packed qkv buffer.
 * qkv [B*T][ld] : q at column 0, k at column d, v at column 2d (d = H*hd), head h at +h*hd.
 * out [B*T][ldo], lse [B][H][T] (natural log of sum exp of scaled scores).
 * ---------------------------------------------------------------------------------------- */
ORC_API void orc_attn_fwd(int B, int H, int T, int hd, const float *qkv, int ld, float *out,
                          int ldo, float *lse, float scale, int emulate) {
    const int d = H * hd;
#pragma omp parallel
    {
        float *p = (float *)malloc(sizeof(float) * (size_t)T);
        float *acc = (float *)malloc(sizeof(float) * (size_t)hd);
#pragma omp for collapse(2) schedule(dynamic, 1)
        for (int b = 0; b < B; ++b)
            for (int h = 0; h < H; ++h)
                for (int t = 0; t < T; ++t) {
                    const float *q = qkv + (size_t)(b * T + t) * ld + h * hd;
                    float high = -INFINITY;
                    for (int s = 0; s <= t; ++s) {
                        const float *k = qkv + (size_t)(b * T + s) * ld + d + h * hd;
                        float dot = 0;
#pragma omp simd reduction(+ : dot)
                        for (int c = 0; c < hd; ++c)
                            dot += q[c] * k[c];
                        p[s] = dot * scale;
                        high = fmaxf(high, p[s]);
                    }
                    float sum = 0;
                    for (int s = 0; s <= t; ++s) {
                        p[s] = expf(p[s] - high);
                        sum += p[s];
                    }
                    memset(acc, 0, sizeof(float) * (size_t)hd);
                    for (int s = 0; s <= t; ++s) {
                        const float *v = qkv + (size_t)(b * T + s) * ld + 2 * d + h * hd;
                        /* the device path feeds bf16 probabilities (unnormalised) to the PV product */
                        const float w = rb(p[s], emulate);
#pragma omp simd
                        for (int c = 0; c < hd; ++c)
                            acc[c] += w * v[c];
                    }
                    float *o = out + (size_t)(b * T + t) * ldo + h * hd;
                    for (int c = 0; c < hd; ++c)
                        o[c] = rb(acc[c] / sum, emulate);
                    lse[((size_t)b * H + h) * T + t] = high + logf(sum);
                }
        free(p);
        free(acc);
    }
}

/* dV = P^T dO ; dP = dO V^T ; dS = P o (dP - rowsum(dO o O)) ; dQ = scale dS K ; dK = scale dS^T Q
 * P is recomputed from q, k and the saved lse.  dqkv has the same packed layout as qkv. */
ORC_API void orc_attn_bwd(int B, int H, int T, int hd, const float *qkv, int ld, const float *out,
                          int ldo, const float *lse, const float *dout, int lddo, float *dqkv,
                          int lddq, float scale, int emulate) {
    const int d = H * hd;
#pragma omp parallel
    {
        float *dq = (float *)malloc(sizeof(float) * (size_t)hd);
        float *dk = (float *)malloc(sizeof(float) * (size_t)T * hd);
        float *dv = (float *)malloc(sizeof(float) * (size_t)T * hd);
#pragma omp for collapse(2) schedule(dynamic, 1)
        for (int b = 0; b < B; ++b)
            for (int h = 0; h < H; ++h) {
                memset(dk, 0, sizeof(float) * (size_t)T * hd);
                memset(dv, 0, sizeof(float) * (size_t)T * hd);
                for (int t = 0; t < T; ++t) {
                    const size_t row = (size_t)(b * T + t);
                    const float *q = qkv + row * ld + h * hd;
                    const float *go = dout + row * lddo + h * hd;
                    const float *o = out + row * ldo + h * hd;
                    const float l = lse[((size_t)b * H + h) * T + t];
                    float delta = 0;
                    for (int c = 0; c < hd; ++c)
                        delta += go[c] * o[c];
                    memset(dq, 0, sizeof(float) * (size_t)hd);
                    for (int s = 0; s <= t; ++s) {
                        const float *k = qkv + (size_t)(b * T + s) * ld + d + h * hd;
                        const float *v = qkv + (size_t)(b * T + s) * ld + 2 * d + h * hd;
                        float dot = 0, dp = 0;
                        for (int c = 0; c < hd; ++c) {
                            dot += q[c] * k[c];
                            dp += go[c] * v[c];
                        }
                        const float p = expf(dot * scale - l);
                        const float pw = rb(p, emulate);                      /* bf16 P into dV */
                        const float ds = rb(p * (dp - delta), emulate) * scale; /* bf16 dS into dQ,dK */
                        for (int c = 0; c < hd; ++c) {
                            dv[(size_t)s * hd + c] += pw * go[c];
                            dk[(size_t)s * hd + c] += ds * q[c];
                            dq[c] += ds * k[c];
                        }
                    }
                    float *gq = dqkv + row * lddq + h * hd;
                    for (int c = 0; c < hd; ++c)
                        gq[c] = rb(dq[c], emulate);
                }
                for (int s = 0; s < T; ++s) {
                    float *gk = dqkv + (size_t)(b * T + s) * lddq + d + h * hd;
                    float *gv = dqkv + (size_t)(b * T + s) * lddq + 2 * d + h * hd;
                    for (int c = 0; c < hd; ++c) {
                        gk[c] = rb(dk[(size_t)s * hd + c], emulate);
                        gv[c] = rb(dv[(size_t)s * hd + c], emulate);
                    }
                }
            }
        free(dq);
        free(dk);
        free(dv);
    }
}

/* ------------------------------------------------------------------------------------------
 * memory-bound operators
 * ---------------------------------------------------------------------------------------- */

/* LayerNorm over the last dimension; gamma/beta are full fp32 (cuda/ops.cuh:61 reads the
 * norm scale through precise_weight).  y = RN((x-mean) * rsqrt(var+eps) * gamma + beta) */
ORC_API void orc_layernorm_fwd(int M, int D, const float *x, const float *gamma, const float *beta,
                               float *y, float eps, int emulate) {
#pragma omp parallel for schedule(static)
    for (int i = 0; i < M; ++i) {
        const float *r = x + (size_t)i * D;
        float mean = 0;
        for (int c = 0; c < D; ++c)
            mean += r[c];
        mean /= D;
        float var = 0;
        for (int c = 0; c < D; ++c)
            var += (r[c] - mean) * (r[c] - mean);
        const float inv = 1.0f / sqrtf(var / D + eps);
        for (int c = 0; c < D; ++c)
            y[(size_t)i * D + c] = rb((r[c] - mean) * inv * gamma[c] + beta[c], emulate);
    }
}

/* dx = RN(LN'(x) dy); if residual: dx = RN(dx_in + RN(...)) (cuda/ops.cuh:74-76 keeps residual
 * gradients in bf16); dgamma += sum dy*xhat, dbeta += sum dy (fp32). */
ORC_API void orc_layernorm_bwd(int M, int D, const float *x, const float *dy, const float *gamma,
                               float *dx, float *dgamma, float *dbeta, float eps, int residual,
                               int emulate) {
    double *dg = (double *)calloc((size_t)D, sizeof(double));
    double *db = (double *)calloc((size_t)D, sizeof(double));
    for (int i = 0; i < M; ++i) {
        const float *r = x + (size_t)i * D, *g = dy + (size_t)i * D;
        float mean = 0;
        for (int c = 0; c < D; ++c)
            mean += r[c];
        mean /= D;
        float var = 0;
        for (int c = 0; c < D; ++c)
            var += (r[c] - mean) * (r[c] - mean);
        const float inv = 1.0f / sqrtf(var / D + eps);
        float s1 = 0, s2 = 0;
        for (int c = 0; c < D; ++c) {
            const float z = (r[c] - mean) * inv, dz = g[c] * gamma[c];
            s1 += dz;
            s2 += dz * z;
            dg[c] += (double)g[c] * z;
            db[c] += g[c];
        }
        for (int c = 0; c < D; ++c) {
            const float z = (r[c] - mean) * inv, dz = g[c] * gamma[c];
            const float value = rb((dz - s1 / D - z * s2 / D) * inv, emulate);
            float *o = dx + (size_t)i * D + c;
            *o = residual ? rb(*o + value, emulate) : value;
        }
    }
    for (int c = 0; c < D; ++c) {
        dgamma[c] += (float)dg[c];
        dbeta[c] += (float)db[c];
    }
    free(dg);
    free(db);
}

static inline float gelu(float x) {
    return 0.5f * x * (1.0f + erff(x * 0.70710678118654752f));
}
/* same closed form as the GELU' of cuda/attention.cuh:64 */
static inline float gelu_grad(float x) {
    return 0.5f * (1.0f + erff(x * 0.70710678118654752f)) +
           x * 0.39894228040143268f * expf(-0.5f * x * x);
}
ORC_API void orc_gelu_fwd(int64_t n, const float *u, float *a, int emulate) {
    for (int64_t i = 0; i < n; ++i)
        a[i] = rb(gelu(u[i]), emulate);
}
ORC_API void orc_gelu_bwd(int64_t n, const float *u, const float *da, float *du, int emulate) {
    for (int64_t i = 0; i < n; ++i)
        du[i] = rb(da[i] * gelu_grad(u[i]), emulate);
}

/* cuda/model.cuh:33-58: per token loss = logsumexp(logits) - logits[y];
 * dlogits = RN((softmax - onehot) * inv_count).  V = vocabulary. */
ORC_API void orc_cross_entropy(int M, int V, const float *logits, const uint8_t *y, float *loss,
                               float *dlogits, float inv_count, int emulate) {
#pragma omp parallel for schedule(static)
    for (int i = 0; i < M; ++i) {
        const float *r = logits + (size_t)i * V;
        float high = -INFINITY;
        for (int c = 0; c < V; ++c)
            high = fmaxf(high, r[c]);
        float sum = 0;
        for (int c = 0; c < V; ++c)
            sum += expf(r[c] - high);
        loss[i] = high + logf(sum) - r[y[i]];
        if (dlogits)
            for (int c = 0; c < V; ++c)
                dlogits[(size_t)i * V + c] =
                    rb((expf(r[c] - high) / sum - (c == y[i] ? 1.0f : 0.0f)) * inv_count, emulate);
    }
}

/* cuda/optim.cuh:92-105 on the fp32 master (hi|lo recombined).  decay[i] selects the
 * weight-decay group; clip_scale = min(1, clip/(||g||+1e-6)) is computed by the caller
 * (cuda/optim.cuh:78).  step is the 0-based index of this update. */
ORC_API void orc_adamw(int64_t n, float *w, float *m, float *v, const float *g,
                       const uint8_t *decay, float lr, float beta1, float beta2, float eps,
                       float weight_decay, float clip_scale, uint64_t step) {
    const float bc1 = 1 - powf(beta1, (float)(step + 1)), bc2 = 1 - powf(beta2, (float)(step + 1));
    for (int64_t i = 0; i < n; ++i) {
        const float gi = g[i] * clip_scale;
        const float mi = m[i] + (1 - beta1) * (gi - m[i]);
        const float vi = beta2 * v[i] + (1 - beta2) * gi * gi;
        m[i] = mi;
        v[i] = vi;
        const float wi = w[i] * (1 - lr * (decay[i] ? weight_decay : 0.f));
        w[i] = wi - (lr / bc1) * mi / (sqrtf(vi) / sqrtf(bc2) + eps);
    }
}
ORC_API float orc_clip_scale(int64_t n, const float *g, float clip) {
    if (!(clip > 0))
        return 1.f;
    double sum = 0;
    for (int64_t i = 0; i < n; ++i)
        sum += (double)g[i] * g[i];
    return fminf(1.f, clip / (sqrtf((float)sum) + 1e-6f));
}

/* optim.h:18-44.  Returns 0 on success, -1 on an invalid schedule/step. */
ORC_API int orc_onecycle_point(int total_steps, double warmup_fraction, double initial_lr_fraction,
                               double final_lr_fraction, double low_momentum, double high_momentum,
                               int step, float *multiplier, float *momentum) {
    if (total_steps < 1 || step < 0 || step >= total_steps ||
        !(warmup_fraction > 0 && warmup_fraction < 1) ||
        !(initial_lr_fraction > 0 && initial_lr_fraction < 1) ||
        !(final_lr_fraction > 0 && final_lr_fraction <= initial_lr_fraction) ||
        !(low_momentum >= 0 && low_momentum < 1) ||
        !(high_momentum >= low_momentum && high_momentum < 1))
        return -1;
    const double warmup_steps = warmup_fraction * total_steps - 1;
    if (warmup_steps == 0)
        return -1;
    const int warming = step <= warmup_steps;
    const double f = warming ? step / warmup_steps
                             : (step - warmup_steps) / (total_steps - 1 - warmup_steps);
    const double c = 0.5 * (1 + cos(3.14159265358979323846 * f));
    if (warming) {
        *multiplier = (float)(1.0 + (initial_lr_fraction - 1.0) * c);
        *momentum = (float)(low_momentum + (high_momentum - low_momentum) * c);
    } else {
        *multiplier = (float)(final_lr_fraction + (1.0 - final_lr_fraction) * c);
        *momentum = (float)(high_momentum + (low_momentum - high_momentum) * c);
    }
    return 0;
}

/* cuda/dataset.cuh:13-27: endpoint = 8 + hash(seed + step*batch + i) mod (n-8);
 * x = data[e-T : e], y = data[e-T+1 : e+1].  Sequences whose window would start before the
 * first byte (possible only when T > 8) wrap to the first T+1 bytes; see the product header. */
ORC_API void orc_sample_batch(const uint8_t *data, int64_t size, uint64_t seed, uint64_t step,
                              int batch, int context, uint8_t *x, uint8_t *y) {
    const int64_t low = context > 8 ? context : 8;
    for (int b = 0; b < batch; ++b) {
        int64_t e = low + (int64_t)(orc_hash_u64(seed + step * (uint64_t)batch + (uint64_t)b) %
                                    (uint64_t)(size - low));
        for (int p = 0; p < context; ++p) {
            x[(size_t)b * context + p] = data[e - context + p];
            y[(size_t)b * context + p] = data[e - context + p + 1];
        }
    }
}

/* ------------------------------------------------------------------------------------------
 * the model: byte-level GPT, pre-LayerNorm, GELU MLP, learned absolute positions.
 * Flat parameter order (every matrix [Out][In] row major, model.h:12-37 extended):
 *   embedding[V][d], positions[T][d],
 *   per layer: ln1_g[d], ln1_b[d], qkv[3d][d], attn_out[d][d], ln2_g[d], ln2_b[d],
 *              mlp_up[F][d], mlp_down[d][F]
 *   lnf_g[d], lnf_b[d], head[V][d]
 * ---------------------------------------------------------------------------------------- */
typedef struct {
    int depth, context, batch, d_model, heads, vocab, ffn;
    float ln_eps;
    int emulate; /* 1: round activations to bf16 at the device path's store points */
} OrcModel;

typedef struct {
    int64_t ln1_g, ln1_b, qkv, attn_out, ln2_g, ln2_b, mlp_up, mlp_down;
} OrcLayer;
typedef struct {
    int64_t embedding, positions, lnf_g, lnf_b, head, count;
    OrcLayer layers[64];
} OrcLayout;

ORC_API int orc_layout(const OrcModel *c, OrcLayout *p) {
    if (c->depth < 1 || c->depth > 64)
        return -1;
    int64_t n = 0;
    const int64_t d = c->d_model, F = c->ffn;
#define TAKE(field, size) \
    do {                  \
        field = n;        \
        n += (size);      \
    } while (0)
    TAKE(p->embedding, (int64_t)c->vocab * d);
    TAKE(p->positions, (int64_t)c->context * d);
    for (int l = 0; l < c->depth; ++l) {
        OrcLayer *b = &p->layers[l];
        TAKE(b->ln1_g, d);
        TAKE(b->ln1_b, d);
        TAKE(b->qkv, 3 * d * d);
        TAKE(b->attn_out, d * d);
        TAKE(b->ln2_g, d);
        TAKE(b->ln2_b, d);
        TAKE(b->mlp_up, F * d);
        TAKE(b->mlp_down, d * F);
    }
    TAKE(p->lnf_g, d);
    TAKE(p->lnf_b, d);
    TAKE(p->head, (int64_t)c->vocab * d);
#undef TAKE
    p->count = n;
    return 0;
}
ORC_API int64_t orc_parameter_count(const OrcModel *c) {
    OrcLayout p;
    return orc_layout(c, &p) ? -1 : p.count;
}
/* 1 where AdamW applies weight decay: hidden matrices and head (cuda/optim.cuh:5-15) */
ORC_API void orc_decay_mask(const OrcModel *c, uint8_t *mask) {
    OrcLayout p;
    orc_layout(c, &p);
    memset(mask, 0, (size_t)p.count);
    for (int l = 0; l < c->depth; ++l) {
        const OrcLayer *b = &p.layers[l];
        memset(mask + b->qkv, 1, (size_t)(b->ln2_g - b->qkv));
        memset(mask + b->mlp_up, 1, (size_t)(2 * (int64_t)c->ffn * c->d_model));
    }
    memset(mask + p.head, 1, (size_t)(p.count - p.head));
}

/* N(0, 0.02) matrices (residual-writing ones scaled by 1/sqrt(2 depth), model.cpp:21-27),
 * gamma = 1, beta = 0.  Streams are keyed like model.cpp's semantic seeds. */
ORC_API void orc_init_weights(const OrcModel *c, uint64_t seed, float scale, float *w) {
    OrcLayout p;
    orc_layout(c, &p);
    memset(w, 0, sizeof(float) * (size_t)p.count);
    const int64_t d = c->d_model, F = c->ffn;
    const float inner = scale / sqrtf(2.0f * c->depth);
    orc_fill_normal(w + p.embedding, (int64_t)c->vocab * d, seed + 1, scale);
    orc_fill_normal(w + p.positions, (int64_t)c->context * d, seed + 2, scale);
    for (int l = 0; l < c->depth; ++l) {
        const OrcLayer *b = &p.layers[l];
        for (int64_t i = 0; i < d; ++i)
            w[b->ln1_g + i] = w[b->ln2_g + i] = 1.f;
        orc_fill_normal(w + b->qkv, 3 * d * d, seed + 100 + l * 10, scale);
        orc_fill_normal(w + b->attn_out, d * d, seed + 101 + l * 10, inner);
        orc_fill_normal(w + b->mlp_up, F * d, seed + 102 + l * 10, scale);
        orc_fill_normal(w + b->mlp_down, d * F, seed + 103 + l * 10, inner);
    }
    for (int64_t i = 0; i < d; ++i)
        w[p.lnf_g + i] = 1.f;
    orc_fill_normal(w + p.head, (int64_t)c->vocab * d, seed + 3, scale);
}

typedef struct {
    float *x, *n1, *qkv, *o, *lse, *mid, *n2, *u, *a;
} OrcSaved;

/* One forward (+ backward when grad != NULL) over a fixed batch, the CPU image of tg_batch
 * (cuda/runtime.cu:291-320).  params: fp32 masters; matrices/embeddings are used through their
 * truncated bf16 high half, norm scales in full fp32 (tests/reference.py:14-21,52).
 * logits [B*T][V] (may be NULL), grad [P] (may be NULL; overwritten), token_loss [B*T]. */
ORC_API int orc_model_batch(const OrcModel *c, const float *params, const uint8_t *x,
                            const uint8_t *y, float *logits_out, float *grad, float *token_loss) {
    OrcLayout p;
    if (orc_layout(c, &p))
        return -1;
    const int E = c->emulate, T = c->context, d = c->d_model, F = c->ffn, V = c->vocab;
    const int H = c->heads, hd = d / H, L = c->depth;
    const int M = c->batch * T;
    const float scale = 1.0f / sqrtf((float)hd);
    float *w = (float *)malloc(sizeof(float) * (size_t)p.count);
    memcpy(w, params, sizeof(float) * (size_t)p.count);
    /* compute weights: truncated, except the norm scales/biases */
    orc_bf16_trunc_array(w + p.embedding, (int64_t)V * d + (int64_t)T * d);
    for (int l = 0; l < L; ++l) {
        orc_bf16_trunc_array(w + p.layers[l].qkv, 4 * (int64_t)d * d);
        orc_bf16_trunc_array(w + p.layers[l].mlp_up, 2 * (int64_t)F * d);
    }
    orc_bf16_trunc_array(w + p.head, (int64_t)V * d);

#define ALLOC(n) (float *)malloc(sizeof(float) * (size_t)(n))
    OrcSaved *S = (OrcSaved *)calloc((size_t)L, sizeof(OrcSaved));
    float *h = ALLOC((size_t)M * d), *nf = ALLOC((size_t)M * d), *logits = ALLOC((size_t)M * V);
    for (int i = 0; i < M; ++i)
        for (int k = 0; k < d; ++k)
            h[(size_t)i * d + k] =
                rb(w[p.embedding + (int64_t)x[i] * d + k] + w[p.positions + (int64_t)(i % T) * d + k], E);
    for (int l = 0; l < L; ++l) {
        const OrcLayer *b = &p.layers[l];
        OrcSaved *s = &S[l];
        s->x = ALLOC((size_t)M * d);
        s->n1 = ALLOC((size_t)M * d);
        s->qkv = ALLOC((size_t)M * 3 * d);
        s->o = ALLOC((size_t)M * d);
        s->lse = ALLOC((size_t)c->batch * H * T);
        s->mid = ALLOC((size_t)M * d);
        s->n2 = ALLOC((size_t)M * d);
        s->u = ALLOC((size_t)M * F);
        s->a = ALLOC((size_t)M * F);
        memcpy(s->x, h, sizeof(float) * (size_t)M * d);
        orc_layernorm_fwd(M, d, s->x, w + b->ln1_g, w + b->ln1_b, s->n1, c->ln_eps, E);
        orc_gemm_fwd(M, 3 * d, d, s->n1, d, w + b->qkv, d, s->qkv, 3 * d, NULL, 0, E);
        orc_attn_fwd(c->batch, H, T, hd, s->qkv, 3 * d, s->o, d, s->lse, scale, E);
        orc_gemm_fwd(M, d, d, s->o, d, w + b->attn_out, d, s->mid, d, s->x, d, E);
        orc_layernorm_fwd(M, d, s->mid, w + b->ln2_g, w + b->ln2_b, s->n2, c->ln_eps, E);
        orc_gemm_fwd(M, F, d, s->n2, d, w + b->mlp_up, d, s->u, F, NULL, 0, E);
        orc_gelu_fwd((int64_t)M * F, s->u, s->a, E);
        orc_gemm_fwd(M, d, F, s->a, F, w + b->mlp_down, F, h, d, s->mid, d, E);
    }
    orc_layernorm_fwd(M, d, h, w + p.lnf_g, w + p.lnf_b, nf, c->ln_eps, E);
    /* logits are stored in bf16 by the head projection (cuda/model.cuh:32) */
    orc_gemm_fwd(M, V, d, nf, d, w + p.head, d, logits, V, NULL, 0, E);
    if (logits_out)
        memcpy(logits_out, logits, sizeof(float) * (size_t)M * V);

    float *dlogits = grad ? ALLOC((size_t)M * V) : NULL;
    orc_cross_entropy(M, V, logits, y, token_loss, dlogits, 1.0f / (float)M, E);

    if (grad) {
        memset(grad, 0, sizeof(float) * (size_t)p.count);
        float *dh = ALLOC((size_t)M * d), *t1 = ALLOC((size_t)M * d), *dqkv = ALLOC((size_t)M * 3 * d);
        float *da = ALLOC((size_t)M * F), *du = ALLOC((size_t)M * F);
        orc_gemm_wgrad(M, V, d, dlogits, V, nf, d, grad + p.head, d, 0);
        orc_gemm_dgrad(M, V, d, dlogits, V, w + p.head, d, t1, d, E);
        orc_layernorm_bwd(M, d, h, t1, w + p.lnf_g, dh, grad + p.lnf_g, grad + p.lnf_b, c->ln_eps, 0, E);
        for (int l = L - 1; l >= 0; --l) {
            const OrcLayer *b = &p.layers[l];
            OrcSaved *s = &S[l];
            orc_gemm_wgrad(M, d, F, dh, d, s->a, F, grad + b->mlp_down, F, 0);
            orc_gemm_dgrad(M, d, F, dh, d, w + b->mlp_down, F, da, F, E);
            orc_gelu_bwd((int64_t)M * F, s->u, da, du, E);
            orc_gemm_wgrad(M, F, d, du, F, s->n2, d, grad + b->mlp_up, d, 0);
            orc_gemm_dgrad(M, F, d, du, F, w + b->mlp_up, d, t1, d, E);
            orc_layernorm_bwd(M, d, s->mid, t1, w + b->ln2_g, dh, grad + b->ln2_g, grad + b->ln2_b,
                              c->ln_eps, 1, E);
            orc_gemm_wgrad(M, d, d, dh, d, s->o, d, grad + b->attn_out, d, 0);
            orc_gemm_dgrad(M, d, d, dh, d, w + b->attn_out, d, t1, d, E);
            orc_attn_bwd(c->batch, H, T, hd, s->qkv, 3 * d, s->o, d, s->lse, t1, d, dqkv, 3 * d,
                         scale, E);
            orc_gemm_wgrad(M, 3 * d, d, dqkv, 3 * d, s->n1, d, grad + b->qkv, d, 0);
            orc_gemm_dgrad(M, 3 * d, d, dqkv, 3 * d, w + b->qkv, d, t1, d, E);
            orc_layernorm_bwd(M, d, s->x, t1, w + b->ln1_g, dh, grad + b->ln1_g, grad + b->ln1_b,
                              c->ln_eps, 1, E);
        }
        /* cuda/model.cuh:96-97 scatter-add, plus the positional table's column sums */
        for (int i = 0; i < M; ++i)
            for (int k = 0; k < d; ++k) {
                grad[p.embedding + (int64_t)x[i] * d + k] += dh[(size_t)i * d + k];
                grad[p.positions + (int64_t)(i % T) * d + k] += dh[(size_t)i * d + k];
            }
        free(dh);
        free(t1);
        free(dqkv);
        free(da);
        free(du);
        free(dlogits);
    }
    for (int l = 0; l < L; ++l) {
        free(S[l].x); free(S[l].n1); free(S[l].qkv); free(S[l].o); free(S[l].lse);
        free(S[l].mid); free(S[l].n2); free(S[l].u); free(S[l].a);
    }
    free(S);
    free(h);
    free(nf);
    free(logits);
    free(w);
#undef ALLOC
    return 0;
}

/* cuda/trainer.cuh:94-97 / cuda/runtime.cu:284-289: mean over the batch per position, in double */
ORC_API void orc_position_means(int batch, int context, const float *token_loss, float *out) {
    for (int p = 0; p < context; ++p) {
        double sum = 0;
        for (int b = 0; b < batch; ++b)
            sum += token_loss[(size_t)b * context + p];
        out[p] = (float)(sum / batch);
    }
}

/* `steps` synchronous optimizer steps on hash-sampled batches, the CPU image of tg_train
 * (cuda/trainer.cuh:103-125 in mode Train).  params/m/v are updated in place; losses
 * [steps][context].  lr schedule: multiplier/momentum arrays of length >= first_step+steps, or
 * NULL for constant rates. */
ORC_API int orc_train(const OrcModel *c, float *params, float *m, float *v, const uint8_t *data,
                      int64_t size, uint64_t seed, uint64_t first_step, int steps, float lr,
                      float beta1, float beta2, float eps, float weight_decay, float clip,
                      const float *multipliers, const float *momenta, float *losses) {
    const int64_t P = orc_parameter_count(c);
    if (P < 0)
        return -1;
    const int M = c->batch * c->context;
    uint8_t *x = (uint8_t *)malloc((size_t)M), *y = (uint8_t *)malloc((size_t)M);
    uint8_t *mask = (uint8_t *)malloc((size_t)P);
    float *g = (float *)malloc(sizeof(float) * (size_t)P), *tl = (float *)malloc(sizeof(float) * (size_t)M);
    orc_decay_mask(c, mask);
    for (int s = 0; s < steps; ++s) {
        const uint64_t step = first_step + (uint64_t)s;
        orc_sample_batch(data, size, seed, step, c->batch, c->context, x, y);
        orc_model_batch(c, params, x, y, NULL, g, tl);
        orc_position_means(c->batch, c->context, tl, losses + (size_t)s * c->context);
        const float cs = orc_clip_scale(P, g, clip);
        const float rate = multipliers ? lr * multipliers[step] : lr;
        const float b1 = momenta ? momenta[step] : beta1;
        orc_adamw(P, params, m, v, g, mask, rate, b1, beta2, eps, weight_decay, cs, step);
    }
    free(x); free(y); free(mask); free(g); free(tl);
    return 0;
}

ORC_API int orc_threads(void) {
#ifdef _OPENMP
    return omp_get_max_threads();
#else
    return 1;
#endif
}
