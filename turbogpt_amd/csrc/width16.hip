// The reference's own network behind the plain Config (config.h:4): width 16, 4 heads of 4, vocabulary
// 256, RMSNorm, partial RoPE, causal arg-max attention with a GELU gate, SwiGLU(48); optimizer pair
// mantissa-preserving AdamW + Muon.  Follows cuda/model.cuh:8-99 (op order and bf16 rounding points),
// cuda/ops.cuh:57-144, cuda/attention.cuh:4-106, cuda/optim.cuh:17-119.
//
// The reference runs this model as one persistent kernel over 32-token tiles held in shared memory.
// Here every operator group is a token-parallel kernel: a lane owns one token's 16-wide row in
// registers and reads the (tiny, wave-uniform) weight matrices through the scalar/constant path;
// sequences only meet in the two attention kernels, which read the other positions' keys / values /
// gradients from the saved rows.  Weight gradients are not accumulated by atomics: every matrix,
// RMSNorm scale and embedding row is one job of a single chunked outer-product kernel whose per-chunk
// partials a second kernel folds in chunk order (bit-reproducible; takes the place of
// weight_gradient's read-modify-write and of reduce_gradients, cuda/ops.cuh:83-109, cuda/trainer.cuh:9-47).
#include "common.h"
#include "../../include/tgk_kernels.h"

namespace {

constexpr int W = 16, HEADS = 4, HD = 4, F = 48, V = 256, MAX_DEPTH = 8;
constexpr int CHUNK = 128; // tokens per weight-gradient partial

struct Layer {
    int attention_norm, qkv, attention, mlp_norm, gate, up, down;
};
struct Layout { // model.h:12-37
    int embedding, final_norm, head, count;
    Layer layers[MAX_DEPTH];
};
Layout make_layout(int depth) {
    Layout p{};
    int n = 0;
    auto take = [&](int size) {
        const int offset = n;
        n += size;
        return offset;
    };
    p.embedding = take(V * W);
    for (int l = 0; l < depth; ++l) {
        Layer &b = p.layers[l];
        b.attention_norm = take(W);
        b.qkv = take(3 * W * W);
        b.attention = take(W * W);
        b.mlp_norm = take(W);
        b.gate = take(F * W);
        b.up = take(F * W);
        b.down = take(W * F);
    }
    p.final_norm = take(W);
    p.head = take(V * W);
    p.count = n;
    return p;
}

// Saved rows of one layer (what forward keeps for backward: cuda/types.cuh:40-44 plus the gate/up
// cache of cuda/model.cuh:25-29) and the rows backward leaves for the weight-gradient jobs.
struct LayerRows {
    bf16_t *x, *qkv, *middle, *gu;        // forward: block input, post-RoPE q|k|v, post-attention residual, gate|up
    int *selected;                        // winning key (token row) per (token, head)
    float *gates, *derivatives;           // GELU(top), GELU'(top)
    bf16_t *n1, *a, *n2, *act, *dgu, *dqkv; // backward: operands of the five weight gradients
    bf16_t *dh_down, *dh_attention;        // the residual gradient as the down / attention projections saw it
    float *gz_attention, *gz_mlp;         // per-token g*z of the two RMSNorm scales
};
struct Rows {
    LayerRows layer[MAX_DEPTH];
    bf16_t *hidden, *nf, *dlogits, *dh, *dattn;
    float *dt, *gz_final, *partials;
    size_t bytes;
};
Rows carve(int depth, int tokens, void *base) {
    Rows r{};
    size_t at = 0;
    auto take = [&](size_t bytes) {
        void *p = base ? static_cast<unsigned char *>(base) + at : nullptr;
        at += (bytes + 255) & ~size_t(255);
        return p;
    };
    const size_t N = size_t(tokens);
    for (int l = 0; l < depth; ++l) {
        LayerRows &b = r.layer[l];
        b.x = static_cast<bf16_t *>(take(N * W * 2));
        b.qkv = static_cast<bf16_t *>(take(N * 3 * W * 2));
        b.middle = static_cast<bf16_t *>(take(N * W * 2));
        b.gu = static_cast<bf16_t *>(take(N * 2 * F * 2));
        b.selected = static_cast<int *>(take(N * HEADS * 4));
        b.gates = static_cast<float *>(take(N * HEADS * 4));
        b.derivatives = static_cast<float *>(take(N * HEADS * 4));
        b.n1 = static_cast<bf16_t *>(take(N * W * 2));
        b.a = static_cast<bf16_t *>(take(N * W * 2));
        b.n2 = static_cast<bf16_t *>(take(N * W * 2));
        b.act = static_cast<bf16_t *>(take(N * F * 2));
        b.dgu = static_cast<bf16_t *>(take(N * 2 * F * 2));
        b.dqkv = static_cast<bf16_t *>(take(N * 3 * W * 2));
        b.dh_down = static_cast<bf16_t *>(take(N * W * 2));
        b.dh_attention = static_cast<bf16_t *>(take(N * W * 2));
        b.gz_attention = static_cast<float *>(take(N * W * 4));
        b.gz_mlp = static_cast<float *>(take(N * W * 4));
    }
    r.hidden = static_cast<bf16_t *>(take(N * W * 2));
    r.nf = static_cast<bf16_t *>(take(N * W * 2));
    r.dlogits = static_cast<bf16_t *>(take(N * V * 2));
    r.dh = static_cast<bf16_t *>(take(N * W * 2));
    r.dattn = static_cast<bf16_t *>(take(N * W * 2));
    r.dt = static_cast<float *>(take(N * HEADS * 4));
    r.gz_final = static_cast<float *>(take(N * W * 4));
    const size_t chunks = (N + CHUNK - 1) / CHUNK;
    r.partials = static_cast<float *>(take(chunks * size_t(make_layout(depth).count) * 4));
    r.bytes = at;
    return r;
}

// ---- device helpers ---------------------------------------------------------------------------------
TG_DEVICE float master(const bf16_t *hi, const uint16_t *lo, int i) { // cuda/ops.cuh:6-9
    return __uint_as_float((uint32_t(hi[i]) << 16) | lo[i]);
}
TG_DEVICE void load_row16(const bf16_t *p, float (&v)[16]) {
    const u32x4 a = *reinterpret_cast<const u32x4 *>(p), b = *reinterpret_cast<const u32x4 *>(p + 8);
#pragma unroll
    for (int e = 0; e < 4; ++e) {
        v[2 * e] = bf16_lo(a[e]), v[2 * e + 1] = bf16_hi(a[e]);
        v[8 + 2 * e] = bf16_lo(b[e]), v[8 + 2 * e + 1] = bf16_hi(b[e]);
    }
}
// stores RN_bf16 of 16 values and leaves the rounded values in v
TG_DEVICE void store_row16(bf16_t *p, float (&v)[16]) {
    u32x4 a, b;
#pragma unroll
    for (int e = 0; e < 4; ++e) {
        a[e] = pack_bf16(v[2 * e], v[2 * e + 1]);
        b[e] = pack_bf16(v[8 + 2 * e], v[8 + 2 * e + 1]);
    }
    *reinterpret_cast<u32x4 *>(p) = a;
    *reinterpret_cast<u32x4 *>(p + 8) = b;
#pragma unroll
    for (int e = 0; e < 16; ++e)
        v[e] = round_bf16(v[e]);
}
// y[o] = sum_i x[i] W[o][i], W row-major [OUT][IN] bf16 at wave-uniform addresses
template <int OUT, int IN> TG_DEVICE void matvec(const bf16_t *__restrict__ w, const float (&x)[IN], float (&y)[OUT]) {
#pragma unroll
    for (int o = 0; o < OUT; ++o) {
        float acc = 0.f;
#pragma unroll
        for (int i = 0; i < IN; ++i)
            acc = fmaf(x[i], bf16_to_float(w[o * IN + i]), acc);
        y[o] = acc;
    }
}
// dx[i] = sum_o dy[o] W[o][i]
template <int OUT, int IN> TG_DEVICE void matvec_t(const bf16_t *__restrict__ w, const float (&dy)[OUT], float (&dx)[IN]) {
#pragma unroll
    for (int i = 0; i < IN; ++i)
        dx[i] = 0.f;
#pragma unroll
    for (int o = 0; o < OUT; ++o)
#pragma unroll
        for (int i = 0; i < IN; ++i)
            dx[i] = fmaf(dy[o], bf16_to_float(w[o * IN + i]), dx[i]);
}
// cuda/ops.cuh:57-67: y = RN_bf16(v * rsqrt(mean(v^2) + 1e-6) * scale), scale read in full fp32
TG_DEVICE float inverse_rms(const float (&v)[16]) {
    float sum = 0.f;
#pragma unroll
    for (int i = 0; i < 16; ++i)
        sum = fmaf(v[i], v[i], sum);
    return rsqrtf(sum * (1.f / 16.f) + 1e-6f);
}
TG_DEVICE void normalize(const float (&v)[16], const bf16_t *hi, const uint16_t *lo, int scale, float (&y)[16]) {
    const float inv = inverse_rms(v);
#pragma unroll
    for (int i = 0; i < 16; ++i)
        y[i] = round_bf16(v[i] * inv * master(hi, lo, scale + i));
}
// cuda/ops.cuh:68-80: returns RN_bf16(dx) in dx and the per-token g*z terms of the scale gradient
TG_DEVICE void normalize_backward(const float (&v)[16], const float (&g)[16], const bf16_t *hi, const uint16_t *lo,
                                  int scale, float (&dx)[16], float *gz) {
    const float inv = inverse_rms(v);
    float dot = 0.f, z[16], dz[16];
#pragma unroll
    for (int i = 0; i < 16; ++i) {
        z[i] = v[i] * inv;
        dz[i] = g[i] * master(hi, lo, scale + i);
        dot = fmaf(dz[i], z[i], dot);
    }
#pragma unroll
    for (int i = 0; i < 16; ++i) {
        dx[i] = round_bf16((dz[i] - z[i] * dot * (1.f / 16.f)) * inv);
        gz[i] = g[i] * z[i];
    }
}
// cuda/attention.cuh:19-30: first pair of every query and key head, one radian per position, unfused
TG_DEVICE void rotate(float (&qkv)[48], int position, bool inverse) {
    float s, c;
    // float32(cos k), float32(sin k), k = 0..7 (cuda/attention.cuh:7-14)
    const float cos_table[8] = {1.0f, 0.5403022766113281f, -0.416146844625473f, -0.9899924993515015f,
                                -0.6536436080932617f, 0.28366219997406006f, 0.9601702690124512f, 0.7539022564888f};
    const float sin_table[8] = {0.0f, 0.8414709568023682f, 0.9092974066734314f, 0.14112000167369843f,
                                -0.756802499294281f, -0.9589242935180664f, -0.279415488243103f, 0.6569865942001343f};
    c = cos_table[position];
    s = inverse ? -sin_table[position] : sin_table[position];
#pragma unroll
    for (int pair = 0; pair < 8; ++pair) {
        const int at = pair * 4; // query heads 0-3, then key heads 0-3
        const float x = qkv[at], y = qkv[at + 1];
        qkv[at] = round_bf16(__fsub_rn(__fmul_rn(x, c), __fmul_rn(y, s)));
        qkv[at + 1] = round_bf16(__fadd_rn(__fmul_rn(x, s), __fmul_rn(y, c)));
    }
}
TG_DEVICE float sigmoid(float x) {
    return 1.f / (1.f + expf(-x));
}

struct Model {
    const bf16_t *hi;
    const uint16_t *lo;
    Layout layout;
    int tokens, context;
};

// ---- forward ---------------------------------------------------------------------------------------
__global__ __launch_bounds__(64) void w16_embed_kernel(Model m, const uint8_t *__restrict__ x, bf16_t *hidden) {
    const int t = blockIdx.x * 64 + threadIdx.x;
    if (t >= m.tokens)
        return;
    const bf16_t *row = m.hi + m.layout.embedding + int(x[t]) * W;
    *reinterpret_cast<u32x4 *>(hidden + size_t(t) * W) = *reinterpret_cast<const u32x4 *>(row);
    *reinterpret_cast<u32x4 *>(hidden + size_t(t) * W + 8) = *reinterpret_cast<const u32x4 *>(row + 8);
}

// save block input, RMSNorm, QKV projection, RoPE (cuda/model.cuh:14-19)
__global__ __launch_bounds__(64) void w16_qkv_kernel(Model m, int l, const bf16_t *__restrict__ hidden, LayerRows rows) {
    const int t = blockIdx.x * 64 + threadIdx.x;
    if (t >= m.tokens)
        return;
    const Layer &p = m.layout.layers[l];
    float v[16], n[16], qkv[48];
    load_row16(hidden + size_t(t) * W, v);
    store_row16(rows.x + size_t(t) * W, v);
    normalize(v, m.hi, m.lo, p.attention_norm, n);
    matvec<48, 16>(m.hi + p.qkv, n, qkv);
#pragma unroll
    for (int o = 0; o < 48; ++o)
        qkv[o] = round_bf16(qkv[o]);
    rotate(qkv, t % m.context, false);
    bf16_t *out = rows.qkv + size_t(t) * 48;
#pragma unroll
    for (int o = 0; o < 48; o += 2)
        *reinterpret_cast<uint32_t *>(out + o) = pack_bf16(qkv[o], qkv[o + 1]);
}

// arg-max attention with its GELU gate, output projection and residual (cuda/model.cuh:20-21,
// cuda/attention.cuh:33-71)
__global__ __launch_bounds__(64) void w16_attention_kernel(Model m, int l, LayerRows rows) {
    const int t = blockIdx.x * 64 + threadIdx.x;
    if (t >= m.tokens)
        return;
    const Layer &p = m.layout.layers[l];
    const int start = t / m.context * m.context;
    const bf16_t *mine = rows.qkv + size_t(t) * 48;
    float a[16];
#pragma unroll
    for (int head = 0; head < HEADS; ++head) {
        float q[4];
#pragma unroll
        for (int c = 0; c < 4; ++c)
            q[c] = bf16_to_float(mine[head * 4 + c]);
        float top = -INFINITY;
        int best = start;
        for (int key = start; key <= t; ++key) {
            const bf16_t *k = rows.qkv + size_t(key) * 48 + 16 + head * 4;
            float score = 0.f;
#pragma unroll
            for (int c = 0; c < 4; ++c)
                score += q[c] * bf16_to_float(k[c]);
            if (score > top) { // first index wins ties
                top = score;
                best = key;
            }
        }
        const float e = 1.f + erff(top * 0.7071067811865475f);
        const float gate = 0.5f * top * e;
        rows.selected[size_t(t) * HEADS + head] = best;
        rows.gates[size_t(t) * HEADS + head] = gate;
        rows.derivatives[size_t(t) * HEADS + head] = 0.5f * e + top * 0.3989422804014327f * expf(-0.5f * top * top);
        const bf16_t *value = rows.qkv + size_t(best) * 48 + 32 + head * 4;
#pragma unroll
        for (int c = 0; c < 4; ++c)
            a[head * 4 + c] = round_bf16(bf16_to_float(value[c]) * gate);
    }
    float y[16], x[16];
    matvec<16, 16>(m.hi + p.attention, a, y);
    load_row16(rows.x + size_t(t) * W, x);
#pragma unroll
    for (int o = 0; o < 16; ++o)
        y[o] = round_bf16(y[o]) + x[o]; // bf16 add of the residual (cuda/mma.cuh:95-97)
    store_row16(rows.middle + size_t(t) * W, y);
}

// cuda/ops.cuh:120-131: RN after SiLU and after the product
TG_DEVICE void swiglu_row(const float (&gu)[96], float (&activated)[48], float (&act)[48]) {
#pragma unroll
    for (int j = 0; j < 48; ++j) {
        activated[j] = round_bf16(gu[j] * sigmoid(gu[j]));
        act[j] = round_bf16(activated[j] * gu[48 + j]);
    }
}

// RMSNorm, packed gate|up projection, SwiGLU, down projection and residual (cuda/model.cuh:22-30)
__global__ __launch_bounds__(64) void w16_mlp_kernel(Model m, int l, LayerRows rows, bf16_t *hidden) {
    const int t = blockIdx.x * 64 + threadIdx.x;
    if (t >= m.tokens)
        return;
    const Layer &p = m.layout.layers[l];
    float v[16], n[16], gu[96], activated[48], act[48], y[16];
    load_row16(rows.middle + size_t(t) * W, v);
    normalize(v, m.hi, m.lo, p.mlp_norm, n);
    matvec<96, 16>(m.hi + p.gate, n, gu); // gate and up are adjacent (model.h:27-31)
    bf16_t *cache = rows.gu + size_t(t) * 96;
#pragma unroll
    for (int o = 0; o < 96; o += 2) {
        *reinterpret_cast<uint32_t *>(cache + o) = pack_bf16(gu[o], gu[o + 1]);
        gu[o] = round_bf16(gu[o]), gu[o + 1] = round_bf16(gu[o + 1]);
    }
    swiglu_row(gu, activated, act);
    matvec<16, 48>(m.hi + p.down, act, y);
#pragma unroll
    for (int o = 0; o < 16; ++o)
        y[o] = round_bf16(y[o]) + v[o];
    store_row16(hidden + size_t(t) * W, y);
}

// final RMSNorm, head, softmax cross-entropy; one wave per token, a lane owns four logits
// (cuda/model.cuh:32-58).  dlogits = RN_bf16((p - onehot) / tokens).
__global__ __launch_bounds__(256) void w16_head_kernel(Model m, const bf16_t *__restrict__ hidden, bf16_t *nf,
                                                       const uint8_t *__restrict__ y, float *token_losses,
                                                       float *logits_out, bf16_t *dlogits, int with_gradient) {
    const int lane = threadIdx.x & 63, t = blockIdx.x * 4 + (threadIdx.x >> 6);
    if (t >= m.tokens)
        return;
    float v[16], n[16];
    load_row16(hidden + size_t(t) * W, v);
    normalize(v, m.hi, m.lo, m.layout.final_norm, n);
    if (lane == 0) {
        float copy[16];
#pragma unroll
        for (int i = 0; i < 16; ++i)
            copy[i] = n[i];
        store_row16(nf + size_t(t) * W, copy);
    }
    float logit[4], high = -INFINITY;
#pragma unroll
    for (int k = 0; k < 4; ++k) {
        const int o = lane + 64 * k;
        float w[16], acc = 0.f;
        load_row16(m.hi + m.layout.head + o * W, w);
#pragma unroll
        for (int i = 0; i < 16; ++i)
            acc = fmaf(n[i], w[i], acc);
        logit[k] = round_bf16(acc);
        high = fmaxf(high, logit[k]);
    }
    high = wave_max(high);
    float sum = 0.f;
#pragma unroll
    for (int k = 0; k < 4; ++k)
        sum += expf(logit[k] - high);
    sum = wave_sum(sum);
    const int target = y[t];
    float picked = 0.f;
#pragma unroll
    for (int k = 0; k < 4; ++k)
        picked += (lane + 64 * k == target) ? logit[k] : 0.f;
    picked = wave_sum(picked);
    if (lane == 0)
        token_losses[t] = high + logf(sum) - picked;
#pragma unroll
    for (int k = 0; k < 4; ++k) {
        const int o = lane + 64 * k;
        if (logits_out)
            logits_out[size_t(t) * V + o] = logit[k];
        if (with_gradient)
            dlogits[size_t(t) * V + o] =
                float_to_bf16((expf(logit[k] - high) / sum - (o == target ? 1.f : 0.f)) / float(m.tokens));
    }
}

// ---- backward --------------------------------------------------------------------------------------
// head input gradient and final RMSNorm backward (cuda/model.cuh:63-66)
__global__ __launch_bounds__(64) void w16_head_backward_kernel(Model m, const bf16_t *__restrict__ hidden,
                                                               const bf16_t *__restrict__ dlogits, bf16_t *dh,
                                                               float *gz_final) {
    const int t = blockIdx.x * 64 + threadIdx.x;
    if (t >= m.tokens)
        return;
    float dn[16];
#pragma unroll
    for (int i = 0; i < 16; ++i)
        dn[i] = 0.f;
    const bf16_t *row = dlogits + size_t(t) * V;
    for (int o = 0; o < V; o += 2) {
        const uint32_t pair = *reinterpret_cast<const uint32_t *>(row + o);
        const float d0 = bf16_lo(pair), d1 = bf16_hi(pair);
        const bf16_t *w = m.hi + m.layout.head + o * W;
#pragma unroll
        for (int i = 0; i < 16; ++i)
            dn[i] = fmaf(d1, bf16_to_float(w[W + i]), fmaf(d0, bf16_to_float(w[i]), dn[i]));
    }
    float v[16], dx[16], gz[16];
#pragma unroll
    for (int i = 0; i < 16; ++i)
        dn[i] = round_bf16(dn[i]);
    load_row16(hidden + size_t(t) * W, v);
    normalize_backward(v, dn, m.hi, m.lo, m.layout.final_norm, dx, gz);
    store_row16(dh + size_t(t) * W, dx);
#pragma unroll
    for (int i = 0; i < 16; ++i)
        gz_final[size_t(t) * W + i] = gz[i];
}

// down projection, SwiGLU, packed gate|up projection and RMSNorm backward (cuda/model.cuh:72-88)
__global__ __launch_bounds__(64) void w16_mlp_backward_kernel(Model m, int l, LayerRows rows, bf16_t *dh) {
    const int t = blockIdx.x * 64 + threadIdx.x;
    if (t >= m.tokens)
        return;
    const Layer &p = m.layout.layers[l];
    float v[16], n[16], d[16], gu[96], activated[48], act[48], dact[48], dgu[96];
    load_row16(rows.middle + size_t(t) * W, v);
    load_row16(dh + size_t(t) * W, d);
    store_row16(rows.dh_down + size_t(t) * W, d);
    normalize(v, m.hi, m.lo, p.mlp_norm, n);
    {
        float copy[16];
#pragma unroll
        for (int i = 0; i < 16; ++i)
            copy[i] = n[i];
        store_row16(rows.n2 + size_t(t) * W, copy);
    }
    const bf16_t *cache = rows.gu + size_t(t) * 96;
#pragma unroll
    for (int o = 0; o < 96; o += 2) {
        const uint32_t pair = *reinterpret_cast<const uint32_t *>(cache + o);
        gu[o] = bf16_lo(pair), gu[o + 1] = bf16_hi(pair);
    }
    swiglu_row(gu, activated, act);
    bf16_t *act_out = rows.act + size_t(t) * F;
#pragma unroll
    for (int j = 0; j < 48; j += 2)
        *reinterpret_cast<uint32_t *>(act_out + j) = pack_bf16(act[j], act[j + 1]);
    matvec_t<16, 48>(m.hi + p.down, d, dact);
    // cuda/ops.cuh:133-144
#pragma unroll
    for (int j = 0; j < 48; ++j) {
        const float dy = round_bf16(dact[j]), g = gu[j], u = gu[48 + j], sig = sigmoid(g);
        const float da = round_bf16(dy * u);
        dgu[j] = round_bf16(da * sig * (1.f + g * (1.f - sig)));
        dgu[48 + j] = round_bf16(dy * activated[j]);
    }
    bf16_t *dgu_out = rows.dgu + size_t(t) * 96;
#pragma unroll
    for (int o = 0; o < 96; o += 2)
        *reinterpret_cast<uint32_t *>(dgu_out + o) = pack_bf16(dgu[o], dgu[o + 1]);
    float dn[16], dx[16], gz[16];
    matvec_t<96, 16>(m.hi + p.gate, dgu, dn);
#pragma unroll
    for (int i = 0; i < 16; ++i)
        dn[i] = round_bf16(dn[i]);
    normalize_backward(v, dn, m.hi, m.lo, p.mlp_norm, dx, gz);
#pragma unroll
    for (int i = 0; i < 16; ++i) {
        d[i] = d[i] + dx[i]; // residual gradients stay bf16 between operators (cuda/ops.cuh:74-76)
        rows.gz_mlp[size_t(t) * W + i] = gz[i];
    }
    store_row16(dh + size_t(t) * W, d);
    store_row16(rows.dh_attention + size_t(t) * W, d);
}

// replays the attention output from the cached winner and gate, output-projection backward and the
// per-(token, head) score gradient (cuda/model.cuh:89-91, cuda/attention.cuh:72-85)
__global__ __launch_bounds__(64) void w16_attention_backward_a_kernel(Model m, int l, LayerRows rows,
                                                                      const bf16_t *__restrict__ dh, bf16_t *dattn,
                                                                      float *dt) {
    const int t = blockIdx.x * 64 + threadIdx.x;
    if (t >= m.tokens)
        return;
    const Layer &p = m.layout.layers[l];
    float d[16], a[16], da[16], value[16];
    load_row16(dh + size_t(t) * W, d);
#pragma unroll
    for (int head = 0; head < HEADS; ++head) {
        const int key = rows.selected[size_t(t) * HEADS + head];
        const float gate = rows.gates[size_t(t) * HEADS + head];
        const bf16_t *vrow = rows.qkv + size_t(key) * 48 + 32 + head * 4;
#pragma unroll
        for (int c = 0; c < 4; ++c) {
            value[head * 4 + c] = bf16_to_float(vrow[c]);
            a[head * 4 + c] = value[head * 4 + c] * gate;
        }
    }
    store_row16(rows.a + size_t(t) * W, a);
    matvec_t<16, 16>(m.hi + p.attention, d, da);
    store_row16(dattn + size_t(t) * W, da);
#pragma unroll
    for (int head = 0; head < HEADS; ++head) {
        float sum = 0.f;
#pragma unroll
        for (int c = 0; c < 4; ++c)
            sum += da[head * 4 + c] * value[head * 4 + c];
        dt[size_t(t) * HEADS + head] = sum * rows.derivatives[size_t(t) * HEADS + head];
    }
}

// query / key / value gradients by gathering over the sequence (no atomics), inverse RoPE, QKV
// projection and RMSNorm backward (cuda/attention.cuh:86-106, cuda/model.cuh:92-96)
__global__ __launch_bounds__(64) void w16_attention_backward_b_kernel(Model m, int l, LayerRows rows,
                                                                      const bf16_t *__restrict__ dattn,
                                                                      const float *__restrict__ dt, bf16_t *dh) {
    const int t = blockIdx.x * 64 + threadIdx.x;
    if (t >= m.tokens)
        return;
    const Layer &p = m.layout.layers[l];
    const int start = t / m.context * m.context;
    float dqkv[48];
#pragma unroll
    for (int head = 0; head < HEADS; ++head) {
        const int key = rows.selected[size_t(t) * HEADS + head];
        const float mine = dt[size_t(t) * HEADS + head];
        const bf16_t *krow = rows.qkv + size_t(key) * 48 + 16 + head * 4;
        float dk[4] = {0.f, 0.f, 0.f, 0.f}, dv[4] = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int c = 0; c < 4; ++c)
            dqkv[head * 4 + c] = mine * bf16_to_float(krow[c]);
        for (int query = start; query < start + m.context; ++query) {
            if (rows.selected[size_t(query) * HEADS + head] != t)
                continue;
            const float their = dt[size_t(query) * HEADS + head], gate = rows.gates[size_t(query) * HEADS + head];
            const bf16_t *qrow = rows.qkv + size_t(query) * 48 + head * 4;
            const bf16_t *drow = dattn + size_t(query) * W + head * 4;
#pragma unroll
            for (int c = 0; c < 4; ++c) {
                dk[c] += their * bf16_to_float(qrow[c]);
                dv[c] += bf16_to_float(drow[c]) * gate;
            }
        }
#pragma unroll
        for (int c = 0; c < 4; ++c) {
            dqkv[16 + head * 4 + c] = dk[c];
            dqkv[32 + head * 4 + c] = dv[c];
        }
    }
#pragma unroll
    for (int o = 0; o < 48; ++o)
        dqkv[o] = round_bf16(dqkv[o]);
    rotate(dqkv, t % m.context, true);
    bf16_t *out = rows.dqkv + size_t(t) * 48;
#pragma unroll
    for (int o = 0; o < 48; o += 2)
        *reinterpret_cast<uint32_t *>(out + o) = pack_bf16(dqkv[o], dqkv[o + 1]);
    float v[16], n[16], d[16], dn[16], dx[16], gz[16];
    load_row16(rows.x + size_t(t) * W, v);
    normalize(v, m.hi, m.lo, p.attention_norm, n);
    store_row16(rows.n1 + size_t(t) * W, n);
    matvec_t<48, 16>(m.hi + p.qkv, dqkv, dn);
#pragma unroll
    for (int i = 0; i < 16; ++i)
        dn[i] = round_bf16(dn[i]);
    normalize_backward(v, dn, m.hi, m.lo, p.attention_norm, dx, gz);
    load_row16(dh + size_t(t) * W, d);
#pragma unroll
    for (int i = 0; i < 16; ++i) {
        d[i] = d[i] + dx[i];
        rows.gz_attention[size_t(t) * W + i] = gz[i];
    }
    store_row16(dh + size_t(t) * W, d);
}

// ---- weight gradients: one job per parameter tensor ----------------------------------------------------
enum JobKind { JOB_OUTER = 0, JOB_COLUMN_SUM = 1, JOB_EMBEDDING = 2 };
struct Job {
    const void *dy; // OUTER: bf16 [tokens][ld_dy]; COLUMN_SUM: float [tokens][16]; EMBEDDING: uint8 token ids
    const bf16_t *x; // OUTER: bf16 [tokens][ld_x]; EMBEDDING: bf16 [tokens][16]
    int ld_dy, ld_x, out, in, offset, kind;
};
constexpr int MAX_JOBS = 3 + MAX_DEPTH * 6;
struct Jobs {
    Job job[MAX_JOBS];
    int count;
};
// partial[chunk][offset + o*in + i] = sum over the chunk's tokens, in token order.  A thread owns output row o
// and a 16-wide slab of inputs: per token it reads one dy value and one 32-byte row piece that every thread of
// the same slab shares, and keeps 16 sums in registers.  (The widest jobs, head and embedding, are 256 x 16.)
__global__ __launch_bounds__(256) void w16_weight_gradient_kernel(Jobs jobs, int tokens, int parameters, float *partials) {
    const Job &job = jobs.job[blockIdx.y];
    const int first = blockIdx.x * CHUNK, last = min(first + CHUNK, tokens);
    const int slabs = job.in >> 4, o = threadIdx.x / slabs, slab = threadIdx.x - o * slabs;
    if (o >= job.out)
        return;
    float acc[16];
#pragma unroll
    for (int k = 0; k < 16; ++k)
        acc[k] = 0.f;
    if (job.kind == JOB_OUTER) {
        const bf16_t *dy = static_cast<const bf16_t *>(job.dy) + o;
        const bf16_t *x = job.x + slab * 16;
        for (int t = first; t < last; ++t) {
            const float d = bf16_to_float(dy[size_t(t) * job.ld_dy]);
            float v[16];
            load_row16(x + size_t(t) * job.ld_x, v);
#pragma unroll
            for (int k = 0; k < 16; ++k)
                acc[k] = fmaf(d, v[k], acc[k]);
        }
    } else if (job.kind == JOB_COLUMN_SUM) {
        const float *gz = static_cast<const float *>(job.dy);
        for (int t = first; t < last; ++t)
#pragma unroll
            for (int k = 0; k < 16; ++k)
                acc[k] += gz[size_t(t) * W + k];
    } else {
        const uint8_t *ids = static_cast<const uint8_t *>(job.dy);
        for (int t = first; t < last; ++t) {
            if (ids[t] != o)
                continue;
            float v[16];
            load_row16(job.x + size_t(t) * W, v);
#pragma unroll
            for (int k = 0; k < 16; ++k)
                acc[k] += v[k];
        }
    }
    float *out = partials + size_t(blockIdx.x) * parameters + job.offset + o * job.in + slab * 16;
#pragma unroll
    for (int k = 0; k < 16; k += 4)
        *reinterpret_cast<f32x4 *>(out + k) = f32x4{acc[k], acc[k + 1], acc[k + 2], acc[k + 3]};
}
__global__ __launch_bounds__(256) void w16_fold_kernel(const float *__restrict__ partials, int chunks, int parameters,
                                                       float *gradient) {
    const int i = blockIdx.x * 256 + threadIdx.x;
    if (i >= parameters)
        return;
    float sum = 0.f;
    for (int c = 0; c < chunks; ++c)
        sum += partials[size_t(c) * parameters + i];
    gradient[i] = sum;
}

// ---- Muon for the hidden matrices: one block per matrix (cuda/optim.cuh:17-62, :107-118) ---------------
struct MuonArgs {
    float clip, lr, momentum, weight_decay;
    int ns_steps, norm_count;
};
__global__ __launch_bounds__(256) void w16_muon_kernel(Layout layout, bf16_t *hi, uint16_t *lo, float *momentum,
                                                       const float *__restrict__ gradient,
                                                       const float *__restrict__ norm_partials, MuonArgs a) {
    __shared__ float wide[16 * 48], product[16 * 48], gram[256], work[256], waves[4], shared_scalar;
    const Layer &p = layout.layers[blockIdx.x / 5];
    const int type = blockIdx.x % 5;
    const int weight = type == 0 ? p.qkv : type == 1 ? p.attention : type == 2 ? p.gate : type == 3 ? p.up : p.down;
    const int rows = (type == 0 || type == 2 || type == 3) ? 48 : 16, cols = type == 4 ? 48 : 16;
    const int n = rows > cols ? rows : cols, size = rows * cols, tid = threadIdx.x;

    float clip = 1.f;
    if (a.clip > 0.f) { // the same fold of the same partials as the AdamW kernel (cuda/optim.cuh:67-80)
        float sum = 0.f;
        for (int i = tid; i < a.norm_count; i += 256)
            sum += norm_partials[i];
        sum = wave_sum(sum);
        if ((tid & 63) == 0)
            waves[tid >> 6] = sum;
        __syncthreads();
        if (tid == 0)
            shared_scalar = fminf(1.f, a.clip / (sqrtf((waves[0] + waves[1]) + (waves[2] + waves[3])) + 1e-6f));
        __syncthreads();
        clip = shared_scalar;
        __syncthreads();
    }
    float squares = 0.f;
    for (int i = tid; i < size; i += 256) {
        const float g = gradient[weight + i] * clip;
        const float m = momentum[weight + i] + (1.f - a.momentum) * (g - momentum[weight + i]);
        momentum[weight + i] = m;
        const float b = round_bf16(g + a.momentum * (m - g));
        wide[rows > cols ? (i % cols) * rows + i / cols : i] = b; // kept as a 16 x n matrix
        squares += b * b;
    }
    squares = wave_sum(squares);
    if ((tid & 63) == 0)
        waves[tid >> 6] = squares;
    __syncthreads();
    if (tid == 0)
        shared_scalar = fmaxf(round_bf16(sqrtf((waves[0] + waves[1]) + (waves[2] + waves[3]))), round_bf16(1e-7f));
    __syncthreads();
    const float norm = shared_scalar;
    for (int i = tid; i < size; i += 256)
        wide[i] = round_bf16(wide[i] / norm);
    __syncthreads();
    for (int step = 0; step < a.ns_steps; ++step) {
        { // A = X X^T, kept in bf16
            const int r = tid >> 4, c = tid & 15;
            float acc = 0.f;
            for (int k = 0; k < n; ++k)
                acc = fmaf(wide[r * n + k], wide[c * n + k], acc);
            gram[tid] = round_bf16(acc);
        }
        __syncthreads();
        { // -4.775 A + 2.0315 A A
            const int r = tid >> 4, c = tid & 15;
            float acc = 0.f;
#pragma unroll
            for (int k = 0; k < 16; ++k)
                acc = fmaf(gram[r * 16 + k], gram[k * 16 + c], acc);
            work[tid] = round_bf16(-4.775f * gram[tid] + 2.0315f * acc);
        }
        __syncthreads();
        for (int i = tid; i < size; i += 256) {
            const int r = i / n, c = i - r * n;
            float acc = 0.f;
#pragma unroll
            for (int k = 0; k < 16; ++k)
                acc = fmaf(work[r * 16 + k], wide[k * n + c], acc);
            product[i] = acc;
        }
        __syncthreads();
        for (int i = tid; i < size; i += 256)
            wide[i] = round_bf16(3.4445f * wide[i] + product[i]);
        __syncthreads();
    }
    const float adjusted = a.lr * sqrtf(fmaxf(1.f, float(rows) / float(cols)));
    for (int i = tid; i < size; i += 256) {
        const int index = rows > cols ? (i % cols) * rows + i / cols : i;
        const float w = master(hi, lo, weight + i) * (1.f - a.lr * a.weight_decay);
        const uint32_t bits = __float_as_uint(w - adjusted * wide[index]);
        hi[weight + i] = uint16_t(bits >> 16); // cuda/ops.cuh:10-14
        lo[weight + i] = uint16_t(bits);
    }
}

void check_shape(int depth, int batch, int context) {
    require(depth >= 1 && depth <= MAX_DEPTH, "w16: depth must be 1..8");
    require(context >= 1 && context <= 8, "w16: context must be 1..8 (the RoPE table has eight entries)");
    require(batch >= 1, "w16: empty batch");
    require(int64_t(batch) * context <= (1 << 24), "w16: too many tokens");
}
Model make_model(int depth, int batch, int context, const uint16_t *hi, const uint16_t *lo) {
    return Model{hi, lo, make_layout(depth), batch * context, context};
}

} // namespace

extern "C" int tgk_w16_parameter_count(int depth) {
    return depth >= 1 && depth <= MAX_DEPTH ? make_layout(depth).count : 0;
}

extern "C" size_t tgk_w16_workspace(int depth, int batch, int context) {
    if (depth < 1 || depth > MAX_DEPTH || batch < 1 || context < 1 || context > 8)
        return 0;
    return carve(depth, batch * context, nullptr).bytes;
}

extern "C" int tgk_w16_forward(hipStream_t stream, int depth, int batch, int context, const uint16_t *weight_hi,
                               const uint16_t *weight_lo, const uint8_t *x, const uint8_t *y, void *workspace,
                               float *token_losses, float *logits, int with_gradient) {
    return guarded([&] {
        check_shape(depth, batch, context);
        require(weight_hi && weight_lo && x && y && workspace && token_losses, "w16_forward: missing operand");
        require(!(reinterpret_cast<uintptr_t>(workspace) & 255), "w16_forward: workspace must be 256-byte aligned");
        const Model m = make_model(depth, batch, context, weight_hi, weight_lo);
        const Rows r = carve(depth, m.tokens, workspace);
        const dim3 per_token((m.tokens + 63) / 64), wave(64);
        hipLaunchKernelGGL(w16_embed_kernel, per_token, wave, 0, stream, m, x, r.hidden);
        for (int l = 0; l < depth; ++l) {
            hipLaunchKernelGGL(w16_qkv_kernel, per_token, wave, 0, stream, m, l, r.hidden, r.layer[l]);
            hipLaunchKernelGGL(w16_attention_kernel, per_token, wave, 0, stream, m, l, r.layer[l]);
            hipLaunchKernelGGL(w16_mlp_kernel, per_token, wave, 0, stream, m, l, r.layer[l], r.hidden);
        }
        hipLaunchKernelGGL(w16_head_kernel, dim3((m.tokens + 3) / 4), dim3(256), 0, stream, m, r.hidden, r.nf, y,
                           token_losses, logits, r.dlogits, with_gradient);
        check_hip(hipGetLastError(), "w16_forward launch: ");
    });
}

extern "C" int tgk_w16_backward(hipStream_t stream, int depth, int batch, int context, const uint16_t *weight_hi,
                                const uint16_t *weight_lo, const uint8_t *x, void *workspace, float *gradient) {
    return guarded([&] {
        check_shape(depth, batch, context);
        require(weight_hi && weight_lo && x && workspace && gradient, "w16_backward: missing operand");
        require(!(reinterpret_cast<uintptr_t>(workspace) & 255), "w16_backward: workspace must be 256-byte aligned");
        const Model m = make_model(depth, batch, context, weight_hi, weight_lo);
        const Rows r = carve(depth, m.tokens, workspace);
        const dim3 per_token((m.tokens + 63) / 64), wave(64);
        hipLaunchKernelGGL(w16_head_backward_kernel, per_token, wave, 0, stream, m, r.hidden, r.dlogits, r.dh, r.gz_final);
        for (int l = depth - 1; l >= 0; --l) {
            hipLaunchKernelGGL(w16_mlp_backward_kernel, per_token, wave, 0, stream, m, l, r.layer[l], r.dh);
            hipLaunchKernelGGL(w16_attention_backward_a_kernel, per_token, wave, 0, stream, m, l, r.layer[l], r.dh, r.dattn,
                               r.dt);
            hipLaunchKernelGGL(w16_attention_backward_b_kernel, per_token, wave, 0, stream, m, l, r.layer[l], r.dattn, r.dt,
                               r.dh);
        }
        Jobs jobs{};
        auto add = [&](const void *dy, int ld_dy, const bf16_t *xs, int ld_x, int out, int in, int offset, int kind) {
            jobs.job[jobs.count++] = Job{dy, xs, ld_dy, ld_x, out, in, offset, kind};
        };
        const Layout &p = m.layout;
        add(x, 0, r.dh, W, V, W, p.embedding, JOB_EMBEDDING);
        for (int l = 0; l < depth; ++l) {
            const LayerRows &b = r.layer[l];
            const Layer &q = p.layers[l];
            add(b.gz_attention, W, nullptr, 0, 1, W, q.attention_norm, JOB_COLUMN_SUM);
            add(b.dqkv, 3 * W, b.n1, W, 3 * W, W, q.qkv, JOB_OUTER);
            add(b.dh_attention, W, b.a, W, W, W, q.attention, JOB_OUTER);
            add(b.gz_mlp, W, nullptr, 0, 1, W, q.mlp_norm, JOB_COLUMN_SUM);
            add(b.dgu, 2 * F, b.n2, W, 2 * F, W, q.gate, JOB_OUTER); // gate and up are adjacent: one packed job
            add(b.dh_down, W, b.act, F, W, F, q.down, JOB_OUTER);
        }
        add(r.gz_final, W, nullptr, 0, 1, W, p.final_norm, JOB_COLUMN_SUM);
        add(r.dlogits, V, r.nf, W, V, W, p.head, JOB_OUTER);
        const int chunks = (m.tokens + CHUNK - 1) / CHUNK;
        hipLaunchKernelGGL(w16_weight_gradient_kernel, dim3(chunks, jobs.count), dim3(256), 0, stream, jobs, m.tokens,
                           p.count, r.partials);
        hipLaunchKernelGGL(w16_fold_kernel, dim3((p.count + 255) / 256), dim3(256), 0, stream, r.partials, chunks,
                           p.count, gradient);
        check_hip(hipGetLastError(), "w16_backward launch: ");
    });
}

extern "C" int tgk_w16_muon(hipStream_t stream, int depth, uint16_t *weight_hi, uint16_t *weight_lo, float *momentum,
                            const float *gradient, const float *norm_partials, int norm_count, float clip, float lr,
                            float momentum_rate, float weight_decay, int ns_steps) {
    return guarded([&] {
        require(depth >= 1 && depth <= MAX_DEPTH, "w16_muon: depth must be 1..8");
        require(weight_hi && weight_lo && momentum && gradient, "w16_muon: missing operand");
        require(!(clip > 0.f) || (norm_partials && norm_count > 0), "w16_muon: clipping needs the norm partials");
        require(ns_steps >= 1 && ns_steps <= 10, "w16_muon: ns_steps must be 1..10");
        const MuonArgs a{clip, lr, momentum_rate, weight_decay, ns_steps, norm_count};
        hipLaunchKernelGGL(w16_muon_kernel, dim3(depth * 5), dim3(256), 0, stream, make_layout(depth), weight_hi,
                           weight_lo, momentum, gradient, norm_partials, a);
        check_hip(hipGetLastError(), "w16_muon launch: ");
    });
}
