// HBM-bound operators of the training step for gfx950: embedding, LayerNorm, cross-entropy,
// AdamW on hi/lo split weights, batch sampling, loss bookkeeping.  Each stands in for a device
// function of the reference named at its entry point.  All are single pass over their operands
// with 16-byte accesses; reductions use a fixed order (no atomics), so results are reproducible.
#include "common.h"
#include "../../include/tgk_kernels.h"

namespace {

constexpr int MAX_LN_CHUNKS = 4; // 16-byte chunks per lane: rows up to 4*64*8 = 2048 columns

TG_DEVICE void unpack8(const u32x4 &v, float (&f)[8]) {
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        f[2 * i] = bf16_lo(v[i]);
        f[2 * i + 1] = bf16_hi(v[i]);
    }
}
TG_DEVICE u32x4 pack8(const float (&f)[8]) {
    u32x4 v;
#pragma unroll
    for (int i = 0; i < 4; ++i)
        v[i] = pack_bf16(f[2 * i], f[2 * i + 1]);
    return v;
}
// fp32 master values of 8 consecutive parameters from their (hi, lo) halves (cuda/ops.cuh:6-9)
TG_DEVICE void join8(const u32x4 &h, const u32x4 &l, float (&f)[8]) {
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        f[2 * i] = __uint_as_float((h[i] << 16) | (l[i] & 0xffffu));
        f[2 * i + 1] = __uint_as_float((h[i] & 0xffff0000u) | (l[i] >> 16));
    }
}
TG_DEVICE void join8(const uint16_t *hi, const uint16_t *lo, float (&f)[8]) {
    join8(*reinterpret_cast<const u32x4 *>(hi), *reinterpret_cast<const u32x4 *>(lo), f);
}
TG_DEVICE uint64_t hash_u64(uint64_t x) { // utils.h:13-18
    x += 0x9e3779b97f4a7c15ULL;
    x = (x ^ (x >> 30)) * 0xbf58476d1ce4e5b9ULL;
    x = (x ^ (x >> 27)) * 0x94d049bb133111ebULL;
    return x ^ (x >> 31);
}

// ---- embedding ------------------------------------------------------------------------------
__global__ __launch_bounds__(256) void embed_fwd_kernel(const uint8_t *__restrict__ x,
                                                        const bf16_t *__restrict__ table,
                                                        const bf16_t *__restrict__ positions,
                                                        bf16_t *__restrict__ out, int rows, int T,
                                                        int D) {
    const int chunks = D >> 3;
    const size_t total = size_t(rows) * chunks;
    for (size_t i = blockIdx.x * size_t(256) + threadIdx.x; i < total; i += size_t(gridDim.x) * 256) {
        const int row = int(i / chunks), c = int(i % chunks) * 8;
        float a[8], b[8];
        unpack8(*reinterpret_cast<const u32x4 *>(table + size_t(x[row]) * D + c), a);
        unpack8(*reinterpret_cast<const u32x4 *>(positions + size_t(row % T) * D + c), b);
#pragma unroll
        for (int k = 0; k < 8; ++k)
            a[k] += b[k];
        *reinterpret_cast<u32x4 *>(out + size_t(row) * D + c) = pack8(a);
    }
}

// dTable[v][c] = sum over tokens t with x[t] == v of dh[t][c].  Pass 1: one wave per (64 columns,
// token segment) walks its segment in token order and adds each row slice into a [256][64] fp32
// table in LDS (each lane owns one column, LDS adds retire in program order: fixed summation
// order), then dumps the table.  Pass 2 folds the segment tables in segment order.
constexpr int EMBED_SEGMENT = 1024; // tokens per segment
__global__ __launch_bounds__(64) void embed_bwd_partial_kernel(const uint8_t *__restrict__ x,
                                                               const bf16_t *__restrict__ dh,
                                                               float *__restrict__ partial, int rows, int D) {
    __shared__ float table[256 * 64];
    const int lane = threadIdx.x, col = blockIdx.x * 64 + lane, segment = blockIdx.y;
    for (int i = lane; i < 256 * 64; i += 64)
        table[i] = 0.f;
    __syncthreads();
    const int begin = segment * EMBED_SEGMENT, end = begin + EMBED_SEGMENT < rows ? begin + EMBED_SEGMENT : rows;
#pragma unroll 8
    for (int t = begin; t < end; ++t)
        atomicAdd(&table[int(x[t]) * 64 + lane], bf16_to_float(dh[size_t(t) * D + col]));
    __syncthreads();
    float *out = partial + size_t(segment) * 256 * D + col;
    for (int v = 0; v < 256; ++v)
        out[size_t(v) * D] = table[v * 64 + lane];
}
__global__ __launch_bounds__(256) void embed_bwd_fold_kernel(const float *__restrict__ partial, int segments,
                                                             float *__restrict__ dtable, size_t count,
                                                             int accumulate) {
    const size_t i = blockIdx.x * size_t(256) + threadIdx.x;
    if (i >= count)
        return;
    float sum = 0.f;
    for (int s = 0; s < segments; ++s)
        sum += partial[size_t(s) * count + i];
    dtable[i] = accumulate ? dtable[i] + sum : sum;
}
// onehot[t][v] = (x[t] == v) in bf16; one thread writes 8 columns
__global__ __launch_bounds__(256) void onehot_kernel(const uint8_t *__restrict__ x, bf16_t *__restrict__ onehot,
                                                     int rows) {
    const size_t total = size_t(rows) * 32;
    for (size_t i = blockIdx.x * size_t(256) + threadIdx.x; i < total; i += size_t(gridDim.x) * 256) {
        const int t = int(i >> 5), c0 = int(i & 31) * 8, hot = int(x[t]) - c0;
        u32x4 v = {0, 0, 0, 0};
        if (hot >= 0 && hot < 8)
            v[hot >> 1] = (hot & 1) ? 0x3f800000u : 0x00003f80u; // bf16 1.0 in the high / low half
        *reinterpret_cast<u32x4 *>(onehot + size_t(t) * 256 + c0) = v;
    }
}
// dPositions[p][c] = sum over sequences b of dh[b*T + p][c]
__global__ __launch_bounds__(256) void embed_bwd_positions_kernel(const bf16_t *__restrict__ dh,
                                                                  float *__restrict__ dpos, int B, int T,
                                                                  int D, int accumulate) {
    const size_t total = size_t(T) * D;
    for (size_t i = blockIdx.x * size_t(256) + threadIdx.x; i < total; i += size_t(gridDim.x) * 256) {
        float sum = 0.f;
        for (int b = 0; b < B; ++b)
            sum += bf16_to_float(dh[size_t(b) * total + i]);
        dpos[i] = accumulate ? dpos[i] + sum : sum;
    }
}

// ---- LayerNorm --------------------------------------------------------------------------------
// A row lives in the registers of GROUP lanes (two-pass mean / variance), NC 16-byte chunks per lane
// (D <= NC * GROUP * 8).  GROUP = 64: one row per wave.  GROUP = 32: two rows per wave, which fits
// D = 768 (96 chunks = 32 x 3) without idle lane slots and keeps three loads per array in flight.
// Sum over the GROUP lanes of a row, result in every lane: four DPP steps inside a row of 16 lanes, then the
// gfx950 lane-swap instructions across rows - all on the vector ALU, no LDS round trips (ds_bpermute, which
// __shfl_xor compiles to, costs an LDS latency per step and these sums sit on every row's critical path).
TG_DEVICE float dpp_add(float x, int control) {
    // control: 0xB1 quad_perm [1,0,3,2], 0x4E quad_perm [2,3,0,1], 0x141 row_half_mirror, 0x140 row_mirror
    switch (control) {
    case 0xB1: return x + __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, x), 0xB1, 0xF, 0xF, true));
    case 0x4E: return x + __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, x), 0x4E, 0xF, 0xF, true));
    case 0x141: return x + __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, x), 0x141, 0xF, 0xF, true));
    default: return x + __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, x), 0x140, 0xF, 0xF, true));
    }
}
template <int GROUP> TG_DEVICE float group_sum(float x) {
    x = dpp_add(x, 0xB1);
    x = dpp_add(x, 0x4E);
    x = dpp_add(x, 0x141);
    x = dpp_add(x, 0x140); // every lane of a 16-lane row holds the row's sum
    const auto rows = __builtin_amdgcn_permlane16_swap(__float_as_uint(x), __float_as_uint(x), false, false);
    x = __uint_as_float(rows[0]) + __uint_as_float(rows[1]); // rows 0+1 and 2+3
    if (GROUP == 64) {
        const auto halves = __builtin_amdgcn_permlane32_swap(__float_as_uint(x), __float_as_uint(x), false, false);
        x = __uint_as_float(halves[0]) + __uint_as_float(halves[1]);
    }
    return x;
}
template <int NC, int GROUP>
__global__ __launch_bounds__(256) void layernorm_fwd_kernel(const bf16_t *__restrict__ x,
                                                            const uint16_t *__restrict__ gamma_hi,
                                                            const uint16_t *__restrict__ gamma_lo,
                                                            const uint16_t *__restrict__ beta_hi,
                                                            const uint16_t *__restrict__ beta_lo,
                                                            bf16_t *__restrict__ y, int rows, int D,
                                                            float eps) {
    constexpr int PER_BLOCK = 256 / GROUP; // rows a block works on at a time
    const int lane = threadIdx.x & (GROUP - 1), slot = threadIdx.x / GROUP, chunks = D >> 3;
    const float inv_d = 1.0f / D;
    // gamma and beta are fetched once, ahead of the first row, and stay packed until they are used: behind
    // the row's reductions they would add a second memory latency to every row
    u32x4 g_hi[NC], g_lo[NC], b_hi[NC], b_lo[NC];
#pragma unroll
    for (int j = 0; j < NC; ++j) {
        const int c = lane + j * GROUP;
        if (c < chunks) {
            g_hi[j] = *reinterpret_cast<const u32x4 *>(gamma_hi + c * 8);
            g_lo[j] = *reinterpret_cast<const u32x4 *>(gamma_lo + c * 8);
            b_hi[j] = *reinterpret_cast<const u32x4 *>(beta_hi + c * 8);
            b_lo[j] = *reinterpret_cast<const u32x4 *>(beta_lo + c * 8);
        }
    }
    // the row loop is uniform over the wave: a wave's second half may run one row past the end.  The next
    // row's chunks are requested before the current row is reduced.
    const int stride = gridDim.x * PER_BLOCK;
    u32x4 raw[NC];
    auto fetch = [&](int row, u32x4 (&into)[NC]) {
#pragma unroll
        for (int j = 0; j < NC; ++j) {
            const int c = lane + j * GROUP;
            into[j] = u32x4{0, 0, 0, 0};
            if (row < rows && c < chunks)
                into[j] = *reinterpret_cast<const u32x4 *>(x + size_t(row) * D + c * 8);
        }
    };
    fetch(blockIdx.x * PER_BLOCK + slot, raw);
    for (int row0 = blockIdx.x * PER_BLOCK; row0 < rows; row0 += stride) {
        const int row = row0 + slot;
        const bool live = row < rows;
        u32x4 next[NC];
        fetch(row0 + stride < rows ? row + stride : rows, next);
        float v[NC][8];
        float sum = 0.f;
#pragma unroll
        for (int j = 0; j < NC; ++j) {
            const int c = lane + j * GROUP;
#pragma unroll
            for (int k = 0; k < 8; ++k)
                v[j][k] = 0.f;
            if (live && c < chunks) {
                unpack8(raw[j], v[j]);
#pragma unroll
                for (int k = 0; k < 8; ++k)
                    sum += v[j][k];
            }
            raw[j] = next[j];
        }
        const float mean = group_sum<GROUP>(sum) * inv_d;
        float sq = 0.f;
#pragma unroll
        for (int j = 0; j < NC; ++j)
            if (lane + j * GROUP < chunks)
#pragma unroll
                for (int k = 0; k < 8; ++k) {
                    v[j][k] -= mean;
                    sq += v[j][k] * v[j][k];
                }
        const float inv = 1.0f / sqrtf(group_sum<GROUP>(sq) * inv_d + eps);
#pragma unroll
        for (int j = 0; j < NC; ++j) {
            const int c = lane + j * GROUP;
            if (live && c < chunks) {
                float gm[8], bt[8], o[8];
                join8(g_hi[j], g_lo[j], gm);
                join8(b_hi[j], b_lo[j], bt);
#pragma unroll
                for (int k = 0; k < 8; ++k)
                    o[k] = v[j][k] * inv * gm[k] + bt[k];
                *reinterpret_cast<u32x4 *>(y + size_t(row) * D + c * 8) = pack8(o);
            }
        }
    }
}

// dx (+ residual), and per-block partial sums of dgamma / dbeta into partial[block][2][D].
template <int NC, int GROUP>
__global__ __launch_bounds__(256) void layernorm_bwd_kernel(const bf16_t *__restrict__ x,
                                                            const bf16_t *__restrict__ dy,
                                                            const uint16_t *__restrict__ gamma_hi,
                                                            const uint16_t *__restrict__ gamma_lo,
                                                            const bf16_t *residual, bf16_t *dx,
                                                            float *__restrict__ partial, int rows, int D,
                                                            float eps) {
    constexpr int PER_BLOCK = 256 / GROUP;
    extern __shared__ float lds[]; // [PER_BLOCK row slots][2][D]
    const int lane = threadIdx.x & (GROUP - 1), slot = threadIdx.x / GROUP, chunks = D >> 3;
    const float inv_d = 1.0f / D;
    float dg[NC][8], db[NC][8], gm[NC][8];
#pragma unroll
    for (int j = 0; j < NC; ++j) {
        const int c = lane + j * GROUP;
#pragma unroll
        for (int k = 0; k < 8; ++k)
            dg[j][k] = db[j][k] = gm[j][k] = 0.f;
        if (c < chunks)
            join8(gamma_hi + c * 8, gamma_lo + c * 8, gm[j]);
    }
    for (int row0 = blockIdx.x * PER_BLOCK; row0 < rows; row0 += gridDim.x * PER_BLOCK) {
        const int row = row0 + slot;
        const bool live = row < rows;
        // the row's residual gradient is only needed at the end, but requested with x and dy: behind the
        // reductions it would add a second memory latency to every row
        u32x4 prior_raw[NC];
        float v[NC][8], g[NC][8];
        float sum = 0.f;
#pragma unroll
        for (int j = 0; j < NC; ++j) {
            const int c = lane + j * GROUP;
            prior_raw[j] = u32x4{0, 0, 0, 0};
#pragma unroll
            for (int k = 0; k < 8; ++k)
                v[j][k] = g[j][k] = 0.f;
            if (live && c < chunks) {
                const u32x4 rx = *reinterpret_cast<const u32x4 *>(x + size_t(row) * D + c * 8);
                const u32x4 rg = *reinterpret_cast<const u32x4 *>(dy + size_t(row) * D + c * 8);
                if (residual) // may be dx itself: every lane reads its chunk before it writes it
                    prior_raw[j] = *reinterpret_cast<const u32x4 *>(residual + size_t(row) * D + c * 8);
                unpack8(rx, v[j]);
                unpack8(rg, g[j]);
#pragma unroll
                for (int k = 0; k < 8; ++k)
                    sum += v[j][k];
            }
        }
        const float mean = group_sum<GROUP>(sum) * inv_d;
        float sq = 0.f;
#pragma unroll
        for (int j = 0; j < NC; ++j)
            if (lane + j * GROUP < chunks)
#pragma unroll
                for (int k = 0; k < 8; ++k) {
                    v[j][k] -= mean;
                    sq += v[j][k] * v[j][k];
                }
        const float inv = 1.0f / sqrtf(group_sum<GROUP>(sq) * inv_d + eps);
        float s1 = 0.f, s2 = 0.f;
#pragma unroll
        for (int j = 0; j < NC; ++j)
            if (live && lane + j * GROUP < chunks)
#pragma unroll
                for (int k = 0; k < 8; ++k) {
                    const float z = v[j][k] * inv, dz = g[j][k] * gm[j][k];
                    v[j][k] = z;
                    s1 += dz;
                    s2 += dz * z;
                    dg[j][k] += g[j][k] * z;
                    db[j][k] += g[j][k];
                }
        s1 = group_sum<GROUP>(s1) * inv_d;
        s2 = group_sum<GROUP>(s2) * inv_d;
#pragma unroll
        for (int j = 0; j < NC; ++j) {
            const int c = lane + j * GROUP;
            if (live && c < chunks) {
                float o[8];
#pragma unroll
                for (int k = 0; k < 8; ++k)
                    o[k] = (g[j][k] * gm[j][k] - s1 - v[j][k] * s2) * inv;
                bf16_t *p = dx + size_t(row) * D + c * 8;
                if (residual) {
                    // residual gradients stay in bf16 between operators (cuda/ops.cuh:74-76)
                    float prior[8];
                    unpack8(prior_raw[j], prior);
#pragma unroll
                    for (int k = 0; k < 8; ++k)
                        o[k] = prior[k] + round_bf16(o[k]);
                }
                *reinterpret_cast<u32x4 *>(p) = pack8(o);
            }
        }
    }
    float *mine = lds + slot * 2 * D;
#pragma unroll
    for (int j = 0; j < NC; ++j) {
        const int c = lane + j * GROUP;
        if (c < chunks)
#pragma unroll
            for (int k = 0; k < 8; ++k) {
                mine[c * 8 + k] = dg[j][k];
                mine[D + c * 8 + k] = db[j][k];
            }
    }
    __syncthreads();
    for (int i = threadIdx.x; i < 2 * D; i += 256) {
        float sum = 0.f;
#pragma unroll
        for (int r = 0; r < PER_BLOCK; ++r) // fixed order
            sum += lds[r * 2 * D + i];
        partial[size_t(blockIdx.x) * 2 * D + i] = sum;
    }
}
// dgamma[c] (+)= sum_b partial[b][0][c], dbeta likewise.  16 columns x 16 row phases per block; every
// thread keeps 8 independent loads in flight; phases are combined in a fixed order.
__global__ __launch_bounds__(256) void layernorm_bwd_reduce_kernel(const float *__restrict__ partial,
                                                                   int blocks, int D,
                                                                   float *__restrict__ dgamma,
                                                                   float *__restrict__ dbeta,
                                                                   int accumulate) {
    __shared__ float part[16][17];
    const int col = threadIdx.x & 15, phase = threadIdx.x >> 4, i = blockIdx.x * 16 + col;
    const size_t row_stride = size_t(2) * D;
    float s[8];
#pragma unroll
    for (int u = 0; u < 8; ++u)
        s[u] = 0.f;
    int b = phase;
    for (; b + 16 * 7 < blocks; b += 16 * 8) {
#pragma unroll
        for (int u = 0; u < 8; ++u)
            s[u] += partial[size_t(b + 16 * u) * row_stride + i];
    }
    for (; b < blocks; b += 16)
        s[0] += partial[size_t(b) * row_stride + i];
    part[phase][col] = ((s[0] + s[1]) + (s[2] + s[3])) + ((s[4] + s[5]) + (s[6] + s[7]));
    __syncthreads();
    if (phase == 0) {
        float sum = 0.f;
#pragma unroll
        for (int p = 0; p < 16; ++p)
            sum += part[p][col];
        float *out = i < D ? dgamma + i : dbeta + (i - D);
        *out = accumulate ? *out + sum : sum;
    }
}

// The same fold for many LayerNorms in one launch: job j sums the partial rows at partial + j * job_stride into
// its own dgamma / dbeta (device array of pointer pairs).  blockIdx.y selects the job.  Same order of additions
// as layernorm_bwd_reduce_kernel, so a gradient folded here equals one folded there bit for bit.
struct LayerNormFoldTarget {
    float *dgamma, *dbeta;
};
__global__ __launch_bounds__(256) void layernorm_bwd_fold_batch_kernel(const float *__restrict__ partial,
                                                                       size_t job_stride, int blocks, int D,
                                                                       const LayerNormFoldTarget *__restrict__ targets,
                                                                       int accumulate) {
    __shared__ float part[16][17];
    const float *mine = partial + size_t(blockIdx.y) * job_stride;
    const int col = threadIdx.x & 15, phase = threadIdx.x >> 4, i = blockIdx.x * 16 + col;
    const size_t row_stride = size_t(2) * D;
    float s[8];
#pragma unroll
    for (int u = 0; u < 8; ++u)
        s[u] = 0.f;
    int b = phase;
    for (; b + 16 * 7 < blocks; b += 16 * 8) {
#pragma unroll
        for (int u = 0; u < 8; ++u)
            s[u] += mine[size_t(b + 16 * u) * row_stride + i];
    }
    for (; b < blocks; b += 16)
        s[0] += mine[size_t(b) * row_stride + i];
    part[phase][col] = ((s[0] + s[1]) + (s[2] + s[3])) + ((s[4] + s[5]) + (s[6] + s[7]));
    __syncthreads();
    if (phase == 0) {
        float sum = 0.f;
#pragma unroll
        for (int p = 0; p < 16; ++p)
            sum += part[p][col];
        const LayerNormFoldTarget t = targets[blockIdx.y];
        float *out = i < D ? t.dgamma + i : t.dbeta + (i - D);
        *out = accumulate ? *out + sum : sum;
    }
}

// ---- cross-entropy over 256 byte classes ------------------------------------------------------
// One wave per token: loss, optional fp32 copy of the logits, dlogits = RN((softmax - onehot) * k)
// written in place over the bf16 logits (cuda/model.cuh:33-58).
__global__ __launch_bounds__(256) void cross_entropy_kernel(bf16_t *__restrict__ logits,
                                                            const uint8_t *__restrict__ y,
                                                            float *__restrict__ loss,
                                                            float *__restrict__ logits_f32, int rows,
                                                            float inv_count, int write_grad) {
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    for (int row = blockIdx.x * 4 + wave; row < rows; row += gridDim.x * 4) {
        bf16_t *p = logits + size_t(row) * 256 + lane * 4;
        const u32x2 raw = *reinterpret_cast<const u32x2 *>(p);
        float v[4] = {bf16_lo(raw.x), bf16_hi(raw.x), bf16_lo(raw.y), bf16_hi(raw.y)};
        const float high = wave_max(fmaxf(fmaxf(v[0], v[1]), fmaxf(v[2], v[3])));
        float e[4], sum = 0.f;
#pragma unroll
        for (int k = 0; k < 4; ++k) {
            e[k] = __expf(v[k] - high);
            sum += e[k];
        }
        sum = wave_sum(sum);
        const int target = y[row];
        const int t3 = target & 3;
        const float own = t3 == 0 ? v[0] : t3 == 1 ? v[1] : t3 == 2 ? v[2] : v[3];
        const float mine = (target >> 2) == lane ? own : 0.f;
        const float picked = wave_sum(mine);
        if (lane == 0)
            loss[row] = high + __logf(sum) - picked;
        if (logits_f32)
            *reinterpret_cast<f32x4 *>(logits_f32 + size_t(row) * 256 + lane * 4) = f32x4{v[0], v[1], v[2], v[3]};
        if (write_grad) {
            const float inv = 1.0f / sum;
            float gr[4];
#pragma unroll
            for (int k = 0; k < 4; ++k)
                gr[k] = (e[k] * inv - (lane * 4 + k == target ? 1.f : 0.f)) * inv_count;
            u32x2 out;
            out.x = pack_bf16(gr[0], gr[1]);
            out.y = pack_bf16(gr[2], gr[3]);
            *reinterpret_cast<u32x2 *>(p) = out;
        }
    }
}

// ---- optimizer --------------------------------------------------------------------------------
__global__ __launch_bounds__(256) void sumsq_kernel(const float *__restrict__ g, size_t n,
                                                    float *__restrict__ partial) {
    __shared__ float waves[4];
    float sum = 0.f;
    const size_t quads = n >> 2;
    for (size_t i = blockIdx.x * size_t(256) + threadIdx.x; i < quads; i += size_t(gridDim.x) * 256) {
        const f32x4 v = *reinterpret_cast<const f32x4 *>(g + i * 4);
        sum += v[0] * v[0] + v[1] * v[1] + v[2] * v[2] + v[3] * v[3];
    }
    if (blockIdx.x == 0 && threadIdx.x < int(n & 3)) {
        const float v = g[(quads << 2) + threadIdx.x];
        sum += v * v;
    }
    sum = wave_sum(sum);
    if ((threadIdx.x & 63) == 0)
        waves[threadIdx.x >> 6] = sum;
    __syncthreads();
    if (threadIdx.x == 0)
        partial[blockIdx.x] = (waves[0] + waves[1]) + (waves[2] + waves[3]);
}

// The same for a list of ranges of g, one block per range (the parameter tensors whose gradients no matrix kernel
// writes: the caller cuts long tensors into ranges of a few thousand elements).  Starts and lengths multiples of 4.
struct SumsqSegment {
    int64_t start, length;
};
__global__ __launch_bounds__(256) void sumsq_segments_kernel(const float *__restrict__ g,
                                                             const SumsqSegment *__restrict__ segments,
                                                             float *__restrict__ partial) {
    __shared__ float waves[4];
    const SumsqSegment segment = segments[blockIdx.x];
    const f32x4 *p = reinterpret_cast<const f32x4 *>(g + segment.start);
    const int quads = int(segment.length >> 2);
    float sum = 0.f;
#pragma unroll 8
    for (int i = threadIdx.x; i < quads; i += 256) {
        const f32x4 v = p[i];
        sum += v[0] * v[0] + v[1] * v[1] + v[2] * v[2] + v[3] * v[3];
    }
    sum = wave_sum(sum);
    if ((threadIdx.x & 63) == 0)
        waves[threadIdx.x >> 6] = sum;
    __syncthreads();
    if (threadIdx.x == 0)
        partial[blockIdx.x] = (waves[0] + waves[1]) + (waves[2] + waves[3]);
}

struct AdamArgs {
    float lr, beta1, beta2, eps, weight_decay, bc1, sqrt_bc2, clip;
};
// cuda/optim.cuh:67-106 on the (hi bf16, lo u16) weight halves (cuda/ops.cuh:6-14).
// bounds: sorted starts of `segments` parameter ranges, bit 0 of flags[s] = weight decay, bit 1 = skip.
__global__ __launch_bounds__(256) void adamw_kernel(bf16_t *__restrict__ hi, uint16_t *__restrict__ lo,
                                                    float *__restrict__ m, float *__restrict__ v,
                                                    const float *__restrict__ g, size_t n,
                                                    const float *__restrict__ norm_partials,
                                                    int norm_count, const int64_t *__restrict__ bounds,
                                                    const uint8_t *__restrict__ flags, int segments,
                                                    AdamArgs a) {
    __shared__ float waves[4];
    __shared__ float clip_scale;
    float scale = 1.f;
    if (a.clip > 0.f) {
        // every block folds the same partials in the same order (cuda/optim.cuh:67-80)
        float sum = 0.f;
        for (int i = threadIdx.x; i < norm_count; i += 256)
            sum += norm_partials[i];
        sum = wave_sum(sum);
        if ((threadIdx.x & 63) == 0)
            waves[threadIdx.x >> 6] = sum;
        __syncthreads();
        if (threadIdx.x == 0)
            clip_scale = fminf(1.f, a.clip / (sqrtf((waves[0] + waves[1]) + (waves[2] + waves[3])) + 1e-6f));
        __syncthreads();
        scale = clip_scale;
    }
    // Every stream here is touched once per step: non-temporal loads and stores keep 3 GB of optimizer state from
    // evicting what the next step's first kernels read (measured -0.6 % on the step).
    const size_t quads = n >> 2;
    for (size_t q = blockIdx.x * size_t(256) + threadIdx.x; q < quads; q += size_t(gridDim.x) * 256) {
        const size_t i = q * 4;
        int lo_s = 0, hi_s = segments - 1; // last segment whose start <= i
        while (lo_s < hi_s) {
            const int mid = (lo_s + hi_s + 1) >> 1;
            if (size_t(bounds[mid]) <= i)
                lo_s = mid;
            else
                hi_s = mid - 1;
        }
        if (flags[lo_s] & 2) // owned by another optimizer (Muon, cuda/optim.cuh:94-96)
            continue;
        const float decay = (flags[lo_s] & 1) ? a.weight_decay : 0.f;
        const f32x4 gv = __builtin_nontemporal_load(reinterpret_cast<const f32x4 *>(g + i));
        f32x4 mv = __builtin_nontemporal_load(reinterpret_cast<const f32x4 *>(m + i)), vv = __builtin_nontemporal_load(reinterpret_cast<const f32x4 *>(v + i));
        const u32x2 hv = __builtin_nontemporal_load(reinterpret_cast<const u32x2 *>(hi + i)), lv = __builtin_nontemporal_load(reinterpret_cast<const u32x2 *>(lo + i));
        uint32_t bits[4] = {(hv.x << 16) | (lv.x & 0xffffu), (hv.x & 0xffff0000u) | (lv.x >> 16),
                            (hv.y << 16) | (lv.y & 0xffffu), (hv.y & 0xffff0000u) | (lv.y >> 16)};
#pragma unroll
        for (int k = 0; k < 4; ++k) {
            const float gk = gv[k] * scale;
            const float mk = mv[k] + (1.f - a.beta1) * (gk - mv[k]);
            const float vk = a.beta2 * vv[k] + (1.f - a.beta2) * gk * gk;
            mv[k] = mk;
            vv[k] = vk;
            const float w = __uint_as_float(bits[k]) * (1.f - a.lr * decay);
            bits[k] = __float_as_uint(w - (a.lr / a.bc1) * mk / (sqrtf(vk) / a.sqrt_bc2 + a.eps));
        }
        __builtin_nontemporal_store(mv, reinterpret_cast<f32x4 *>(m + i));
        __builtin_nontemporal_store(vv, reinterpret_cast<f32x4 *>(v + i));
        u32x2 ho, lw;
        ho.x = (bits[0] >> 16) | (bits[1] & 0xffff0000u);
        ho.y = (bits[2] >> 16) | (bits[3] & 0xffff0000u);
        lw.x = (bits[0] & 0xffffu) | (bits[1] << 16);
        lw.y = (bits[2] & 0xffffu) | (bits[3] << 16);
        __builtin_nontemporal_store(ho, reinterpret_cast<u32x2 *>(hi + i));
        __builtin_nontemporal_store(lw, reinterpret_cast<u32x2 *>(lo + i));
    }
}

// ---- data and loss bookkeeping ---------------------------------------------------------------
// cuda/dataset.cuh:13-27; the window start is kept inside the data for contexts longer than 8
__global__ __launch_bounds__(256) void sample_batch_kernel(const uint8_t *__restrict__ data, int64_t size,
                                                           uint64_t seed, uint64_t step, int batch,
                                                           int context, uint8_t *__restrict__ x,
                                                           uint8_t *__restrict__ y) {
    const int b = blockIdx.x;
    const int64_t low = context > 8 ? context : 8;
    const int64_t e = low + int64_t(hash_u64(seed + step * uint64_t(batch) + uint64_t(b)) % uint64_t(size - low));
    for (int p = threadIdx.x; p < context; p += 256) {
        x[size_t(b) * context + p] = data[e - context + p];
        y[size_t(b) * context + p] = data[e - context + p + 1];
    }
}
// cuda/trainer.cuh:79-100: mean over the batch per position, accumulated in double
__global__ __launch_bounds__(256) void position_means_kernel(const float *__restrict__ token_loss,
                                                             int batch, int context,
                                                             float *__restrict__ out) {
    // one wave per position: a lane sums every 64th sequence, then the lanes are folded in a fixed tree
    const int p = blockIdx.x * 4 + (threadIdx.x >> 6), lane = threadIdx.x & 63;
    if (p >= context)
        return;
    double sum = 0;
    for (int b = lane; b < batch; b += 64)
        sum += token_loss[size_t(b) * context + p];
#pragma unroll
    for (int k = 32; k; k >>= 1)
        sum += __shfl_xor(sum, k, 64);
    if (lane == 0)
        out[p] = float(sum / batch);
}

// ---- batched bf16 transposes ------------------------------------------------------------------
// out[c][r] = in[r][c] for a list of row-major matrices that live at the same offset in `in` and
// `out`.  64x64 tiles through LDS; a block finds its matrix from the running tile counts.
struct TransposeJob {
    int64_t offset; // element offset of the matrix in both buffers
    int rows, cols; // of the source
    int first_tile; // running count of 64x64 tiles before this matrix
    int pad;
};
__global__ __launch_bounds__(256) void transpose_batch_kernel(const bf16_t *__restrict__ in,
                                                              bf16_t *__restrict__ out,
                                                              const TransposeJob *__restrict__ jobs, int count) {
    __shared__ bf16_t tile[64][66];
    int lo = 0, hi = count - 1; // last job whose first_tile <= blockIdx.x
    while (lo < hi) {
        const int mid = (lo + hi + 1) >> 1;
        if (jobs[mid].first_tile <= int(blockIdx.x))
            lo = mid;
        else
            hi = mid - 1;
    }
    const TransposeJob job = jobs[lo];
    const int t = blockIdx.x - job.first_tile, tiles_c = job.cols >> 6;
    const int r0 = (t / tiles_c) << 6, c0 = (t % tiles_c) << 6;
    const bf16_t *src = in + job.offset;
    bf16_t *dst = out + job.offset;
    const int tx = threadIdx.x & 31, ty = threadIdx.x >> 5; // 32 column pairs x 8 rows
#pragma unroll
    for (int i = 0; i < 8; ++i) {
        const int r = ty + i * 8;
        const uint32_t pair = *reinterpret_cast<const uint32_t *>(src + size_t(r0 + r) * job.cols + c0 + tx * 2);
        tile[r][tx * 2] = bf16_t(pair);
        tile[r][tx * 2 + 1] = bf16_t(pair >> 16);
    }
    __syncthreads();
#pragma unroll
    for (int i = 0; i < 8; ++i) {
        const int c = ty + i * 8; // source column = destination row
        const uint32_t pair = uint32_t(tile[tx * 2][c]) | (uint32_t(tile[tx * 2 + 1][c]) << 16);
        __builtin_nontemporal_store(pair, reinterpret_cast<uint32_t *>(dst + size_t(c0 + c) * job.rows + r0 + tx * 2));
    }
}

int grid_for(size_t work_items, int per_block, int cap = 4096) {
    const size_t blocks = (work_items + per_block - 1) / per_block;
    return int(blocks < size_t(cap) ? (blocks ? blocks : 1) : cap);
}
void aligned(const void *p, const char *name) {
    if (!p || (reinterpret_cast<uintptr_t>(p) & 15))
        throw std::invalid_argument(std::string(name) + " must be non-null and 16-byte aligned");
}

} // namespace

extern "C" int tgk_embed_fwd(hipStream_t stream, int rows, int T, int D, const uint8_t *x,
                             const uint16_t *table, const uint16_t *positions, uint16_t *out) {
    return guarded([&] {
        require(rows > 0 && T > 0 && D > 0 && D % 8 == 0, "embed_fwd: D must be a positive multiple of 8");
        require(x != nullptr, "embed_fwd: missing tokens");
        aligned(table, "embed_fwd: table");
        aligned(positions, "embed_fwd: positions");
        aligned(out, "embed_fwd: out");
        hipLaunchKernelGGL(embed_fwd_kernel, dim3(grid_for(size_t(rows) * D / 8, 256)), dim3(256), 0, stream, x,
                           table, positions, out, rows, T, D);
        check_hip(hipGetLastError(), "embed_fwd launch: ");
    });
}

// The token-table gradient is a product: dTable[v][c] = sum_t onehot[t][v] dh[t][c], i.e. the weight-
// gradient GEMM with the one-hot matrix as its "dY" (exact in bf16).  Shapes that GEMM does not take
// go through the LDS-table kernels above.
static bool embed_bwd_as_gemm(int rows, int D) {
    return rows % 32 == 0 && D % 128 == 0;
}
static size_t onehot_bytes(int rows) {
    return size_t(rows) * 256 * sizeof(bf16_t);
}
extern "C" size_t tgk_embed_bwd_workspace(int rows, int D) {
    if (rows <= 0 || D <= 0)
        return 0;
    if (embed_bwd_as_gemm(rows, D))
        return onehot_bytes(rows) + tgk_gemm_wgrad_workspace(rows, 256, D);
    return size_t((rows + EMBED_SEGMENT - 1) / EMBED_SEGMENT) * 256 * D * sizeof(float);
}
extern "C" int tgk_embed_bwd_onehot(hipStream_t stream, int B, int T, int D, const uint8_t *x, const uint16_t *dh,
                                    uint16_t *onehot, float *dpositions, int accumulate) {
    return guarded([&] {
        require(B > 0 && T > 0 && D > 0 && D % 64 == 0, "embed_bwd_onehot: D must be a positive multiple of 64");
        require(x && dh && dpositions, "embed_bwd_onehot: missing operand");
        aligned(onehot, "embed_bwd_onehot: onehot");
        const int rows = B * T;
        hipLaunchKernelGGL(onehot_kernel, dim3(grid_for(size_t(rows) * 32, 256)), dim3(256), 0, stream, x, onehot, rows);
        hipLaunchKernelGGL(embed_bwd_positions_kernel, dim3(grid_for(size_t(T) * D, 256)), dim3(256), 0, stream,
                           dh, dpositions, B, T, D, accumulate);
        check_hip(hipGetLastError(), "embed_bwd_onehot launch: ");
    });
}
extern "C" int tgk_embed_bwd(hipStream_t stream, int B, int T, int D, int vocab, const uint8_t *x,
                             const uint16_t *dh, float *dtable, float *dpositions, int accumulate,
                             void *workspace, size_t workspace_bytes) {
    return guarded([&] {
        require(B > 0 && T > 0 && D > 0 && D % 64 == 0, "embed_bwd: D must be a positive multiple of 64");
        require(vocab == 256, "embed_bwd: vocabulary must be 256 (byte tokens)");
        require(x && dh && dtable && dpositions, "embed_bwd: missing operand");
        const int rows = B * T, segments = (rows + EMBED_SEGMENT - 1) / EMBED_SEGMENT;
        require(workspace && workspace_bytes >= tgk_embed_bwd_workspace(rows, D) &&
                    !(reinterpret_cast<uintptr_t>(workspace) & 15),
                "embed_bwd: workspace too small (see tgk_embed_bwd_workspace)");
        if (embed_bwd_as_gemm(rows, D)) {
            bf16_t *onehot = static_cast<bf16_t *>(workspace);
            hipLaunchKernelGGL(onehot_kernel, dim3(grid_for(size_t(rows) * 32, 256)), dim3(256), 0, stream, x,
                               onehot, rows);
            check_hip(hipGetLastError(), "embed_bwd launch: ");
            if (tgk_gemm_wgrad(stream, rows, 256, D, onehot, 256, dh, D, dtable, D, accumulate,
                               static_cast<char *>(workspace) + onehot_bytes(rows),
                               workspace_bytes - onehot_bytes(rows)) != 0)
                throw std::runtime_error("embed_bwd: " + tg_last_error);
        } else {
            float *partial = static_cast<float *>(workspace);
            hipLaunchKernelGGL(embed_bwd_partial_kernel, dim3(D / 64, segments), dim3(64), 0, stream, x, dh,
                               partial, rows, D);
            const size_t count = size_t(256) * D;
            hipLaunchKernelGGL(embed_bwd_fold_kernel, dim3(unsigned((count + 255) / 256)), dim3(256), 0, stream,
                               partial, segments, dtable, count, accumulate);
        }
        hipLaunchKernelGGL(embed_bwd_positions_kernel, dim3(grid_for(size_t(T) * D, 256)), dim3(256), 0, stream,
                           dh, dpositions, B, T, D, accumulate);
        check_hip(hipGetLastError(), "embed_bwd launch: ");
    });
}

// lanes per row and 16-byte chunks per lane: half a wave per row where that leaves fewer idle lane slots
struct LayerNormShape {
    int group, chunks;
};
static LayerNormShape layernorm_shape(int D) {
    const int chunks = D / 8, per64 = (chunks + 63) / 64, per32 = (chunks + 31) / 32;
    if (per32 < 2 * per64 && per32 <= 3)
        return {32, per32}; // 1 or 3 chunks per lane (2 never wins over a whole wave)
    return {64, per64 <= 2 ? per64 : 4};
}
extern "C" int tgk_layernorm_fwd(hipStream_t stream, int rows, int D, const uint16_t *x,
                                 const uint16_t *gamma_hi, const uint16_t *gamma_lo,
                                 const uint16_t *beta_hi, const uint16_t *beta_lo, uint16_t *y, float eps) {
    return guarded([&] {
        require(rows > 0 && D > 0 && D % 8 == 0 && D <= MAX_LN_CHUNKS * 512,
                "layernorm: D must be a multiple of 8, at most 2048");
        aligned(x, "layernorm: x");
        aligned(y, "layernorm: y");
        aligned(gamma_hi, "layernorm: gamma_hi");
        aligned(gamma_lo, "layernorm: gamma_lo");
        aligned(beta_hi, "layernorm: beta_hi");
        aligned(beta_lo, "layernorm: beta_lo");
        const LayerNormShape shape = layernorm_shape(D);
        // two blocks per CU (256 CUs), each walking its rows with gamma and beta in registers: measured best
        // of 256..2048 blocks at 16384 rows
        const dim3 grid(grid_for(rows, 256 / shape.group, 512));
#define TG_LN_FWD(NC, GROUP)                                                                                      \
    hipLaunchKernelGGL((layernorm_fwd_kernel<NC, GROUP>), grid, dim3(256), 0, stream, x, gamma_hi, gamma_lo,      \
                       beta_hi, beta_lo, y, rows, D, eps)
        if (shape.group == 32 && shape.chunks == 1)
            TG_LN_FWD(1, 32);
        else if (shape.group == 32)
            TG_LN_FWD(3, 32);
        else if (shape.chunks == 1)
            TG_LN_FWD(1, 64);
        else if (shape.chunks == 2)
            TG_LN_FWD(2, 64);
        else
            TG_LN_FWD(4, 64);
#undef TG_LN_FWD
        check_hip(hipGetLastError(), "layernorm_fwd launch: ");
    });
}

static int layernorm_bwd_blocks(int rows) {
    return grid_for(rows, 8, 768); // three blocks per CU: measured best of 512 / 768 / 1024 at 16384 rows
}
extern "C" size_t tgk_layernorm_bwd_workspace(int rows, int D) {
    return rows > 0 && D > 0 ? size_t(layernorm_bwd_blocks(rows)) * 2 * D * sizeof(float) : 0;
}
namespace {
// the row kernel: dx, and one partial row pair (dgamma | dbeta) per block into `partial`
void launch_layernorm_bwd_rows(hipStream_t stream, int rows, int D, const uint16_t *x, const uint16_t *dy,
                               const uint16_t *gamma_hi, const uint16_t *gamma_lo, const uint16_t *residual, uint16_t *dx,
                               float eps, float *partial) {
    require(rows > 0 && D > 0 && D % 64 == 0 && D <= MAX_LN_CHUNKS * 512,
            "layernorm_bwd: D must be a multiple of 64, at most 2048");
    aligned(x, "layernorm: x");
    aligned(dy, "layernorm: dy");
    aligned(dx, "layernorm: dx");
    aligned(gamma_hi, "layernorm: gamma_hi");
    aligned(gamma_lo, "layernorm: gamma_lo");
    if (residual)
        aligned(residual, "layernorm: residual");
    const int blocks = layernorm_bwd_blocks(rows);
    // one row per wave here: two rows per wave cost registers (148 for D = 768) and LDS that lower the
    // occupancy, and measured slower
    const int per_lane = (D / 8 + 63) / 64;
    const size_t lds = size_t(4) * 2 * D * sizeof(float);
#define TG_LN_BWD(NC, GROUP)                                                                                      \
    hipLaunchKernelGGL((layernorm_bwd_kernel<NC, GROUP>), dim3(blocks), dim3(256), lds, stream, x, dy, gamma_hi,  \
                       gamma_lo, residual, dx, partial, rows, D, eps)
    if (per_lane == 1)
        TG_LN_BWD(1, 64);
    else if (per_lane == 2)
        TG_LN_BWD(2, 64);
    else
        TG_LN_BWD(4, 64);
#undef TG_LN_BWD
    check_hip(hipGetLastError(), "layernorm_bwd launch: ");
}
} // namespace

extern "C" int tgk_layernorm_bwd_add(hipStream_t stream, int rows, int D, const uint16_t *x,
                                     const uint16_t *dy, const uint16_t *gamma_hi, const uint16_t *gamma_lo,
                                     const uint16_t *residual, uint16_t *dx, float *dgamma, float *dbeta,
                                     float eps, int accumulate, void *workspace, size_t workspace_bytes) {
    return guarded([&] {
        require(dgamma && dbeta, "layernorm_bwd: missing operand");
        require(workspace && workspace_bytes >= tgk_layernorm_bwd_workspace(rows, D),
                "layernorm_bwd: workspace too small (see tgk_layernorm_bwd_workspace)");
        float *partial = static_cast<float *>(workspace);
        launch_layernorm_bwd_rows(stream, rows, D, x, dy, gamma_hi, gamma_lo, residual, dx, eps, partial);
        hipLaunchKernelGGL(layernorm_bwd_reduce_kernel, dim3(2 * D / 16), dim3(256), 0, stream, partial,
                           layernorm_bwd_blocks(rows), D, dgamma, dbeta, accumulate);
        check_hip(hipGetLastError(), "layernorm_bwd launch: ");
    });
}
extern "C" int tgk_layernorm_bwd_rows(hipStream_t stream, int rows, int D, const uint16_t *x, const uint16_t *dy,
                                      const uint16_t *gamma_hi, const uint16_t *gamma_lo, const uint16_t *residual,
                                      uint16_t *dx, float eps, void *partials, size_t partials_bytes) {
    return guarded([&] {
        require(partials && partials_bytes >= tgk_layernorm_bwd_workspace(rows, D) &&
                    !(reinterpret_cast<uintptr_t>(partials) & 15),
                "layernorm_bwd_rows: partials too small (see tgk_layernorm_bwd_workspace)");
        launch_layernorm_bwd_rows(stream, rows, D, x, dy, gamma_hi, gamma_lo, residual, dx, eps,
                                  static_cast<float *>(partials));
    });
}
extern "C" int tgk_layernorm_bwd_fold(hipStream_t stream, int rows, int D, int count, const void *partials,
                                      size_t job_stride_bytes, const void *targets, int accumulate) {
    return guarded([&] {
        require(rows > 0 && D > 0 && D % 64 == 0 && count > 0 && count <= 65535, "layernorm_bwd_fold: bad shape");
        require(partials && targets && job_stride_bytes % 16 == 0 &&
                    job_stride_bytes >= tgk_layernorm_bwd_workspace(rows, D),
                "layernorm_bwd_fold: missing operand or job stride below tgk_layernorm_bwd_workspace");
        hipLaunchKernelGGL(layernorm_bwd_fold_batch_kernel, dim3(2 * D / 16, count), dim3(256), 0, stream,
                           static_cast<const float *>(partials), job_stride_bytes / sizeof(float),
                           layernorm_bwd_blocks(rows), D, static_cast<const LayerNormFoldTarget *>(targets), accumulate);
        check_hip(hipGetLastError(), "layernorm_bwd_fold launch: ");
    });
}
extern "C" int tgk_layernorm_bwd(hipStream_t stream, int rows, int D, const uint16_t *x,
                                 const uint16_t *dy, const uint16_t *gamma_hi, const uint16_t *gamma_lo,
                                 uint16_t *dx, float *dgamma, float *dbeta, float eps, int residual,
                                 int accumulate, void *workspace, size_t workspace_bytes) {
    return tgk_layernorm_bwd_add(stream, rows, D, x, dy, gamma_hi, gamma_lo, residual ? dx : nullptr, dx, dgamma,
                                 dbeta, eps, accumulate, workspace, workspace_bytes);
}

extern "C" int tgk_cross_entropy(hipStream_t stream, int rows, int vocab, uint16_t *logits,
                                 const uint8_t *y, float *loss, float *logits_f32, float inv_count,
                                 int write_grad) {
    return guarded([&] {
        require(rows > 0, "cross_entropy: empty batch");
        require(vocab == 256, "cross_entropy: vocabulary must be 256 (byte tokens)");
        aligned(logits, "cross_entropy: logits");
        require(y && loss, "cross_entropy: missing operand");
        require(!logits_f32 || !(reinterpret_cast<uintptr_t>(logits_f32) & 15),
                "cross_entropy: fp32 logits must be 16-byte aligned");
        hipLaunchKernelGGL(cross_entropy_kernel, dim3(grid_for(rows, 4, 8192)), dim3(256), 0, stream, logits, y,
                           loss, logits_f32, rows, inv_count, write_grad);
        check_hip(hipGetLastError(), "cross_entropy launch: ");
    });
}

extern "C" int tgk_sumsq_partials(hipStream_t stream, const float *g, size_t n, float *partials,
                                  int count) {
    return guarded([&] {
        aligned(g, "sumsq: g");
        require(partials && count > 0 && count <= 4096, "sumsq: 1..4096 partials");
        hipLaunchKernelGGL(sumsq_kernel, dim3(count), dim3(256), 0, stream, g, n, partials);
        check_hip(hipGetLastError(), "sumsq launch: ");
    });
}

extern "C" int tgk_sumsq_segments(hipStream_t stream, const float *g, const void *segments, int count, float *partials) {
    return guarded([&] {
        aligned(g, "sumsq_segments: g");
        require(segments && !(reinterpret_cast<uintptr_t>(segments) & 7) && partials && count > 0 && count <= 4096,
                "sumsq_segments: 1..4096 ranges in a device array, and their partials");
        hipLaunchKernelGGL(sumsq_segments_kernel, dim3(count), dim3(256), 0, stream, g,
                           static_cast<const SumsqSegment *>(segments), partials);
        check_hip(hipGetLastError(), "sumsq_segments launch: ");
    });
}
extern "C" int tgk_adamw(hipStream_t stream, size_t n, uint16_t *weight_hi, uint16_t *weight_lo, float *m,
                         float *v, const float *g, const float *norm_partials, int norm_count,
                         const int64_t *segment_starts, const uint8_t *segment_flags, int segments,
                         float lr, float beta1, float beta2, float eps, float weight_decay, float clip,
                         uint64_t step) {
    return guarded([&] {
        require(n > 0 && n % 4 == 0, "adamw: parameter count must be a positive multiple of 4");
        aligned(weight_hi, "adamw: weight_hi");
        aligned(weight_lo, "adamw: weight_lo");
        aligned(m, "adamw: m");
        aligned(v, "adamw: v");
        aligned(g, "adamw: g");
        require(segment_starts && segment_flags && segments > 0, "adamw: missing segment table");
        require(!(clip > 0.f) || (norm_partials && norm_count > 0), "adamw: clipping needs the norm partials");
        // bias correction with the current beta1 (cuda/optim.cuh:90-91), evaluated on the host in fp32
        AdamArgs a{lr, beta1, beta2, eps, weight_decay, 1.f - powf(beta1, float(step + 1)),
                   sqrtf(1.f - powf(beta2, float(step + 1))), clip};
        hipLaunchKernelGGL(adamw_kernel, dim3(grid_for(n / 4, 256, 8192)), dim3(256), 0, stream, weight_hi,
                           weight_lo, m, v, g, n, norm_partials, norm_count, segment_starts, segment_flags,
                           segments, a);
        check_hip(hipGetLastError(), "adamw launch: ");
    });
}

extern "C" int tgk_sample_batch(hipStream_t stream, const uint8_t *data, int64_t size, uint64_t seed,
                                uint64_t step, int batch, int context, uint8_t *x, uint8_t *y) {
    return guarded([&] {
        require(data && x && y, "sample_batch: missing operand");
        require(batch > 0 && context > 0, "sample_batch: empty batch");
        require(size > (context > 8 ? context : 8), "sample_batch: dataset shorter than one window");
        hipLaunchKernelGGL(sample_batch_kernel, dim3(batch), dim3(256), 0, stream, data, size, seed, step, batch,
                           context, x, y);
        check_hip(hipGetLastError(), "sample_batch launch: ");
    });
}

extern "C" int tgk_position_means(hipStream_t stream, const float *token_loss, int batch, int context,
                                  float *out) {
    return guarded([&] {
        require(token_loss && out && batch > 0 && context > 0, "position_means: missing operand");
        hipLaunchKernelGGL(position_means_kernel, dim3((context + 3) / 4), dim3(256), 0, stream, token_loss,
                           batch, context, out);
        check_hip(hipGetLastError(), "position_means launch: ");
    });
}

extern "C" int tgk_transpose_batch(hipStream_t stream, const uint16_t *in, uint16_t *out, const void *jobs,
                                   int count, int total_tiles) {
    return guarded([&] {
        require(in && out && jobs && count > 0 && total_tiles > 0, "transpose_batch: missing operand");
        hipLaunchKernelGGL(transpose_batch_kernel, dim3(total_tiles), dim3(256), 0, stream, in, out,
                           static_cast<const TransposeJob *>(jobs), count);
        check_hip(hipGetLastError(), "transpose_batch launch: ");
    });
}
