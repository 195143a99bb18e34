// Causal softmax attention for gfx950, head_dim 64: flash-style forward (online softmax, fp32
// log-sum-exp saved) and recompute backward.  Takes the slot of attention_forward /
// attention_backward in the reference's layer (cuda/attention.cuh:48-106; called from
// cuda/model.cuh:20 and :86-88); the packed [token][q|k|v] buffer and the [token][head*64+d]
// output keep the reference's layout (cuda/attention.cuh:38-39,68), so no permutes are needed.
//
// All three kernels work on 32x32 MFMA tiles (v_mfma_f32_32x32x16_bf16) and are written in the
// "transposed" form: the score tile is produced as S^T[key][query] so that one lane owns one
// query row - row maxima / sums / rescales are per-lane scalars - and the fp32 accumulator
// registers of S^T can be fed back, converted to bf16, as the B operand of the next product with
// no cross-lane movement.  The operand that must then be read "k-strided" (V for P.V, K for dS.K,
// Q and dO for the dK/dV products) is fetched with the transposing LDS read ds_read_b64_tr_b16.
//
// backward = two launches: dQ (one block per 128 queries, loops over key tiles; it also computes
// delta = rowsum(dO o O) for its queries), then dK/dV (one block per 128 keys, loops over query
// tiles).  No atomics: every output element has one owner and a fixed summation order, so results
// are bit-reproducible.
#include "common.h"
#include <atomic>
#include "../../include/tgk_kernels.h"

namespace {

constexpr int HD = 64;      // head dimension
constexpr float LOG2E = 1.4426950408889634f, LN2 = 0.6931471805599453f;

typedef short s16x4 __attribute__((ext_vector_type(4)));
typedef short s16x8 __attribute__((ext_vector_type(8)));
typedef __attribute__((address_space(3))) s16x4 lds_s16x4;

TG_DEVICE f32x16 zero16() {
    f32x16 z;
#pragma unroll
    for (int r = 0; r < 16; ++r)
        z[r] = 0.f;
    return z;
}
TG_DEVICE f32x16 mfma(bf16x8 rows_to_regs, bf16x8 rows_to_lanes, f32x16 acc) {
    return __builtin_amdgcn_mfma_f32_32x32x16_bf16(rows_to_regs, rows_to_lanes, acc, 0, 0, 0);
}
// row index owned by accumulator register r of a 32x32 tile (lane half g = lane/32)
TG_DEVICE int acc_row(int r, int g) {
    return 8 * (r >> 2) + 4 * g + (r & 3);
}
// registers 8*kk2 .. 8*kk2+7 of an fp32 accumulator as a bf16 operand fragment
TG_DEVICE bf16x8 acc_to_frag(const f32x16 &acc, int kk2) {
    bf16x8 f;
#pragma unroll
    for (int j = 0; j < 8; ++j)
        f[j] = (__bf16)acc[8 * kk2 + j];
    return f;
}
TG_DEVICE float exp2_fast(float x) {
    return __builtin_amdgcn_exp2f(x);
}

// ---- swizzled 64 x 64 LDS tiles filled by wave-wide global -> LDS copies -------------------------
// 128-byte rows, no padding (a copy fills 1 KiB contiguously); the 16-byte chunk c of row r sits at
// chunk c ^ swz(r).  swz is chosen so that both access patterns are bank-conflict free: fragments along
// the rows (16 consecutive rows, one chunk each) and transposing reads along the columns (4 consecutive
// rows, 32 bytes each).
constexpr int TILE_ELEMS = 64 * 64;
TG_DEVICE int swz(int row) {
    return (((row >> 1) & 1) << 2) | ((row >> 2) & 3);
}
// this wave's two copies (regions wave and wave+4, 8 rows each) of a 64-row tile starting at `base`
TG_DEVICE void tile_copy_async_one(uint32_t lds_tile, const bf16_t *base, int ld, int wave, int lane, int j) {
    const int region = wave + 4 * j, row = region * 8 + (lane >> 3), chunk = (lane & 7) ^ swz(row);
    async_copy16(__builtin_amdgcn_readfirstlane(lds_tile + region * 1024), base + size_t(row) * ld + chunk * 8);
}
// byte offset of this lane's 16 bytes within a 64-row tile whose rows are ld elements apart
TG_DEVICE uint32_t tile_copy_offset(int ld, int wave, int lane, int j) {
    const int region = wave + 4 * j, row = region * 8 + (lane >> 3), chunk = (lane & 7) ^ swz(row);
    return uint32_t(row * ld + chunk * 8) * 2;
}
TG_DEVICE void tile_copy_async(uint32_t lds_tile, const bf16_t *base, int ld, int wave, int lane) {
#pragma unroll
    for (int j = 0; j < 2; ++j)
        tile_copy_async_one(lds_tile, base, ld, wave, lane, j);
}
// The swizzle terms of both fragment kinds depend on the lane only (swz(row + 32) = swz(row);
// swz(r + 16) = swz(r)), so a kernel computes these element offsets once and adds compile-time
// constants per k-step / tile inside its loops.
// operand fragment along the rows: row mt*32 + lane%32, k = ks*16 + 8*(lane/32) .. +7
struct RowFragOffsets {
    int at[4];
    TG_DEVICE explicit RowFragOffsets(int lane) {
        const int row = lane & 31;
#pragma unroll
        for (int ks = 0; ks < 4; ++ks)
            at[ks] = row * 64 + (((ks * 2 + (lane >> 5)) ^ swz(row)) << 3);
    }
    TG_DEVICE bf16x8 load(const bf16_t *tile, int mt, int ks) const {
        return *reinterpret_cast<const bf16x8 *>(tile + at[ks] + mt * 32 * 64);
    }
};
// operand fragment along the columns (transposing reads): column dt*32 + lane%32 and the 8 rows
// kk*16 + 4g + {0..3}, kk*16 + 8 + 4g + {0..3} - the rows that accumulator registers 8*(kk%2) .. +7 of a
// 32x32 tile hold (acc_row), so a converted accumulator and this fragment agree on the reduced index
struct ColFragOffsets {
    int lo[2], hi[2];
    TG_DEVICE explicit ColFragOffsets(int lane) {
        const int g = lane >> 5, blk = (lane >> 4) & 1, i = lane & 15;
        const int r = 4 * g + (i >> 2);
#pragma unroll
        for (int dt = 0; dt < 2; ++dt) {
            const int col = dt * 32 + 16 * blk + 4 * (i & 3);
            lo[dt] = r * 64 + (((col >> 3) ^ swz(r)) << 3) + (col & 7);
            hi[dt] = (r + 8) * 64 + (((col >> 3) ^ swz(r + 8)) << 3) + (col & 7);
        }
    }
    TG_DEVICE bf16x8 load(const bf16_t *tile, int kk, int dt) const {
        const s16x4 a = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_s16x4 *)(tile + lo[dt] + kk * 16 * 64));
        const s16x4 b = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_s16x4 *)(tile + hi[dt] + kk * 16 * 64));
        const s16x8 both = __builtin_shufflevector(a, b, 0, 1, 2, 3, 4, 5, 6, 7);
        return __builtin_bit_cast(bf16x8, both);
    }
};

// Block placement.  The work of a causal tile grows with its index and consecutive block ids go to the
// eight XCDs in turn, so a (tile, head, batch) grid whose tile extent is a multiple of 8 hands one XCD
// all the heaviest tiles.  Instead each XCD takes every eighth (batch, head) pair with all of that
// pair's tiles - which also keeps a pair's keys and values in one L2 - heaviest rank first.
struct CausalBlock {
    int rank, h, b;
    bool live;
};
TG_DEVICE CausalBlock causal_block(int H, int pairs) {
    const int xcd = blockIdx.x & 7, slot = blockIdx.x >> 3, per_xcd = (pairs + 7) >> 3;
    const int pair = (slot % per_xcd) * 8 + xcd;
    return {slot / per_xcd, pair % H, pair / H, pair < pairs};
}
unsigned causal_grid(int tiles, int pairs) {
    return unsigned(tiles) * unsigned((pairs + 7) / 8) * 8u;
}

template <int N> struct Const {
    static constexpr int value = N;
};
// Lanes i and i+32 own the two halves of one query's keys.  v_permlane32_swap of a value with itself
// leaves the lower lanes' values in every lane of the first result and the upper lanes' in the second.
TG_DEVICE float halves_max(float x) {
    const auto both = __builtin_amdgcn_permlane32_swap(__float_as_uint(x), __float_as_uint(x), false, false);
    return fmaxf(__uint_as_float(both[0]), __uint_as_float(both[1]));
}
TG_DEVICE float halves_sum(float x) {
    const auto both = __builtin_amdgcn_permlane32_swap(__float_as_uint(x), __float_as_uint(x), false, false);
    return __uint_as_float(both[0]) + __uint_as_float(both[1]);
}
// Writes a 32 x 32 accumulator whose rows (lane % 32) are rows of memory: `row` points at this lane's row, first
// of the 32 columns.  Lane l holds columns 8*q4 + 4*g + {0..3} (registers 4*q4 ..) of its row, lane l + 32 the
// other four of every eight.  The two trade halves, so that one ends up with columns 0..15 and the other with
// 16..31 and each writes 32 contiguous bytes: a quarter of the store instructions and of the cache lines touched
// per instruction that 8-byte pieces take.
TG_DEVICE void store_acc_rows(bf16_t *row, const f32x16 &acc, float scale, int g) {
    uint32_t x[4], y[4];
#pragma unroll
    for (int q4 = 0; q4 < 4; ++q4) {
        x[q4] = pack_bf16(acc[q4 * 4 + 0] * scale, acc[q4 * 4 + 1] * scale);
        y[q4] = pack_bf16(acc[q4 * 4 + 2] * scale, acc[q4 * 4 + 3] * scale);
    }
#pragma unroll
    for (int h = 0; h < 2; ++h) {
        const auto ax = __builtin_amdgcn_permlane32_swap(x[h], x[h + 2], false, false);
        const auto ay = __builtin_amdgcn_permlane32_swap(y[h], y[h + 2], false, false);
        *reinterpret_cast<u32x4 *>(row + 16 * g + 8 * h) = u32x4{ax[0], ay[0], ax[1], ay[1]};
    }
}

// ---------------------------------------------------------------------------------------------
// forward: block = 128 queries (4 waves x 32), key/value tiles of 64 in three LDS stages filled by
// asynchronous copies issued two tiles ahead; heavy (late) query tiles first.  The tile loop is
// unrolled by the stage count so every LDS address is a per-lane constant plus an immediate; three
// resident waves per SIMD overlap one wave's softmax with another's matrix work.
// ---------------------------------------------------------------------------------------------
__global__ __launch_bounds__(256, 3) void attn_fwd_kernel(const bf16_t *__restrict__ Q,
                                                          const bf16_t *__restrict__ K,
                                                          const bf16_t *__restrict__ V, int ld,
                                                          bf16_t *__restrict__ O, int ldo,
                                                          float *__restrict__ LSE, int T, int H,
                                                          int pairs, float c) {
    __shared__ __align__(1024) bf16_t stages[3][2][TILE_ELEMS]; // [stage][K | V]
    const CausalBlock block = causal_block(H, pairs);
    if (!block.live)
        return;
    const int q0 = (T / 128 - 1 - block.rank) * 128, h = block.h, b = block.b;
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6, g = lane >> 5;
    const int wave_q0 = q0 + wave * 32, qrow = wave_q0 + (lane & 31);
    const size_t token0 = size_t(b) * T;
    const int tiles = (q0 + 128) / 64;
    const int my_tiles = wave_q0 / 64 + 1; // tiles with a key visible to this wave (wave uniform)
    const bf16_t *kbase = K + token0 * ld + h * HD, *vbase = V + token0 * ld + h * HD;
    const uint32_t lds0 = lds_address(&stages[0][0][0]);
    // a copy takes a wave-uniform tile address and a per-lane byte offset computed once: no vector arithmetic per tile
    const uint32_t lane_offset[2] = {tile_copy_offset(ld, wave, lane, 0), tile_copy_offset(ld, wave, lane, 1)};
    auto produce = [&](int stage, int j) {
        const uint32_t slot = lds0 + uint32_t(stage) * (2 * TILE_ELEMS * 2);
        const bf16_t *kt = kbase + size_t(j) * 64 * ld, *vt = vbase + size_t(j) * 64 * ld;
#pragma unroll
        for (int n = 0; n < 2; ++n) {
            async_copy16(__builtin_amdgcn_readfirstlane(slot + (wave + 4 * n) * 1024), kt, lane_offset[n]);
            async_copy16(__builtin_amdgcn_readfirstlane(slot + TILE_ELEMS * 2 + (wave + 4 * n) * 1024), vt, lane_offset[n]);
        }
    };
    produce(0, 0);
    if (tiles > 1)
        produce(1, 1);

    bf16x8 qf[4];
    {
        const bf16_t *qp = Q + (token0 + qrow) * ld + h * HD + g * 8;
#pragma unroll
        for (int ks = 0; ks < 4; ++ks)
            qf[ks] = *reinterpret_cast<const bf16x8 *>(qp + ks * 16);
    }
    f32x16 o[2] = {zero16(), zero16()};
    float m = -INFINITY, l = 0.f; // l: this lane's half of the keys only, halves are joined at the end
    const RowFragOffsets krows(lane);
    const ColFragOffsets vcols(lane);

    auto step = [&](auto stage_tag, int j) {
        constexpr int STAGE = decltype(stage_tag)::value;
        // tile j was issued two steps ago; only tile j+1's four copies may still be in flight
        if (j + 1 < tiles)
            wait_vmcnt<4>();
        else
            wait_vmcnt<0>();
        __syncthreads(); // tile j visible to every wave; everyone is done with tile j-1's stage
        // the copies of tile j+2 go out at the end of the step, where the waves have drifted apart: behind
        // the barrier every wave of the CU would queue its copies at the same moment
        if (j >= my_tiles) {
            if (j + 2 < tiles)
                produce((STAGE + 2) % 3, j + 2);
            return;
        }
        const bf16_t *kt = stages[STAGE][0], *vt = stages[STAGE][1];
        const int kv0 = j * 64;
        f32x16 s[2] = {zero16(), zero16()};
#pragma unroll
        for (int ks = 0; ks < 4; ++ks)
#pragma unroll
            for (int mt = 0; mt < 2; ++mt)
                s[mt] = mfma(krows.load(kt, mt, ks), qf[ks], s[mt]);
        if (kv0 + 63 > wave_q0) { // diagonal tile: hide keys after the query
#pragma unroll
            for (int mt = 0; mt < 2; ++mt)
#pragma unroll
                for (int r = 0; r < 16; ++r)
                    if (kv0 + mt * 32 + acc_row(r, g) > qrow)
                        s[mt][r] = -INFINITY;
        }
        float mx = -INFINITY;
#pragma unroll
        for (int mt = 0; mt < 2; ++mt)
#pragma unroll
            for (int r = 0; r < 16; ++r)
                mx = fmaxf(mx, s[mt][r]);
        mx = halves_max(mx);
        const float m_new = fmaxf(m, mx * c);
        const float alpha = exp2_fast(m - m_new);
        float sum = 0.f;
#pragma unroll
        for (int mt = 0; mt < 2; ++mt)
#pragma unroll
            for (int r = 0; r < 16; ++r) {
                const float p = exp2_fast(fmaf(s[mt][r], c, -m_new));
                s[mt][r] = p;
                sum += p;
            }
        l = l * alpha + sum;
        if (__builtin_amdgcn_ballot_w64(m_new != m)) { // rescale only when some row's maximum moved
#pragma unroll
            for (int dt = 0; dt < 2; ++dt)
#pragma unroll
                for (int r = 0; r < 16; ++r)
                    o[dt][r] *= alpha;
        }
        m = m_new;
#pragma unroll
        for (int kk = 0; kk < 4; ++kk) {
            const bf16x8 pf = acc_to_frag(s[kk >> 1], kk & 1);
#pragma unroll
            for (int dt = 0; dt < 2; ++dt)
                o[dt] = mfma(vcols.load(vt, kk, dt), pf, o[dt]);
        }
        if (j + 2 < tiles)
            produce((STAGE + 2) % 3, j + 2);
    };
    for (int j = 0; j < tiles; j += 3) { // tiles is block uniform
        step(Const<0>{}, j);
        if (j + 1 < tiles)
            step(Const<1>{}, j + 1);
        if (j + 2 < tiles)
            step(Const<2>{}, j + 2);
    }
    l = halves_sum(l);
    const float inv = 1.0f / l;
    bf16_t *op = O + (token0 + qrow) * ldo + h * HD;
#pragma unroll
    for (int dt = 0; dt < 2; ++dt)
        store_acc_rows(op + dt * 32, o[dt], inv, g);
    if (g == 0)
        LSE[(size_t(b) * H + h) * T + qrow] = (m + __log2f(l)) * LN2;
}

// ---------------------------------------------------------------------------------------------
// dK, dV: block = 128 keys (4 waves x 32), loops over 64-query tiles from the diagonal on; Q and dO
// tiles (plus the 64 log-sum-exps and deltas of the tile) arrive by asynchronous copies two tiles
// ahead.  Scores are produced as S[query][key] here: one lane owns one KEY, which is the row index
// of both outputs.  The two 32-query halves of a tile are processed one after the other to keep the
// live accumulators, and with them the register count, down.
// ---------------------------------------------------------------------------------------------
__global__ __launch_bounds__(256, 2) void attn_bwd_dkdv_kernel(
    const bf16_t *__restrict__ Q, const bf16_t *__restrict__ K, const bf16_t *__restrict__ V, int ld,
    const bf16_t *__restrict__ dO, int lddo, const float *__restrict__ lse2,
    const float *__restrict__ delta, bf16_t *__restrict__ dK, bf16_t *__restrict__ dV, int lddq, int T,
    int H, int pairs, float scale) {
    __shared__ __align__(1024) bf16_t stages[3][2][TILE_ELEMS]; // [stage][Q | dO]
    __shared__ __align__(256) float rows[3][2][64];             // [stage][lse2 | -delta]
    const CausalBlock block = causal_block(H, pairs);
    if (!block.live)
        return;
    const int k0 = block.rank * 128, h = block.h, b = block.b; // early keys see the most queries
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6, g = lane >> 5;
    const int wave_k0 = k0 + wave * 32, krow = wave_k0 + (lane & 31);
    const size_t token0 = size_t(b) * T;
    const float c = scale * LOG2E;
    const int first = k0 / 64, tiles = T / 64 - first;
    const bf16_t *qbase = Q + (token0 + first * 64) * ld + h * HD;
    const bf16_t *gbase = dO + (token0 + first * 64) * lddo + h * HD;
    const float *row_source = ((wave & 1) ? delta : lse2) + (size_t(b) * H + h) * T + first * 64 + lane;
    const uint32_t lds0 = lds_address(&stages[0][0][0]), rows0 = lds_address(&rows[0][wave & 1][0]);
    const uint32_t q_offset[2] = {tile_copy_offset(ld, wave, lane, 0), tile_copy_offset(ld, wave, lane, 1)};
    const uint32_t g_offset[2] = {tile_copy_offset(lddo, wave, lane, 0), tile_copy_offset(lddo, wave, lane, 1)};
    auto produce_one = [&](int stage, int j, int n) { // n-th of a wave's five copies for tile j
        const uint32_t slot = lds0 + uint32_t(stage) * (2 * TILE_ELEMS * 2);
        if (n < 2)
            async_copy16(__builtin_amdgcn_readfirstlane(slot + (wave + 4 * n) * 1024), qbase + size_t(j) * 64 * ld,
                         q_offset[n]);
        else if (n < 4)
            async_copy16(__builtin_amdgcn_readfirstlane(slot + TILE_ELEMS * 2 + (wave + 4 * (n - 2)) * 1024),
                         gbase + size_t(j) * 64 * lddo, g_offset[n - 2]);
        else
            async_copy4(__builtin_amdgcn_readfirstlane(rows0 + uint32_t(stage) * (2 * 64 * 4)), row_source + j * 64);
    };
    auto produce = [&](int stage, int j) {
#pragma unroll
        for (int n = 0; n < 5; ++n)
            produce_one(stage, j, n);
    };
    produce(0, 0);
    produce(1, tiles > 1 ? 1 : 0);

    bf16x8 kf[4], vf[4];
    {
        const bf16_t *kp = K + (token0 + krow) * ld + h * HD + g * 8;
        const bf16_t *vp = V + (token0 + krow) * ld + h * HD + g * 8;
#pragma unroll
        for (int ks = 0; ks < 4; ++ks) {
            kf[ks] = *reinterpret_cast<const bf16x8 *>(kp + ks * 16);
            vf[ks] = *reinterpret_cast<const bf16x8 *>(vp + ks * 16);
        }
    }
    f32x16 dk[2] = {zero16(), zero16()}, dv[2] = {zero16(), zero16()};
    const RowFragOffsets qrows(lane);
    const ColFragOffsets qcols(lane);

    auto step = [&](auto stage_tag, int j) {
        constexpr int STAGE = decltype(stage_tag)::value;
        wait_vmcnt<5>(); // only the five copies issued during tile j-1 may still be in flight
        __syncthreads(); // tile j visible to every wave; everyone is done with tile j-1's stage
        // The copies of tile j+2 go out at the end of the step, where the waves have drifted apart: behind the
        // barrier all eight waves of the CU queue theirs at once and wait for one another (measured -2 %).
        // Every step issues five (past the end the last tile once more, into the stage nobody reads any
        // more), so the wait above is always the same.
        const int ahead = j + 2 < tiles ? j + 2 : tiles - 1;
        const bf16_t *qt_tile = stages[STAGE][0], *gt_tile = stages[STAGE][1];
        const int q0 = (first + j) * 64;
        auto half = [&](auto half_tag) {
            constexpr int qt = decltype(half_tag)::value;
            const int qh = q0 + qt * 32;
            if (qh + 31 < wave_k0) // every query of this half precedes this wave's keys (wave uniform)
                return;
            // dP - delta in one go: the product accumulates onto -delta of its rows (the dQ kernel leaves the deltas
            // negated), one subtraction per score less on the vector ALU that bounds this kernel
            f32x16 s = zero16(), dp;
#pragma unroll
            for (int q4 = 0; q4 < 4; ++q4) {
                const f32x4 minus4 = *reinterpret_cast<const f32x4 *>(&rows[STAGE][1][qt * 32 + 8 * q4 + 4 * g]);
#pragma unroll
                for (int e = 0; e < 4; ++e)
                    dp[q4 * 4 + e] = minus4[e];
            }
#pragma unroll
            for (int ks = 0; ks < 4; ++ks) {
                s = mfma(qrows.load(qt_tile, qt, ks), kf[ks], s);
                dp = mfma(qrows.load(gt_tile, qt, ks), vf[ks], dp);
            }
            // the causal mask costs three instructions per score: only in the half tiles that straddle the
            // diagonal (a wave-uniform branch; as a per-element condition it is paid everywhere)
            auto probabilities = [&](auto masked) {
#pragma unroll
                for (int q4 = 0; q4 < 4; ++q4) {
                    const int at = qt * 32 + 8 * q4 + 4 * g;
                    const f32x4 lse4 = *reinterpret_cast<const f32x4 *>(&rows[STAGE][0][at]);
#pragma unroll
                    for (int e = 0; e < 4; ++e) {
                        const int r = q4 * 4 + e;
                        float p = exp2_fast(fmaf(s[r], c, -lse4[e]));
                        if (decltype(masked)::value && krow > q0 + at + e)
                            p = 0.f;
                        s[r] = p;
                        dp[r] = p * dp[r];
                    }
                }
            };
            if (qh < wave_k0 + 31)
                probabilities(Const<1>{});
            else
                probabilities(Const<0>{});
#pragma unroll
            for (int kk2 = 0; kk2 < 2; ++kk2) {
                const bf16x8 pf = acc_to_frag(s, kk2);
                const bf16x8 dsf = acc_to_frag(dp, kk2);
#pragma unroll
                for (int dt = 0; dt < 2; ++dt) {
                    dv[dt] = mfma(qcols.load(gt_tile, qt * 2 + kk2, dt), pf, dv[dt]);
                    dk[dt] = mfma(qcols.load(qt_tile, qt * 2 + kk2, dt), dsf, dk[dt]);
                }
            }
        };
        half(Const<0>{});
        half(Const<1>{});
        produce((STAGE + 2) % 3, ahead);
    };
    for (int j = 0; j < tiles; j += 3) { // tiles is block uniform
        step(Const<0>{}, j);
        if (j + 1 < tiles)
            step(Const<1>{}, j + 1);
        if (j + 2 < tiles)
            step(Const<2>{}, j + 2);
    }
    wait_vmcnt<0>(); // no copy may land in LDS after the block has left
    bf16_t *kp = dK + (token0 + krow) * lddq + h * HD;
    bf16_t *vp = dV + (token0 + krow) * lddq + h * HD;
#pragma unroll
    for (int dt = 0; dt < 2; ++dt) {
        store_acc_rows(kp + dt * 32, dk[dt], scale, g);
        store_acc_rows(vp + dt * 32, dv[dt], 1.0f, g);
    }
}

// ---------------------------------------------------------------------------------------------
// dQ: block = 128 queries (4 waves x 32), loops over 64-key tiles up to the diagonal; K and V tiles
// arrive by asynchronous copies two tiles ahead; 32-key halves are processed in turn.
// ---------------------------------------------------------------------------------------------
__global__ __launch_bounds__(256, 3) void attn_bwd_dq_kernel(
    const bf16_t *__restrict__ Q, const bf16_t *__restrict__ K, const bf16_t *__restrict__ V, int ld,
    const bf16_t *__restrict__ dO, int lddo, const bf16_t *__restrict__ O, int ldo,
    const float *__restrict__ LSE, float *__restrict__ lse2_out, float *__restrict__ delta_out,
    bf16_t *__restrict__ dQ, int lddq, int T, int H, int pairs, float scale) {
    __shared__ __align__(1024) bf16_t stages[3][2][TILE_ELEMS]; // [stage][K | V]
    const CausalBlock block = causal_block(H, pairs);
    if (!block.live)
        return;
    const int q0 = (T / 128 - 1 - block.rank) * 128, h = block.h, b = block.b;
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6, g = lane >> 5;
    const int wave_q0 = q0 + wave * 32, qrow = wave_q0 + (lane & 31);
    const size_t token0 = size_t(b) * T;
    const float c = scale * LOG2E;
    const int tiles = (q0 + 128) / 64;
    const int my_tiles = wave_q0 / 64 + 1;
    const bf16_t *kbase = K + token0 * ld + h * HD, *vbase = V + token0 * ld + h * HD;
    const uint32_t lds0 = lds_address(&stages[0][0][0]);
    // a copy takes a wave-uniform tile address and a per-lane byte offset computed once: no vector arithmetic per tile
    const uint32_t lane_offset[2] = {tile_copy_offset(ld, wave, lane, 0), tile_copy_offset(ld, wave, lane, 1)};
    auto produce = [&](int stage, int j) {
        const uint32_t slot = lds0 + uint32_t(stage) * (2 * TILE_ELEMS * 2);
        const bf16_t *kt = kbase + size_t(j) * 64 * ld, *vt = vbase + size_t(j) * 64 * ld;
#pragma unroll
        for (int n = 0; n < 2; ++n) {
            async_copy16(__builtin_amdgcn_readfirstlane(slot + (wave + 4 * n) * 1024), kt, lane_offset[n]);
            async_copy16(__builtin_amdgcn_readfirstlane(slot + TILE_ELEMS * 2 + (wave + 4 * n) * 1024), vt, lane_offset[n]);
        }
    };
    produce(0, 0);
    if (tiles > 1)
        produce(1, 1);

    bf16x8 qf[4], gf[4];
    {
        const bf16_t *qp = Q + (token0 + qrow) * ld + h * HD + g * 8;
        const bf16_t *gp = dO + (token0 + qrow) * lddo + h * HD + g * 8;
#pragma unroll
        for (int ks = 0; ks < 4; ++ks) {
            qf[ks] = *reinterpret_cast<const bf16x8 *>(qp + ks * 16);
            gf[ks] = *reinterpret_cast<const bf16x8 *>(gp + ks * 16);
        }
    }
    // delta = rowsum(dO o O) and the log-sum-exp in base 2, for this block's own queries; also left in
    // memory for the dK/dV kernel, which runs after this one
    float del = 0.f;
    {
        const bf16_t *op = O + (token0 + qrow) * ldo + h * HD + g * 8;
#pragma unroll
        for (int ks = 0; ks < 4; ++ks) {
            const bf16x8 of = *reinterpret_cast<const bf16x8 *>(op + ks * 16);
#pragma unroll
            for (int e = 0; e < 8; ++e)
                del += float(gf[ks][e]) * float(of[e]);
        }
        del = halves_sum(del);
    }
    const size_t row_at = (size_t(b) * H + h) * T + qrow;
    const float lse = LSE[row_at] * LOG2E;
    if (g == 0) {
        delta_out[row_at] = -del; // negated: the dK/dV kernel starts its dP product from it
        lse2_out[row_at] = lse;
    }
    f32x16 dq[2] = {zero16(), zero16()};
    f32x16 minus_delta;
#pragma unroll
    for (int r = 0; r < 16; ++r)
        minus_delta[r] = -del;
    const RowFragOffsets krows(lane);
    const ColFragOffsets kcols(lane);

    auto step = [&](auto stage_tag, int j) {
        constexpr int STAGE = decltype(stage_tag)::value;
        if (j + 1 < tiles)
            wait_vmcnt<4>();
        else
            wait_vmcnt<0>();
        __syncthreads();
        // the copies of tile j+2 go out at the end of the step, where the waves have drifted apart: behind
        // the barrier every wave of the CU would queue its copies at the same moment
        if (j >= my_tiles) {
            if (j + 2 < tiles)
                produce((STAGE + 2) % 3, j + 2);
            return;
        }
        const bf16_t *kt = stages[STAGE][0], *vt = stages[STAGE][1];
        const int kv0 = j * 64;
        const bool diagonal = kv0 + 63 > wave_q0;
#pragma unroll
        for (int mt = 0; mt < 2; ++mt) {
            if (kv0 + mt * 32 > wave_q0 + 31) // every key of this half follows this wave's queries
                continue;
            // dP - delta in one go: the product accumulates onto a register set that holds -delta of this lane's query
            f32x16 s = zero16(), dp;
#pragma unroll
            for (int ks = 0; ks < 4; ++ks) {
                s = mfma(krows.load(kt, mt, ks), qf[ks], s);
                dp = mfma(krows.load(vt, mt, ks), gf[ks], ks == 0 ? minus_delta : dp);
            }
            // the causal mask only in the tiles that straddle the diagonal (wave-uniform branch)
            auto probabilities = [&](auto masked) {
#pragma unroll
                for (int r = 0; r < 16; ++r) {
                    float p = exp2_fast(fmaf(s[r], c, -lse));
                    if (decltype(masked)::value && kv0 + mt * 32 + acc_row(r, g) > qrow)
                        p = 0.f;
                    dp[r] = p * dp[r];
                }
            };
            if (diagonal)
                probabilities(Const<1>{});
            else
                probabilities(Const<0>{});
#pragma unroll
            for (int kk2 = 0; kk2 < 2; ++kk2) {
                const bf16x8 dsf = acc_to_frag(dp, kk2);
#pragma unroll
                for (int dt = 0; dt < 2; ++dt)
                    dq[dt] = mfma(kcols.load(kt, mt * 2 + kk2, dt), dsf, dq[dt]);
            }
        }
        if (j + 2 < tiles)
            produce((STAGE + 2) % 3, j + 2);
    };
    for (int j = 0; j < tiles; j += 3) { // tiles is block uniform
        step(Const<0>{}, j);
        if (j + 1 < tiles)
            step(Const<1>{}, j + 1);
        if (j + 2 < tiles)
            step(Const<2>{}, j + 2);
    }
    bf16_t *qp = dQ + (token0 + qrow) * lddq + h * HD;
#pragma unroll
    for (int dt = 0; dt < 2; ++dt)
        store_acc_rows(qp + dt * 32, dq[dt], scale, g);
}

void check_attention_shape(int B, int H, int T, int hd) {
    require(B > 0 && H > 0 && T > 0, "attention: empty shape");
    require(hd == HD, "attention: head_dim must be 64");
    require(T % 128 == 0, "attention: context must be a multiple of 128");
    require(size_t(B) * T < (size_t(1) << 31), "attention: too many tokens");
}
void check_matrix(const void *p, int ld, const char *name) {
    if (!p || (reinterpret_cast<uintptr_t>(p) & 15) || ld % 8)
        throw std::invalid_argument(std::string("attention operand ") + name +
                                    " must be non-null, 16-byte aligned, leading dimension % 8 == 0");
}

} // namespace

extern "C" int tgk_attn_fwd(hipStream_t stream, int B, int H, int T, int hd, const uint16_t *Q,
                            const uint16_t *K, const uint16_t *V, int ld, uint16_t *O, int ldo,
                            float *lse, float scale) {
    return guarded([&] {
        check_attention_shape(B, H, T, hd);
        check_matrix(Q, ld, "Q");
        check_matrix(K, ld, "K");
        check_matrix(V, ld, "V");
        check_matrix(O, ldo, "O");
        require(lse && !(reinterpret_cast<uintptr_t>(lse) & 15), "attention: lse must be 16-byte aligned");
        hipLaunchKernelGGL(attn_fwd_kernel, dim3(causal_grid(T / 128, B * H)), dim3(256), 0, stream, Q, K, V,
                           ld, O, ldo, lse, T, H, B * H, scale * LOG2E);
        check_hip(hipGetLastError(), "attention forward launch: ");
    });
}

extern "C" size_t tgk_attn_bwd_workspace(int B, int H, int T) {
    return 2 * size_t(B) * H * T * sizeof(float); // delta, and the log-sum-exp in base 2
}

namespace {
void attn_bwd_check(int B, int H, int T, int hd, const uint16_t *Q, const uint16_t *K, const uint16_t *V, int ld,
                    const uint16_t *O, int ldo, const float *lse, const uint16_t *dO, int lddo, uint16_t *dQ,
                    uint16_t *dK, uint16_t *dV, int lddq) {
    check_attention_shape(B, H, T, hd);
    check_matrix(Q, ld, "Q");
    check_matrix(K, ld, "K");
    check_matrix(V, ld, "V");
    check_matrix(O, ldo, "O");
    check_matrix(dO, lddo, "dO");
    check_matrix(dQ, lddq, "dQ");
    check_matrix(dK, lddq, "dK");
    check_matrix(dV, lddq, "dV");
    require(lse && !(reinterpret_cast<uintptr_t>(lse) & 15), "attention: lse must be 16-byte aligned");
}
// both backward kernels; `rows` holds delta[B*H*T] followed by the base-2 log-sum-exps[B*H*T]
void attn_bwd_launch(hipStream_t stream, int B, int H, int T, const uint16_t *Q, const uint16_t *K,
                     const uint16_t *V, int ld, const uint16_t *O, int ldo, const float *lse, const uint16_t *dO,
                     int lddo, uint16_t *dQ, uint16_t *dK, uint16_t *dV, int lddq, float scale, float *rows) {
    float *delta = rows, *lse2 = delta + size_t(B) * H * T;
    const dim3 grid(causal_grid(T / 128, B * H));
    hipLaunchKernelGGL(attn_bwd_dq_kernel, grid, dim3(256), 0, stream, Q, K, V, ld, dO, lddo, O, ldo, lse, lse2,
                       delta, dQ, lddq, T, H, B * H, scale);
    hipLaunchKernelGGL(attn_bwd_dkdv_kernel, grid, dim3(256), 0, stream, Q, K, V, ld, dO, lddo, lse2, delta, dK, dV,
                       lddq, T, H, B * H, scale);
    check_hip(hipGetLastError(), "attention backward launch: ");
}
} // namespace

extern "C" int tgk_attn_bwd(hipStream_t stream, int B, int H, int T, int hd, const uint16_t *Q,
                            const uint16_t *K, const uint16_t *V, int ld, const uint16_t *O, int ldo,
                            const float *lse, const uint16_t *dO, int lddo, uint16_t *dQ, uint16_t *dK,
                            uint16_t *dV, int lddq, float scale, void *workspace,
                            size_t workspace_bytes) {
    return guarded([&] {
        attn_bwd_check(B, H, T, hd, Q, K, V, ld, O, ldo, lse, dO, lddo, dQ, dK, dV, lddq);
        require(workspace && workspace_bytes >= tgk_attn_bwd_workspace(B, H, T) &&
                    !(reinterpret_cast<uintptr_t>(workspace) & 15),
                "attention backward: workspace too small (see tgk_attn_bwd_workspace)");
        attn_bwd_launch(stream, B, H, T, Q, K, V, ld, O, ldo, lse, dO, lddo, dQ, dK, dV, lddq, scale,
                        static_cast<float *>(workspace));
    });
}

// ---- the same backward for callers that cannot allocate -------------------------------------------
// The two row vectors the kernels exchange (delta and the base-2 log-sum-exp, B*H*T floats each) live in
// a device array of this library instead of a caller's workspace.  Every GPU the library runs on holds
// its own copy of the array at its own address; the address is looked up once per device, with that
// device current, and only that address - never the array's name - is handed to kernels.  The dQ kernel
// overwrites every row the dK/dV kernel reads, so nothing has to be cleared between calls.
namespace {
constexpr size_t STATIC_BWD_ROWS = size_t(1) << 20; // B*H*T of one call: 8 MiB of device memory per GPU
static __device__ __align__(256) float scratch[2 * STATIC_BWD_ROWS];
constexpr int STATIC_MAX_DEVICES = 64;
std::atomic<float *> scratch_address[STATIC_MAX_DEVICES];

float *scratch_on_current_device() {
    int device = 0;
    check_hip(hipGetDevice(&device), "attention backward (static): ");
    require(device >= 0 && device < STATIC_MAX_DEVICES, "attention backward (static): device index out of range");
    float *address = scratch_address[device].load(std::memory_order_acquire);
    if (!address) {
        void *found = nullptr;
        check_hip(hipGetSymbolAddress(&found, HIP_SYMBOL(scratch)), "attention backward (static) scratch address: ");
        require(found != nullptr, "attention backward (static): the scratch array has no device address");
        address = static_cast<float *>(found);
        scratch_address[device].store(address, std::memory_order_release);
    }
    return address;
}
} // namespace

// Also the set-up call: it looks up the array's address on the current device, so that a later tgk_attn_bwd_static
// on this device (under stream capture, say) has nothing left to resolve.  A failed lookup is reported by that call.
extern "C" size_t tgk_attn_bwd_static_max_rows(void) {
    try {
        (void)scratch_on_current_device();
    } catch (const std::exception &) {
    }
    return STATIC_BWD_ROWS;
}

extern "C" int tgk_attn_bwd_static(hipStream_t stream, int B, int H, int T, int hd, const uint16_t *Q,
                                   const uint16_t *K, const uint16_t *V, int ld, const uint16_t *O, int ldo,
                                   const float *lse, const uint16_t *dO, int lddo, uint16_t *dQ, uint16_t *dK,
                                   uint16_t *dV, int lddq, float scale) {
    return guarded([&] {
        attn_bwd_check(B, H, T, hd, Q, K, V, ld, O, ldo, lse, dO, lddo, dQ, dK, dV, lddq);
        require(size_t(B) * H * T <= STATIC_BWD_ROWS,
                "attention backward (static): B*H*T exceeds tgk_attn_bwd_static_max_rows() = 1048576; "
                "use tgk_attn_bwd with a workspace");
        attn_bwd_launch(stream, B, H, T, Q, K, V, ld, O, ldo, lse, dO, lddo, dQ, dK, dV, lddq, scale,
                        scratch_on_current_device());
    });
}
