// bf16 MFMA GEMM family for gfx950: forward Y = X W^T, dgrad dX = dY W, wgrad dW = dY^T X.
// Replaces project / matmul+cast_result / weight_gradient of the reference
// (cuda/mma.cuh:77-108, cuda/ops.cuh:30-55, cuda/ops.cuh:83-109) and, through the fixed-order
// folds of split-K pieces, reduce_gradients (cuda/trainer.cuh:9-47).
//
// Every kernel computes C[m][n] = sum_k A(m,k) B(n,k).  Each operand is either "k-contiguous" (stored
// [row][k]) or "k-strided" (stored [k][row]):
//   forward : A = X  [M][K] k-contiguous, B = W [N][K] k-contiguous
//   dgrad   : A = dY [M][N] k-contiguous, B = the transposed weight Wt [K][N] k-contiguous (tgk_gemm_dgrad_t),
//             or W [N][K] read as (n = K index, k = N index): k-strided (tgk_gemm_dgrad)
//   wgrad   : A = dY [M][N] k-strided (m = out index), B = X [M][K] k-strided, fp32 out, split-K
//
// Data path: global -> LDS directly (global_load_lds_dwordx4: no staging registers, no LDS store
// instructions); the copies keep running across tile boundaries, because a block is persistent and walks a
// list of work items (tile x split).  LDS tiles are unpadded and XOR-swizzled on 16-byte chunks (a wave-wide
// copy fills 1 KiB of LDS contiguously, so padding is not available); measured bank conflicts are zero.
// k-contiguous tiles give each MFMA fragment with one ds_read_b128; k-strided tiles keep the natural [k][row]
// image and are read with the transposing ds_read_b64_tr_b16.  256 threads = 2x2 waves; the 64-k kernels use
// v_mfma_f32_16x16x32_bf16 (more flops per watt on real operands, and the kernels run against the power limit),
// gemm_kernel v_mfma_f32_32x32x16_bf16; either way the instruction's A operand is fed with *our B rows* so that a
// lane ends up holding 4 consecutive n for one m.  Results leave through a wave-private LDS transposition so that stores cover
// whole row pieces, with the residual / GELU / GELU' epilogues applied in that layout.
//
// Three kernels: gemm64_kernel (two stages of 64 k, copies placed between the MFMAs: every training shape),
// gemm_kernel (S stages of 32 k: the shapes gemm64_kernel does not take), wgrad_batch_kernel (the weight
// gradients of several matrices in one launch).
#include "common.h"
#include <atomic>
#include <type_traits>
#include <vector>
#include "../../include/tgk_kernels.h"

namespace {

enum EpilogueMode { EPI_PLAIN = 0, EPI_RESIDUAL = 1, EPI_GELU = 2, EPI_GELU_BWD = 3 };

// An accumulator lane holds 4 consecutive n of one m per register quad.  A plain epilogue (fp32
// outputs) stores from that layout.  A STAGED epilogue has the kernel round each 32x32 tile to bf16 and
// transpose it through a wave-private LDS buffer, and then works on 8 consecutive n of one row per
// lane: one load / store instruction covers 16 rows x 64 contiguous bytes instead of 32 rows x 16
// bytes.  Its second input (residual, saved pre-activation) is fetched in that row layout two k-tiles
// before the end of the reduction, so the epilogue does not wait on memory.
struct EpilogueBf16 {
    static constexpr bool BF16 = true;
    bf16_t *out;
    int ld_out;
    const bf16_t *aux; // residual (EPI_RESIDUAL) or saved pre-activation (EPI_GELU_BWD)
    int ld_aux;
    bf16_t *out2; // GELU output (EPI_GELU)
    int ld_out2;
    int mode;
    TG_DEVICE bool wants_aux() const { return mode == EPI_RESIDUAL || mode == EPI_GELU_BWD; }
    TG_DEVICE u32x4 load_aux(int m, int n) const {
        return *reinterpret_cast<const u32x4 *>(aux + size_t(m) * ld_aux + n);
    }
    // y: the bf16-rounded accumulators of row m, columns n .. n+7
    template <int MODE> TG_DEVICE void finish_as(int m, int n, u32x4 y, u32x4 a) const {
        if constexpr (MODE == EPI_RESIDUAL) {
            // RN(RN(acc) + residual): the bf16 add of cuda/mma.cuh:95-97
#pragma unroll
            for (int e = 0; e < 4; ++e)
                y[e] = pack_bf16(bf16_lo(y[e]) + bf16_lo(a[e]), bf16_hi(y[e]) + bf16_hi(a[e]));
        } else if constexpr (MODE == EPI_GELU_BWD) {
            // du = RN(RN(acc) * gelu'(u))
#pragma unroll
            for (int e = 0; e < 4; ++e)
                y[e] = pack_bf16(bf16_lo(y[e]) * gelu_grad_f(bf16_lo(a[e])),
                                 bf16_hi(y[e]) * gelu_grad_f(bf16_hi(a[e])));
        } else if constexpr (MODE == EPI_GELU) {
            u32x4 g;
#pragma unroll
            for (int e = 0; e < 4; ++e)
                g[e] = pack_bf16(gelu_f(bf16_lo(y[e])), gelu_f(bf16_hi(y[e])));
            // Both outputs stream past the L2: the pre-activation is not read again before the backward pass, and the
            // activation (100 MB at the training shape) is far larger than the L2, whose lines the operand panels of
            // this product need (measured on the step: -0.8 % for the first, another -0.8 % for the second; the
            // same on the plain and residual outputs costs 1 %).
            __builtin_nontemporal_store(g, reinterpret_cast<u32x4 *>(out2 + size_t(m) * ld_out2 + n));
            __builtin_nontemporal_store(y, reinterpret_cast<u32x4 *>(out + size_t(m) * ld_out + n));
            return;
        }
        *reinterpret_cast<u32x4 *>(out + size_t(m) * ld_out + n) = y;
    }
    TG_DEVICE void finish(int m, int n, u32x4 y, u32x4 a) const {
        if (mode == EPI_RESIDUAL)
            finish_as<EPI_RESIDUAL>(m, n, y, a);
        else if (mode == EPI_GELU_BWD)
            finish_as<EPI_GELU_BWD>(m, n, y, a);
        else if (mode == EPI_GELU)
            finish_as<EPI_GELU>(m, n, y, a);
        else
            finish_as<EPI_PLAIN>(m, n, y, a);
    }
};
// The same with the mode fixed at compile time.  A wave's loads and stores share one in-order counter, and a wait
// names how many younger operations may stay outstanding: with the mode decided by branches that number is unknown
// and every 32 x 32 block of the epilogue ends up waiting for its own stores to be acknowledged; with straight-line
// code the stores of a block stay in flight while the next is rounded and transposed.
template <int MODE> struct EpilogueBf16As {
    static constexpr bool BF16 = true;
    // vector-memory instructions per 32 x 32 block of the staged epilogue: two 16-byte stores (four with the GELU
    // output), two 16-byte loads of the second input
    static constexpr int MEMORY_OPS_PER_BLOCK = MODE == EPI_PLAIN ? 2 : 4;
    EpilogueBf16 any;
    TG_DEVICE bool wants_aux() const { return MODE == EPI_RESIDUAL || MODE == EPI_GELU_BWD; }
    TG_DEVICE u32x4 load_aux(int m, int n) const { return any.load_aux(m, n); }
    TG_DEVICE void finish(int m, int n, u32x4 y, u32x4 a) const { any.finish_as<MODE>(m, n, y, a); }
};

// fp32 outputs (weight gradients, split-K slabs): tiles go through the same kind of wave-private LDS
// buffer untouched, and a lane finishes 4 consecutive n - 8 lanes cover a 128-byte row piece.
struct EpilogueF32 {
    static constexpr bool BF16 = false;
    float *out;
    int ld_out;
    size_t split_stride; // elements between split-K slabs
    int accumulate;      // only honoured when there is a single split
    TG_DEVICE bool wants_aux() const { return false; }
    TG_DEVICE u32x4 load_aux(int, int) const { return u32x4{0, 0, 0, 0}; }
    TG_DEVICE void finish(int m, int n, f32x4 value, int split) const {
        f32x4 *p = reinterpret_cast<f32x4 *>(out + split * split_stride + size_t(m) * ld_out + n);
        if (accumulate)
            value += *p;
        *p = value;
    }
};

// bf16 outputs: each 32x32 accumulator tile is rounded and transposed through a wave-private LDS buffer
// (32 rows of 64 bytes, 16-byte chunk c of row r at c ^ ((r >> 2) & 3)), so that a lane finishes 8
// consecutive n of rows get_row and get_row + 16.  LDS operations of one wave execute in order, so no
// barrier is needed around the buffer.  The epilogue's second input (residual, saved pre-activation) is
// fetched in that row layout one 32x32 tile ahead; `first` is the pair for tile (0, 0), requested by the
// caller before its last MFMAs (load_aux_pair) - holding all FM x FN pairs there costs 48 registers.
template <int FM, int FN, class Epilogue>
TG_DEVICE void load_aux_pair(const Epilogue &epilogue, int tile, int m_base, int n_base, int lane, u32x4 (&pair)[2]) {
    const int i = tile / FN, j = tile - i * FN;
    const int m = m_base + i * 32 + (lane >> 2), n = n_base + j * 32 + (lane & 3) * 8;
    pair[0] = epilogue.load_aux(m, n);
    pair[1] = epilogue.load_aux(m + 16, n);
}
template <int FM, int FN, class Epilogue>
TG_DEVICE void staged_store_bf16(const f32x16 (&acc)[FM][FN], const u32x4 (&first)[2], unsigned char *mine,
                                 const Epilogue &epilogue, int m_base, int n_base, int lane) {
    const int get_row = lane >> 2, get_chunk = lane & 3;
    const int row = lane & 31;
    unsigned char *put = mine + row * 64 + (lane >> 5) * 8;
    const int put_swizzle = (row >> 2) & 3;
    // rows r and r + 16 share a swizzle term, so the second half is 1 KiB further on
    const unsigned char *get = mine + get_row * 64 + ((get_chunk ^ ((get_row >> 2) & 3)) << 4);
    const bool wants_aux = epilogue.wants_aux();
    u32x4 aux[2] = {first[0], first[1]};
#pragma unroll
    for (int i = 0; i < FM; ++i)
#pragma unroll
        for (int j = 0; j < FN; ++j) {
            u32x4 next[2] = {aux[0], aux[1]};
            if (wants_aux && i * FN + j + 1 < FM * FN)
                load_aux_pair<FM, FN>(epilogue, i * FN + j + 1, m_base, n_base, lane, next);
            const int m = m_base + i * 32 + get_row, n = n_base + j * 32 + get_chunk * 8;
#pragma unroll
            for (int q = 0; q < 4; ++q) {
                u32x2 packed;
                packed.x = pack_bf16(acc[i][j][q * 4 + 0], acc[i][j][q * 4 + 1]);
                packed.y = pack_bf16(acc[i][j][q * 4 + 2], acc[i][j][q * 4 + 3]);
                *reinterpret_cast<u32x2 *>(put + ((q ^ put_swizzle) << 4)) = packed;
            }
            epilogue.finish(m, n, *reinterpret_cast<const u32x4 *>(get), aux[0]);
            epilogue.finish(m + 16, n, *reinterpret_cast<const u32x4 *>(get + 1024), aux[1]);
            aux[0] = next[0];
            aux[1] = next[1];
        }
}

// fp32 outputs: the same through a buffer of 32 rows of 128 bytes (16-byte chunk c of row r at c ^ ((r >> 1) & 7));
// a lane finishes 4 consecutive n, 8 lanes cover a 128-byte row piece.
template <int FM, int FN, class Epilogue>
TG_DEVICE void staged_store_f32(const f32x16 (&acc)[FM][FN], unsigned char *mine, const Epilogue &epilogue,
                                int m_base, int n_base, int lane, int split) {
    const int row = lane & 31;
    unsigned char *put = mine + row * 128;
    const int put_swizzle = (row >> 1) & 7, g = lane >> 5;
    const int first_row = lane >> 3, chunk = lane & 7;
#pragma unroll
    for (int i = 0; i < FM; ++i)
#pragma unroll
        for (int j = 0; j < FN; ++j) {
#pragma unroll
            for (int q = 0; q < 4; ++q) {
                const f32x4 v = {acc[i][j][q * 4 + 0], acc[i][j][q * 4 + 1], acc[i][j][q * 4 + 2], acc[i][j][q * 4 + 3]};
                *reinterpret_cast<f32x4 *>(put + (((2 * q + g) ^ put_swizzle) << 4)) = v;
            }
#pragma unroll
            for (int part = 0; part < 4; ++part) {
                const int r = first_row + part * 8;
                const f32x4 v = *reinterpret_cast<const f32x4 *>(mine + r * 128 + ((chunk ^ ((r >> 1) & 7)) << 4));
                epilogue.finish(m_base + i * 32 + r, n_base + j * 32 + chunk * 4, v, split);
            }
        }
}

// The same two stores for accumulators kept as 2 x 2 tiles of 16 x 16 per 32 x 32 block (v_mfma_f32_16x16x32_bf16 fed
// with B rows as its first operand): tile [tm][tn] of a block holds, in lane l, row m = 16 tm + l % 16 and columns
// n = 16 tn + 4 (l / 16) .. + 3.
template <int FM, int FN, class Epilogue>
TG_DEVICE void staged_store_bf16(const f32x4 (&acc)[FM][FN][2][2], const u32x4 (&first)[2], unsigned char *mine,
                                 const Epilogue &epilogue, int m_base, int n_base, int lane) {
    const int get_row = lane >> 2, get_chunk = lane & 3;
    const int row = lane & 15;
    unsigned char *put = mine + row * 64 + ((lane >> 4) & 1) * 8;
    const int put_swizzle = (row >> 2) & 3, put_chunk = lane >> 5;
    const unsigned char *get = mine + get_row * 64 + ((get_chunk ^ ((get_row >> 2) & 3)) << 4);
    const bool wants_aux = epilogue.wants_aux();
    // the second input is fetched one block ahead (two or more measured no faster, and cost registers)
    u32x4 aux[2] = {first[0], first[1]};
#pragma unroll
    for (int i = 0; i < FM; ++i)
#pragma unroll
        for (int j = 0; j < FN; ++j) {
            u32x4 next[2] = {aux[0], aux[1]};
            if (wants_aux && i * FN + j + 1 < FM * FN)
                load_aux_pair<FM, FN>(epilogue, i * FN + j + 1, m_base, n_base, lane, next);
            const int m = m_base + i * 32 + get_row, n = n_base + j * 32 + get_chunk * 8;
#pragma unroll
            for (int tm = 0; tm < 2; ++tm)
#pragma unroll
                for (int tn = 0; tn < 2; ++tn) {
                    const f32x4 &tile = acc[i][j][tm][tn];
                    u32x2 packed;
                    packed.x = pack_bf16(tile[0], tile[1]);
                    packed.y = pack_bf16(tile[2], tile[3]);
                    *reinterpret_cast<u32x2 *>(put + tm * 1024 + (((2 * tn + put_chunk) ^ put_swizzle) << 4)) = packed;
                }
            epilogue.finish(m, n, *reinterpret_cast<const u32x4 *>(get), aux[0]);
            epilogue.finish(m + 16, n, *reinterpret_cast<const u32x4 *>(get + 1024), aux[1]);
            aux[0] = next[0];
            aux[1] = next[1];
        }
}
template <int FM, int FN, class Epilogue>
TG_DEVICE void staged_store_f32(const f32x4 (&acc)[FM][FN][2][2], unsigned char *mine, const Epilogue &epilogue,
                                int m_base, int n_base, int lane, int split) {
    const int row = lane & 15;
    unsigned char *put = mine + row * 128;
    const int put_swizzle = (row >> 1) & 7, put_chunk = lane >> 4;
    const int first_row = lane >> 3, chunk = lane & 7;
#pragma unroll
    for (int i = 0; i < FM; ++i)
#pragma unroll
        for (int j = 0; j < FN; ++j) {
#pragma unroll
            for (int tm = 0; tm < 2; ++tm)
#pragma unroll
                for (int tn = 0; tn < 2; ++tn)
                    *reinterpret_cast<f32x4 *>(put + tm * 2048 + (((4 * tn + put_chunk) ^ put_swizzle) << 4)) =
                        acc[i][j][tm][tn];
#pragma unroll
            for (int part = 0; part < 4; ++part) {
                const int r = first_row + part * 8;
                const f32x4 v = *reinterpret_cast<const f32x4 *>(mine + r * 128 + ((chunk ^ ((r >> 1) & 7)) << 4));
                epilogue.finish(m_base + i * 32 + r, n_base + j * 32 + chunk * 4, v, split);
            }
        }
}

constexpr int BK = 32;
typedef short s16x4 __attribute__((ext_vector_type(4)));
typedef short s16x8 __attribute__((ext_vector_type(8)));
typedef __attribute__((address_space(3))) s16x4 lds_s16x4;

// ---- k-contiguous operand tile: ROWS rows x 32 k, 64-byte rows, 16-byte chunk c of row r stored
// at chunk c ^ ((r >> 2) & 3) ------------------------------------------------------------------
template <int ROWS> struct TileKC {
    static constexpr int LOADS = ROWS * 4 / 256; // wave-wide copies per thread per stage
    static constexpr int BYTES = ROWS * 64;
    // element offset (relative to the tile origin at k = 0) that this lane fetches for copy j
    TG_DEVICE static int64_t source_offset(int j, int tid, int ld) {
        const int wave = tid >> 6, lane = tid & 63;
        const int row = (j * 4 + wave) * 16 + (lane >> 2), phys = lane & 3;
        const int chunk = phys ^ ((row >> 2) & 3);
        return int64_t(row) * ld + chunk * 8;
    }
    TG_DEVICE static uint32_t lds_offset(int j, int tid) { // wave-uniform
        return uint32_t((j * 4 + (tid >> 6)) * 1024);
    }
    // fragment for rows row0 + lane%32, k-step ks (16 k): k = ks*16 + 8*(lane/32) .. +7
    TG_DEVICE static bf16x8 frag(const unsigned char *tile, int row0, int ks, int lane) {
        const int row = row0 + (lane & 31), chunk = (ks * 2 + (lane >> 5)) ^ ((row >> 2) & 3);
        return *reinterpret_cast<const bf16x8 *>(tile + row * 64 + chunk * 16);
    }
};

// ---- k-strided operand tile: source is [k][row]; LDS image 32 k-rows x ROWS columns, natural
// layout with 16-byte chunk p of k-row r stored at p ^ swizzle(r); read with the transposing load
template <int ROWS> struct TileKS {
    static constexpr int LOADS = ROWS * 4 / 256;
    static constexpr int BYTES = ROWS * 64;
    static constexpr int CHUNKS_PER_ROW = ROWS / 8;
    TG_DEVICE static int swizzle(int r) {
        // row stride of 256 B multiples: 4 consecutive k-rows start in the same bank; 384 B: every other one.  The
        // 16-row fragments read k-rows r and r + 8 in one pass, 32 bytes of each: bit 3 of r moves them 32 bytes apart.
        return (ROWS % 128 == 0 ? ((r & 3) << 2) : (((r >> 1) & 1) << 2)) | (((r >> 3) & 1) << 1);
    }
    TG_DEVICE static int64_t source_offset(int j, int tid, int ld) {
        const int wave = tid >> 6, lane = tid & 63;
        const int q = (j * 4 + wave) * 64 + lane, r = q / CHUNKS_PER_ROW, p = q - r * CHUNKS_PER_ROW;
        const int chunk = p ^ swizzle(r);
        return int64_t(r) * ld + chunk * 8;
    }
    TG_DEVICE static uint32_t lds_offset(int j, int tid) {
        return uint32_t((j * 4 + (tid >> 6)) * 1024);
    }
    // fragment for columns (operand rows) row0 + lane%32, k = ks*16 + 8*(lane/32) .. +7, natural order
    TG_DEVICE static bf16x8 frag(const unsigned char *tile, int row0, int ks, int lane) {
        const int g = lane >> 5, blk = (lane >> 4) & 1, i = lane & 15;
        const int r = ks * 16 + 8 * g + (i >> 2);
        const int col = row0 + 16 * blk + 4 * (i & 3);
        const int chunk = (col >> 3) ^ swizzle(r);
        const unsigned char *p = tile + r * (ROWS * 2) + chunk * 16 + (i & 1) * 8;
        const s16x4 lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_s16x4 *)(p));
        const s16x4 hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_s16x4 *)(p + 4 * ROWS * 2));
        const s16x8 both = __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7);
        return __builtin_bit_cast(bf16x8, both);
    }
    // fragment of a 16-column tile: columns row0 + lane%16, k = k0 + 8*(lane/16) .. +7
    TG_DEVICE static bf16x8 frag16(const unsigned char *tile, int row0, int k0, int lane) {
        const int g = lane >> 4, i = lane & 15;
        const int r = k0 + 8 * g + (i >> 2);
        const int col = row0 + 4 * (i & 3);
        const unsigned char *p = tile + r * (ROWS * 2) + (i & 1) * 8;
        const s16x4 lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_s16x4 *)(p + (((col >> 3) ^ swizzle(r)) << 4)));
        const s16x4 hi =
            __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_s16x4 *)(p + 4 * ROWS * 2 + (((col >> 3) ^ swizzle(r + 4)) << 4)));
        const s16x8 both = __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7);
        return __builtin_bit_cast(bf16x8, both);
    }
};

template <int ROWS, bool KC> struct TileOf;
template <int ROWS> struct TileOf<ROWS, true> { using type = TileKC<ROWS>; };
template <int ROWS> struct TileOf<ROWS, false> { using type = TileKS<ROWS>; };

// pipeline stages plus one 32 x 32 output tile per wave for the row-coalescing epilogue
template <int BM, int BN, int S, class Epilogue> constexpr size_t lds_bytes() {
    return size_t(S) * (BM + BN) * 64 + 4 * (Epilogue::BF16 ? 2048 : 4096);
}

// C[m][n] = sum_k A(m,k) B(n,k).  A k-contiguous: A[m][k] (lda); k-strided: A[k][m] (lda).  Same for B.
// Work items = tiles x splits, dealt to persistent blocks; loads run S-1 k-tiles ahead of the MFMAs and
// continue across item boundaries.
template <int BM, int BN, int S, bool AKC, bool BKC, class Epilogue>
__global__ __launch_bounds__(256, 2) void gemm_kernel(const bf16_t *__restrict__ A, int lda,
                                                    const bf16_t *__restrict__ B, int ldb, int k_tiles,
                                                    int splits, int tiles_n, int tiles_total, int xcd_cols,
                                                    Epilogue epilogue) {
    using TA = typename TileOf<BM, AKC>::type;
    using TB = typename TileOf<BN, BKC>::type;
    constexpr int WM = BM / 2, WN = BN / 2, FM = WM / 32, FN = WN / 32;
    constexpr int LA = TA::LOADS, LB = TB::LOADS, LOADS = LA + LB;
    constexpr int STAGE = TA::BYTES + TB::BYTES;
    extern __shared__ __align__(16) unsigned char smem[];
    const uint32_t smem_base = lds_address(smem);

    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int wm = (wave >> 1) * WM, wn = (wave & 1) * WN;
    const int items = tiles_total * splits, stride = gridDim.x;

    // item -> (m0, n0, first k-tile, k-tile count).  Consecutive block ids sit on consecutive XCDs, each
    // with an L2 of its own, so item i belongs to XCD i % 8 and is that XCD's (i / 8)-th item.  The tile
    // grid is cut into (8 / xcd_cols) x xcd_cols rectangles, one per XCD, walked row-major: an XCD
    // streams its rows of A once and keeps its columns of B in L2.  (xcd_cols = 1 with split-K items:
    // every XCD owns a contiguous run of (split, tile).)
    auto locate = [&](int item, int &m0, int &n0, int &kt0, int &nk) {
        int split = 0, tile_m, tile_n;
        if ((items & 7) == 0 && xcd_cols > 1) {
            const int xcd = item & 7, index = item >> 3;
            const int cols = tiles_n / xcd_cols, rows = (tiles_total / tiles_n) / (8 / xcd_cols);
            tile_m = (xcd / xcd_cols) * rows + index / cols;
            tile_n = (xcd % xcd_cols) * cols + index % cols;
        } else {
            int logical = item;
            if ((items & 7) == 0)
                logical = (item & 7) * (items >> 3) + (item >> 3);
            split = logical / tiles_total;
            const int tile = logical - split * tiles_total;
            tile_m = tile / tiles_n;
            tile_n = tile % tiles_n;
        }
        m0 = tile_m * BM;
        n0 = tile_n * BN;
        kt0 = split * k_tiles / splits;
        nk = (split + 1) * k_tiles / splits - kt0;
        return split;
    };

    // ---- producer state -------------------------------------------------------------------------
    int p_item = blockIdx.x, p_left = 0, p_slot = 0;
    const bf16_t *pa[LA], *pb[LB];
    int64_t a_step = AKC ? BK : int64_t(BK) * lda, b_step = BKC ? BK : int64_t(BK) * ldb;
    auto producer_open = [&]() { // point the copy sources at the first k-tile of p_item
        int m0, n0, kt0, nk;
        locate(p_item, m0, n0, kt0, nk);
        p_left = nk;
        const bf16_t *a0 = AKC ? A + int64_t(m0) * lda + int64_t(kt0) * BK : A + int64_t(kt0) * BK * lda + m0;
        const bf16_t *b0 = BKC ? B + int64_t(n0) * ldb + int64_t(kt0) * BK : B + int64_t(kt0) * BK * ldb + n0;
#pragma unroll
        for (int j = 0; j < LA; ++j)
            pa[j] = a0 + TA::source_offset(j, tid, lda);
#pragma unroll
        for (int j = 0; j < LB; ++j)
            pb[j] = b0 + TB::source_offset(j, tid, ldb);
    };
    auto produce = [&]() { // issue the copies of one k-tile into slot p_slot; returns false when out of work
        if (p_left == 0) {
            p_item += stride;
            if (p_item >= items)
                return false;
            producer_open();
        }
        const uint32_t base = smem_base + uint32_t(p_slot) * STAGE;
#pragma unroll
        for (int j = 0; j < LA; ++j) {
            async_copy16(__builtin_amdgcn_readfirstlane(base + TA::lds_offset(j, tid)), pa[j]);
            pa[j] += a_step;
        }
#pragma unroll
        for (int j = 0; j < LB; ++j) {
            async_copy16(__builtin_amdgcn_readfirstlane(base + TA::BYTES + TB::lds_offset(j, tid)), pb[j]);
            pb[j] += b_step;
        }
        --p_left;
        p_slot = p_slot + 1 == S ? 0 : p_slot + 1;
        return true;
    };

    if (p_item >= items)
        return;
    producer_open();
    int inflight = 0; // stages issued and not yet consumed
#pragma unroll
    for (int s = 0; s < S - 1; ++s)
        if (produce())
            ++inflight;

    // Wait until at most `allowed` of this wave's newest stages are still in flight.
    auto wait_stages = [&](int allowed) {
        if (S >= 5 && allowed >= 3)
            wait_vmcnt<3 * LOADS>();
        else if (S >= 4 && allowed == 2)
            wait_vmcnt<2 * LOADS>();
        else if (S >= 3 && allowed == 1)
            wait_vmcnt<1 * LOADS>();
        else
            wait_vmcnt<0>();
    };
    auto load_frags = [&](bf16x8 (&af)[FM], bf16x8 (&bfr)[FN], int slot, int ks) {
        const unsigned char *sa = smem + slot * STAGE, *sb = sa + TA::BYTES;
#pragma unroll
        for (int i = 0; i < FM; ++i)
            af[i] = TA::frag(sa, wm + i * 32, ks, lane);
#pragma unroll
        for (int j = 0; j < FN; ++j)
            bfr[j] = TB::frag(sb, wn + j * 32, ks, lane);
    };

    // ---- consumer ---------------------------------------------------------------------------------
    // Stages are made visible one k-tile early: iteration t starts by making stage t+1 visible, so the
    // first fragments of tile t+1 can be read at the end of iteration t and the MFMAs of the next
    // iteration start straight after its barrier.
    bf16x8 af0[FM], bf0[FN], af1[FM], bf1[FN];
    int c_slot = 0;
    wait_stages(inflight - 1); // stage 0 landed
    __syncthreads();
    load_frags(af0, bf0, 0, 0);
    for (int item = blockIdx.x; item < items; item += stride) {
        int m0, n0, kt0, nk;
        const int split = locate(item, m0, n0, kt0, nk);
        f32x16 acc[FM][FN];
#pragma unroll
        for (int i = 0; i < FM; ++i)
#pragma unroll
            for (int j = 0; j < FN; ++j)
#pragma unroll
                for (int r = 0; r < 16; ++r)
                    acc[i][j][r] = 0.f;
        u32x4 aux[2] = {u32x4{0, 0, 0, 0}, u32x4{0, 0, 0, 0}}; // the epilogue's second input for tile (0, 0)
        const int aux_at = nk > 2 ? nk - 2 : 0;
        for (int kt = 0; kt < nk; ++kt) {
            if constexpr (Epilogue::BF16)
                if (kt == aux_at && epilogue.wants_aux())
                    load_aux_pair<FM, FN>(epilogue, 0, m0 + wm, n0 + wn, lane, aux);
            // in flight now: the stage being consumed (landed), then inflight-1 younger ones; the next one
            // must land too
            wait_stages(inflight >= 2 ? inflight - 2 : 0);
            __syncthreads();
            --inflight;
            if (produce())
                ++inflight;
            const int next_slot = c_slot + 1 == S ? 0 : c_slot + 1;
            load_frags(af1, bf1, c_slot, 1);
#pragma unroll
            for (int i = 0; i < FM; ++i)
#pragma unroll
                for (int j = 0; j < FN; ++j)
                    acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(bf0[j], af0[i], acc[i][j], 0, 0, 0);
            load_frags(af0, bf0, next_slot, 0);
#pragma unroll
            for (int i = 0; i < FM; ++i)
#pragma unroll
                for (int j = 0; j < FN; ++j)
                    acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(bf1[j], af1[i], acc[i][j], 0, 0, 0);
            c_slot = next_slot;
        }
        if constexpr (Epilogue::BF16) {
            staged_store_bf16<FM, FN>(acc, aux, smem + S * STAGE + wave * 2048, epilogue, m0 + wm, n0 + wn, lane);
        } else {
            staged_store_f32<FM, FN>(acc, smem + S * STAGE + wave * 4096, epilogue, m0 + wm, n0 + wn, lane, split);
        }
    }
    wait_vmcnt<0>();
}

// ---- 64 k per stage, two stages --------------------------------------------------------------------
// k-contiguous tile of ROWS rows x 64 k: 128-byte rows (every copy request is a whole cache line), 16-byte
// chunk c of row r stored at chunk c ^ ((r >> 1) & 7): conflict-free for ds_read_b128 with 64 banks.
template <int ROWS> struct TileKC64 {
    static constexpr int LOADS = ROWS * 128 / 4096; // wave-wide copies per thread per stage
    static constexpr int BYTES = ROWS * 128;
    TG_DEVICE static int64_t step(int) { return 64; } // elements from one stage to the next
    TG_DEVICE static int64_t origin(int row0, int k0, int ld) { return int64_t(row0) * ld + k0; }
    TG_DEVICE static int64_t source_offset(int j, int tid, int ld) {
        const int wave = tid >> 6, lane = tid & 63;
        const int row = (j * 4 + wave) * 8 + (lane >> 3), phys = lane & 7;
        const int chunk = phys ^ ((row >> 1) & 7);
        return int64_t(row) * ld + chunk * 8;
    }
    TG_DEVICE static uint32_t lds_offset(int j, int tid) { return uint32_t((j * 4 + (tid >> 6)) * 1024); }
    // fragment for rows row0 + lane%32, 16-k step ks of the stage (0..3): k = ks*16 + 8*(lane/32) .. +7
    TG_DEVICE static bf16x8 frag(const unsigned char *tile, int row0, int ks, int lane) {
        const int row = row0 + (lane & 31), chunk = (ks * 2 + (lane >> 5)) ^ ((row >> 1) & 7);
        return *reinterpret_cast<const bf16x8 *>(tile + row * 128 + chunk * 16);
    }
    // fragment of a 16-row tile for the 32-k step ks (0..1): rows row0 + lane%16, k = ks*32 + 8*(lane/16) .. +7
    TG_DEVICE static bf16x8 frag16(const unsigned char *tile, int row0, int ks, int lane) {
        const int row = row0 + (lane & 15), chunk = (ks * 4 + (lane >> 4)) ^ ((row >> 1) & 7);
        return *reinterpret_cast<const bf16x8 *>(tile + row * 128 + chunk * 16);
    }
};
// k-strided tile: 64 k-rows x ROWS columns in the natural [k][row] image, swizzled and read like TileKS
template <int ROWS> struct TileKS64 {
    static constexpr int LOADS = ROWS * 128 / 4096;
    static constexpr int BYTES = ROWS * 128;
    static constexpr int CHUNKS_PER_ROW = ROWS / 8;
    TG_DEVICE static int64_t step(int ld) { return int64_t(64) * ld; }
    TG_DEVICE static int64_t origin(int row0, int k0, int ld) { return int64_t(k0) * ld + row0; }
    TG_DEVICE static int64_t source_offset(int j, int tid, int ld) {
        const int wave = tid >> 6, lane = tid & 63;
        const int q = (j * 4 + wave) * 64 + lane, r = q / CHUNKS_PER_ROW, p = q - r * CHUNKS_PER_ROW;
        const int chunk = p ^ TileKS<ROWS>::swizzle(r);
        return int64_t(r) * ld + chunk * 8;
    }
    TG_DEVICE static uint32_t lds_offset(int j, int tid) { return uint32_t((j * 4 + (tid >> 6)) * 1024); }
    TG_DEVICE static bf16x8 frag(const unsigned char *tile, int row0, int ks, int lane) {
        return TileKS<ROWS>::frag(tile, row0, ks, lane); // k-rows ks*16 .. of the 64
    }
    TG_DEVICE static bf16x8 frag16(const unsigned char *tile, int row0, int ks, int lane) {
        return TileKS<ROWS>::frag16(tile, row0, ks * 32, lane); // k-rows ks*32 .. of the 64
    }
};
template <int ROWS, bool KC> struct Tile64Of;
template <int ROWS> struct Tile64Of<ROWS, true> { using type = TileKC64<ROWS>; };
template <int ROWS> struct Tile64Of<ROWS, false> { using type = TileKS64<ROWS>; };

// One 64-k stage of a wave's FM x FN blocks of 32 x 32 with v_mfma_f32_16x16x32_bf16: two 32-k steps, every block as
// 2 x 2 tiles of 16 x 16.  The kernels run against the board's power limit, and on random operands this instruction
// sustains about 15 % more than the 32x32x16 form at the same power (measured from registers: 2.06 against 1.79
// PFLOP/s; it moves half the accumulator bytes per flop).  Copy n of the next stage goes out behind matrix
// instruction 2n (see gemm64_kernel).
template <class TA, class TB, int FM, int FN, int LOADS, class Copy>
TG_DEVICE void multiply_stage(f32x4 (&acc)[FM][FN][2][2], const unsigned char *slot, int wm, int wn, int lane,
                                bool copy, Copy &&copy_one) {
    // A column = one 16-row B fragment against the 2 FM A fragments of its 32-k step.  The A fragments of both steps
    // are held (the second step's are read during the first), B fragments are read one column ahead.
    constexpr int AF = 2 * FM, BF = 2 * FN, COLUMNS = 2 * BF;
    static_assert(BF >= AF, "the second step's A fragments are read while the first step's B columns are walked");
    const unsigned char *sa = slot, *sb = sa + TA::BYTES;
    bf16x8 af[2][AF], bfr[2];
#pragma unroll
    for (int i = 0; i < AF; ++i)
        af[0][i] = TA::frag16(sa, wm + i * 16, 0, lane);
    bfr[0] = TB::frag16(sb, wn, 0, lane);
#pragma unroll
    for (int column = 0; column < COLUMNS; ++column) {
        const int ks = column / BF, j = column % BF;
        if (column + 1 < COLUMNS)
            bfr[(column + 1) & 1] = TB::frag16(sb, wn + ((column + 1) % BF) * 16, (column + 1) / BF, lane);
        if (ks == 0 && j < AF)
            af[1][j] = TA::frag16(sa, wm + j * 16, 1, lane);
#pragma unroll
        for (int i = 0; i < AF; ++i) {
            f32x4 &t = acc[i >> 1][j >> 1][i & 1][j & 1];
            t = __builtin_amdgcn_mfma_f32_16x16x32_bf16(bfr[column & 1], af[ks][i], t, 0, 0, 0);
            const int q = column * AF + i; // instruction number within the stage
            if ((q & 1) == 0 && q / 2 < LOADS) {
                __builtin_amdgcn_sched_barrier(0);
                if (copy)
                    copy_one(q / 2);
                __builtin_amdgcn_sched_barrier(0);
            }
        }
    }
}

// The same product as gemm_kernel with two 64-k stages of (BM + BN) * 128 bytes: per stage one wait, one barrier,
// and the copies of the next stage issued one behind each of the first MFMAs.  A copy instruction that finds the
// vector-memory queue full stalls its wave, and with it the wave's MFMAs; kept apart, the copies overlap them.
// With only two stages a copy has what is left of the stage to land, so they go out as early as that allows
// (measured on the training step: one behind every second MFMA +3 %, all ten behind the first MFMA +1.5 %).  k-contiguous operands are
// copied in whole 128-byte lines and read with ds_read_b128.  The epilogue's transposition buffers lie in the
// stage consumed last; the stage being filled is the other one.  The reduced dimension is a multiple of 64.
template <int BM, int BN, bool AKC, bool BKC, class Epilogue>
__global__ __launch_bounds__(256, 2) void gemm64_kernel(const bf16_t *__restrict__ A, int lda,
                                                      const bf16_t *__restrict__ B, int ldb, int k_chunks,
                                                      int splits, int tiles_n, int tiles_total, int xcd_cols,
                                                      Epilogue epilogue) {
    using TA = typename Tile64Of<BM, AKC>::type;
    using TB = typename Tile64Of<BN, BKC>::type;
    constexpr int WM = BM / 2, WN = BN / 2, FM = WM / 32, FN = WN / 32;
    constexpr int LA = TA::LOADS, LB = TB::LOADS, LOADS = LA + LB;
    constexpr int SLOT = TA::BYTES + TB::BYTES;
    static_assert(LOADS <= FM * FN * 4, "copies are paired with the MFMAs of one stage");
    static_assert(4 * (Epilogue::BF16 ? 2048 : 4096) <= SLOT, "the epilogue buffers fit one stage");
    extern __shared__ __align__(16) unsigned char smem[];
    const uint32_t smem_base = lds_address(smem);

    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int wm = (wave >> 1) * WM, wn = (wave & 1) * WN;
    const int items = tiles_total * splits, stride = gridDim.x;

    // Same placement as gemm_kernel: item i belongs to XCD i % 8 and is that XCD's (i / 8)-th item; without
    // split-K the tile grid is cut into (8 / xcd_cols) x xcd_cols rectangles, one per XCD.
    auto locate = [&](int item, int &m0, int &n0, int &c0, int &nc) {
        int split = 0, tile_m, tile_n;
        if ((items & 7) == 0 && xcd_cols > 1) {
            const int xcd = item & 7, index = item >> 3;
            const int cols = tiles_n / xcd_cols, rows = (tiles_total / tiles_n) / (8 / xcd_cols);
            tile_m = (xcd / xcd_cols) * rows + index / cols;
            tile_n = (xcd % xcd_cols) * cols + index % cols;
        } else {
            int logical = item;
            if ((items & 7) == 0)
                logical = (item & 7) * (items >> 3) + (item >> 3);
            split = logical / tiles_total;
            const int tile = logical - split * tiles_total;
            tile_m = tile / tiles_n;
            tile_n = tile % tiles_n;
        }
        m0 = tile_m * BM;
        n0 = tile_n * BN;
        c0 = split * k_chunks / splits;
        nc = (split + 1) * k_chunks / splits - c0;
        return split;
    };

    // ---- producer: the stage after the one being consumed ------------------------------------------
    int p_item = blockIdx.x, p_left = 0, p_slot = 0;
    const bf16_t *pa[LA], *pb[LB];
    const int64_t a_step = TA::step(lda), b_step = TB::step(ldb);
    auto producer_open = [&]() {
        int m0, n0, c0, nc;
        locate(p_item, m0, n0, c0, nc);
        p_left = nc;
        const bf16_t *a0 = A + TA::origin(m0, c0 * 64, lda), *b0 = B + TB::origin(n0, c0 * 64, ldb);
#pragma unroll
        for (int j = 0; j < LA; ++j)
            pa[j] = a0 + TA::source_offset(j, tid, lda);
#pragma unroll
        for (int j = 0; j < LB; ++j)
            pb[j] = b0 + TB::source_offset(j, tid, ldb);
    };
    auto copy_one = [&](int n) { // n-th of the LOADS copies of a stage, into slot p_slot
        const uint32_t to = smem_base + uint32_t(p_slot) * SLOT;
        if (n < LA) {
            async_copy16(__builtin_amdgcn_readfirstlane(to + TA::lds_offset(n, tid)), pa[n]);
            pa[n] += a_step;
        } else {
            async_copy16(__builtin_amdgcn_readfirstlane(to + TA::BYTES + TB::lds_offset(n - LA, tid)), pb[n - LA]);
            pb[n - LA] += b_step;
        }
    };
    if (p_item >= items)
        return;
    producer_open();
#pragma unroll
    for (int n = 0; n < LOADS; ++n)
        copy_one(n);
    --p_left;
    p_slot = 1;

    int c_slot = 0;
    for (int item = blockIdx.x; item < items; item += stride) {
        int m0, n0, c0, nc;
        const int split = locate(item, m0, n0, c0, nc);
        f32x4 acc[FM][FN][2][2]; // 32 x 32 blocks as 2 x 2 tiles of 16 x 16
#pragma unroll
        for (int i = 0; i < FM; ++i)
#pragma unroll
            for (int j = 0; j < FN; ++j)
#pragma unroll
                for (int t = 0; t < 4; ++t)
                    acc[i][j][t >> 1][t & 1] = f32x4{0.f, 0.f, 0.f, 0.f};
        u32x4 aux[2] = {u32x4{0, 0, 0, 0}, u32x4{0, 0, 0, 0}}; // the epilogue's second input for tile (0, 0)
        for (int c = 0; c < nc; ++c) {
            wait_vmcnt<0>(); // this wave's copies of stage c (and the previous tile's stores) are done
            __syncthreads(); // everyone's are, and everyone is done reading the other slot
            if constexpr (Epilogue::BF16)
                if (c == nc - 1 && epilogue.wants_aux())
                    load_aux_pair<FM, FN>(epilogue, 0, m0 + wm, n0 + wn, lane, aux); // lands during the last stage
            bool copy = true;
            if (p_left == 0) {
                p_item += stride;
                copy = p_item < items;
                if (copy)
                    producer_open();
            }
            multiply_stage<TA, TB, FM, FN, LOADS>(acc, smem + c_slot * SLOT, wm, wn, lane, copy, copy_one);
            if (copy) {
                --p_left;
                p_slot ^= 1;
            }
            c_slot ^= 1;
        }
        // The transposition buffers lie in the stage consumed last (c_slot ^ 1 now); other waves may still be
        // reading fragments there.
        __syncthreads();
        unsigned char *slot = smem + (c_slot ^ 1) * SLOT;
        if constexpr (Epilogue::BF16)
            staged_store_bf16<FM, FN>(acc, aux, slot + wave * 2048, epilogue, m0 + wm, n0 + wn, lane);
        else
            staged_store_f32<FM, FN>(acc, slot + wave * 4096, epilogue, m0 + wm, n0 + wn, lane, split);
    }
    wait_vmcnt<0>();
}

TG_DEVICE uint32_t kc64_frag16_offset(int row0, int ks, int lane) { // TileKC64::frag16's address
    const int row = row0 + (lane & 15), chunk = (ks * 4 + (lane >> 4)) ^ ((row >> 1) & 7);
    return uint32_t(row * 128 + chunk * 16);
}
// ---- 256-row tiles, one wave per SIMD: forward and input-gradient products with a long or plain epilogue -------------
// C = A B^T with both operands k-contiguous, a 256 x BN tile per block, four waves of 128 x BN/2 outputs each, one
// block per compute unit.  What bounds these products is a compute unit's copy path: bytes per flop, whole
// cache lines per request, and how many requests it keeps in flight.  Hence: 9.1 bytes per kFLOP at BN = 192 without
// relying on another block's lines in L1; 64 k per stage (every request a whole 128-byte line); and rings of different
// depth for the two operands - RA slots for A (activations, streamed from beyond the L2: a copy has two stages to
// land) and two for B (the weights, mostly L2 hits: one stage).  With a lone wave per SIMD the fragments of the
// next 32-k step are read into a second register set between the matrix instructions of the current one:
//   first half of stage g : matrix instructions on (g, k 0..31), fragment reads of (g, k 32..63)
//   wait (all but A's youngest stage), barrier: stage g + 1 is visible, nobody reads stage g's slots any more
//   second half           : matrix instructions on (g, k 32..63), copies of B's stage g + 2 and A's stage g + RA,
//                           fragment reads of (g + 1, k 0..31)
// The loop is unrolled over the rings' common period P, so that every LDS address is a constant, and the reduced
// dimension is a multiple of 64 P.  Two instantiations:
//   BN = 192, RA = 3 (P = 6, 144 KB of rings + 8 KB for the epilogue): widths that 192 and 384 divide;
//   BN = 128, RA = 4 (P = 4, 160 KB of rings: all of the LDS): widths that 128 and 256 divide (d_model 1024).  Three
//   slots would do for A as far as latency goes - the fourth only makes the period a power of two.  The epilogue's
//   buffers then lie in the first 8 KB of the A slot that the tile's last stage leaves, and the two copies per wave that
//   refill those rows are held back until the wave's epilogue is over (each wave then copies the rows under its own
//   buffer, so no barrier is needed; in their place copies 2 and 3 of the stage go out twice, which keeps the loop
//   free of branches and every wait count fixed).
template <int BN, int RA, class Epilogue>
__global__ __launch_bounds__(256, 1) void gemm256_kernel(const bf16_t *__restrict__ A, int lda,
                                                       const bf16_t *__restrict__ B, int ldb, int k_periods,
                                                       int tiles_n, int tiles_total, int xcd_cols,
                                                       Epilogue epilogue) {
    constexpr int BM = 256;
    constexpr int P = RA % 2 ? 2 * RA : RA; // stages per period of the two rings (RA slots for A, two for B)
    constexpr int WM = BM / 2, WN = BN / 2, FM = WM / 32, FN = WN / 32, AF = 2 * FM, BF = 2 * FN, MFMAS = AF * BF;
    constexpr int A_BYTES = BM * 128, B_BYTES = BN * 128, B_RING = RA * A_BYTES, BUFFERS = B_RING + 2 * B_BYTES;
    // Where the rings fill the LDS, the epilogue's four transposition buffers (8 KB) lie in the first rows of the A slot
    // that a tile's last stage leaves, and the two copies per wave that would refill those rows wait for the epilogue.
    constexpr bool ALIAS = BUFFERS + 4 * 2048 > 160 * 1024;
    static_assert(!ALIAS || (P == RA && BUFFERS <= 160 * 1024), "the aliased buffers assume the last stage's slot is the ring's last");
    constexpr int LA = BM * 128 / 4096, LB = BN * 128 / 4096, LOADS = LA + LB; // copies per wave and stage
    constexpr int READ_EVERY = MFMAS / (AF + BF), COPY_EVERY = MFMAS / LOADS;
    extern __shared__ __align__(16) unsigned char smem[];
    const uint32_t smem_base = lds_address(smem);
    const int tid = threadIdx.x, lane = tid & 63, wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int wm = (wave >> 1) * WM, wn = (wave & 1) * WN;
    const int stride = gridDim.x;

    auto locate = [&](int item, int &m0, int &n0) {
        int tile_m, tile_n;
        if ((tiles_total & 7) == 0 && xcd_cols > 1) {
            const int xcd = item & 7, index = item >> 3;
            const int cols = tiles_n / xcd_cols, rows = (tiles_total / tiles_n) / (8 / xcd_cols);
            tile_m = (xcd / xcd_cols) * rows + index / cols;
            tile_n = (xcd % xcd_cols) * cols + index % cols;
        } else {
            const int logical = (tiles_total & 7) == 0 ? (item & 7) * (tiles_total >> 3) + (item >> 3) : item;
            tile_m = logical / tiles_n;
            tile_n = logical % tiles_n;
        }
        m0 = tile_m * BM;
        n0 = tile_n * BN;
    };

    // ---- producers: A three stages ahead of the consumer, B two --------------------------------------------------
    const int copy_row = lane >> 3, copy_chunk = (lane & 7) ^ ((((wave & 1) * 4) + (lane >> 4)) & 7);
    const uint32_t la = uint32_t(copy_row * lda + copy_chunk * 8) * 2, lb = uint32_t(copy_row * ldb + copy_chunk * 8) * 2;
    const int64_t a_rows32 = int64_t(32) * lda * 2, b_rows32 = int64_t(32) * ldb * 2;
    // wave-uniform: the stage either producer copies next (this wave's first row of it), the first stage of the tile
    // after the current one, and the bytes from one stage to the next (0 once the list is exhausted: the copies go
    // on, re-reading a stage into slots nobody consumes, and the loop stays straight-line code)
    const char *pa_at = nullptr, *pb_at = nullptr, *a_next = nullptr, *b_next = nullptr;
    int64_t pa_step = 128, pb_step = 128, next_step = 128;
    auto tile_origin = [&](int item, const char *&a, const char *&b) {
        int m0, n0;
        locate(item, m0, n0);
        a = reinterpret_cast<const char *>(A + int64_t(m0 + wave * 8) * lda);
        b = reinterpret_cast<const char *>(B + int64_t(n0 + wave * 8) * ldb);
    };
    auto prepare_next = [&](int item) { // keeps the current origins when there is no further tile
        if (item < tiles_total)
            tile_origin(item, a_next, b_next);
        else
            next_step = 0;
    };
    auto copy_a = [&](int n, int slot) __attribute__((always_inline)) {
        async_copy16(smem_base + uint32_t(slot * A_BYTES + (n * 4 + wave) * 1024), pa_at + n * a_rows32, la);
    };
    auto copy_b = [&](int n, int slot) __attribute__((always_inline)) {
        async_copy16(smem_base + uint32_t(B_RING + slot * B_BYTES + (n * 4 + wave) * 1024), pb_at + n * b_rows32, lb);
    };
    if (int(blockIdx.x) >= tiles_total)
        return;
    tile_origin(blockIdx.x, pa_at, pb_at);
    a_next = pa_at, b_next = pb_at;
    prepare_next(blockIdx.x + stride);
    // stages 0 and 1 of both, then A's further stages (so that A's youngest stages are the last ones issued, as in the loop)
#pragma unroll
    for (int s = 0; s < 2; ++s) {
#pragma unroll
        for (int n = 0; n < LB; ++n)
            copy_b(n, s);
#pragma unroll
        for (int n = 0; n < LA; ++n)
            copy_a(n, s);
        pa_at += pa_step, pb_at += pb_step;
    }
#pragma unroll
    for (int s = 2; s < RA; ++s) {
#pragma unroll
        for (int n = 0; n < LA; ++n)
            copy_a(n, s);
        pa_at += pa_step;
    }

    // ---- consumer ----------------------------------------------------------------------------------------------------
    uint32_t fa_at[2], fa_far[2], fb_at[2]; // fragment 0 of either 32-k step; fragment i lies 2048 i bytes further on
#pragma unroll
    for (int ks = 0; ks < 2; ++ks) {
        fa_at[ks] = kc64_frag16_offset(wm, ks, lane);
        fa_far[ks] = fa_at[ks] + 2 * A_BYTES; // slot 2 lies beyond a ds_read's 16-bit offset
        fb_at[ks] = B_RING + kc64_frag16_offset(wn, ks, lane);
    }
    auto read_fragment = [&](bf16x8 (&fa)[AF], bf16x8 (&fb)[BF], int slot_a, int slot_b, int ks, int f)
                             __attribute__((always_inline)) {
        if (f < AF)
            fa[f] = slot_a >= 2 ? *reinterpret_cast<const bf16x8 *>(smem + fa_far[ks] + (slot_a - 2) * A_BYTES + f * 2048)
                                : *reinterpret_cast<const bf16x8 *>(smem + fa_at[ks] + slot_a * A_BYTES + f * 2048);
        else
            fb[f - AF] = *reinterpret_cast<const bf16x8 *>(smem + fb_at[ks] + slot_b * B_BYTES + (f - AF) * 2048);
    };
    f32x4 acc[FM][FN][2][2];
    bool last_period = k_periods == 1; // the consumer is in a tile's last period of stages
    bool behind_epilogue = false;
    static_assert(LA + FM * FN * Epilogue::MEMORY_OPS_PER_BLOCK + (ALIAS ? 2 : 0) < 64, "the wait count has six bits");
    // One 32-k step on `cur`; meanwhile the fragments of (next slots, next_ks) are read into `next`, and, in a
    // stage's second half, the copies go out: B first, A behind it (so that a wait can leave A's youngest stage out).
    auto half = [&](auto copy_tag, int next_a_slot, int next_b_slot, int next_ks, int copy_a_slot, int copy_b_slot,
                    bool hold_back, const bf16x8 (&cur_a)[AF], const bf16x8 (&cur_b)[BF], bf16x8 (&next_a)[AF],
                    bf16x8 (&next_b)[BF]) __attribute__((always_inline)) {
        constexpr bool COPY = decltype(copy_tag)::value;
#pragma unroll
        for (int j = 0; j < BF; ++j)
#pragma unroll
            for (int i = 0; i < AF; ++i) {
                // accumulators pinned to the accumulation registers (see wgrad_list_kernel)
                asm volatile("v_mfma_f32_16x16x32_bf16 %0, %1, %2, %0"
                             : "+a"(acc[i >> 1][j >> 1][i & 1][j & 1])
                             : "v"(cur_b[j]), "v"(cur_a[i]));
                const int q = j * AF + i;
                if (q % READ_EVERY == 0 && q / READ_EVERY < AF + BF)
                    read_fragment(next_a, next_b, next_a_slot, next_b_slot, next_ks, q / READ_EVERY);
                if (COPY && q % COPY_EVERY == 1 % COPY_EVERY && q / COPY_EVERY < LOADS) {
                    const int n = q / COPY_EVERY;
                    if (n < LB)
                        copy_b(n, copy_b_slot);
                    else if (ALIAS && n - LB < 2) // held back: the rows under the epilogue's buffers; copy 2 or 3 goes twice instead
                        copy_a(hold_back ? n - LB + 2 : n - LB, copy_a_slot);
                    else
                        copy_a(n - LB, copy_a_slot);
                }
                __builtin_amdgcn_sched_barrier(0);
            }
    };
    // stage g = STAGE (mod P): A slot g % RA, B slot g % 2
    auto stage = [&](auto stage_tag, bf16x8 (&fa0)[AF], bf16x8 (&fb0)[BF], bf16x8 (&fa1)[AF], bf16x8 (&fb1)[BF])
                     __attribute__((always_inline)) {
        constexpr int G = decltype(stage_tag)::value, SA = G % RA, SB = G % 2;
        // In a tile's last period the producers cross into the next tile: A with the copies of stage P - RA (RA
        // stages ahead), B with those of stage P - 2.  Selects, not branches.
        if (G == P - RA && last_period)
            pa_at = a_next, pa_step = next_step;
        if (G == P - 2 && last_period)
            pb_at = b_next, pb_step = next_step;
        half(std::false_type{}, SA, SB, 1, 0, 0, false, fa0, fb0, fa1, fb1);
        // Everything but A's youngest stage has landed.  A wave's loads and stores retire in order through one counter;
        // behind a tile's epilogue its loads and stores are the youngest operations, and their number is known.
        if (G == 0 && behind_epilogue)
            wait_vmcnt<LA + FM * FN * Epilogue::MEMORY_OPS_PER_BLOCK + (ALIAS ? 2 : 0)>();
        else
            wait_vmcnt<LA>();
        if (G == 0)
            behind_epilogue = false;
        __builtin_amdgcn_s_waitcnt(0xc07f); // lgkmcnt(0): and this wave's reads of this stage are done
        __builtin_amdgcn_s_barrier();
        __builtin_amdgcn_sched_barrier(0);
        // copies: B's stage g + 2 into B slot g % 2, A's stage g + 3 into A slot g % 3 (the slots this stage leaves)
        half(std::true_type{}, (SA + 1) % RA, SB ^ 1, 0, SA, SB, ALIAS && G == P - 1 && last_period, fa1, fb1, fa0, fb0);
        pa_at += pa_step, pb_at += pb_step;
    };
    const bf16x8 zeros = {0, 0, 0, 0, 0, 0, 0, 0};
    auto clear = [&]() __attribute__((always_inline)) {
#pragma unroll
        for (int i = 0; i < FM; ++i)
#pragma unroll
            for (int j = 0; j < FN; ++j)
#pragma unroll
                for (int t = 0; t < 4; ++t)
                    asm volatile("s_nop 4\n\tv_mfma_f32_16x16x32_bf16 %0, %1, %1, 0"
                                 : "+a"(acc[i][j][t >> 1][t & 1])
                                 : "v"(zeros)); // zeroed in place, wait states included (see wgrad_list_kernel)
    };
    bf16x8 fa0[AF], fb0[BF], fa1[AF], fb1[BF];
    wait_vmcnt<(RA - 1) * LA + LB>(); // stage 0
    __builtin_amdgcn_s_barrier();
#pragma unroll
    for (int f = 0; f < AF + BF; ++f)
        read_fragment(fa0, fb0, 0, 0, 0, f);
    unsigned char *mine = smem + (ALIAS ? (RA - 1) * A_BYTES : BUFFERS) + wave * 2048;
    int item = blockIdx.x, periods_left = k_periods;
    clear();
    for (;;) {
        stage(std::integral_constant<int, 0>{}, fa0, fb0, fa1, fb1);
        stage(std::integral_constant<int, 1>{}, fa0, fb0, fa1, fb1);
        stage(std::integral_constant<int, 2>{}, fa0, fb0, fa1, fb1);
        stage(std::integral_constant<int, 3>{}, fa0, fb0, fa1, fb1);
        if constexpr (P == 6) {
            stage(std::integral_constant<int, 4>{}, fa0, fb0, fa1, fb1);
            stage(std::integral_constant<int, 5>{}, fa0, fb0, fa1, fb1);
        }
        if (--periods_left) {
            last_period = periods_left == 1;
            continue;
        }
        asm volatile("s_nop 7\n\ts_nop 7\n\ts_nop 7"); // the compiler does not know that matrix instructions wrote the accumulators
        int m0, n0;
        locate(item, m0, n0);
        u32x4 aux[2] = {u32x4{0, 0, 0, 0}, u32x4{0, 0, 0, 0}};
        if (epilogue.wants_aux())
            load_aux_pair<FM, FN>(epilogue, 0, m0 + wm, n0 + wn, lane, aux);
        staged_store_bf16<FM, FN>(acc, aux, mine, epilogue, m0 + wm, n0 + wn, lane);
        behind_epilogue = true; // the stores stay in flight under the next tile's first stage
        if (ALIAS) {
            // the two copies held back in the last stage, as the rows that lie under this wave's own buffer (rows 16 w
            // to 16 w + 15 of the stage: nobody else's buffer is touched, so no barrier); the producer has moved on
            // by one stage since
            __builtin_amdgcn_s_waitcnt(0xc07f); // this wave's reads of its buffer have returned
#pragma unroll
            for (int n = 0; n < 2; ++n) { // 1 KB piece 2 w + n of the stage: its rows' swizzle term goes by n, not by w
                const int chunk = (lane & 7) ^ ((n * 4 + (lane >> 4)) & 7);
                async_copy16(smem_base + uint32_t((RA - 1) * A_BYTES + (2 * wave + n) * 1024),
                             pa_at - pa_step + int64_t(wave + n) * 8 * lda * 2, uint32_t(copy_row * lda + chunk * 8) * 2);
            }
        }
        item += stride;
        if (item >= tiles_total)
            break;
        prepare_next(item + stride);
        periods_left = k_periods;
        last_period = k_periods == 1;
        clear();
    }
    wait_vmcnt<0>();
}

// ---- several weight gradients in one launch ------------------------------------------------------
// dW_j[N_j][K_j] = dY_j^T X_j for up to four (dY, X) pairs that share the reduced dimension (the tokens).  One
// matrix rarely has as many 128x192 tiles as the GPU holds blocks, and split into as many token ranges as fill
// it, it writes that many fp32 partial sums per tile.  Here the tiles of all jobs form one list, cut in two
// groups: the first `tiles_a` tiles are split `splits_a` ways and the rest `splits_b` ways, chosen so that
// each group makes one work item per resident block and every block gets one long and one short item of the
// same total length (four gradients of a d = 768 block: 256 tiles x 2 + 32 tiles x 16 on 512 blocks, 144
// chunks of 64 tokens each, 98 MB of partial sums instead of 193 MB, one prologue and one tail instead of
// four).  Within a group the blocks of an XCD work on the same token range of neighbouring tiles, so the rows
// of dY^T and X they share are read from HBM once per XCD.  wgrad_batch_fold_kernel sums a tile's pieces in
// split order (fixed, bit-reproducible); a tile that is not split writes the gradient itself.
constexpr int MAX_WGRAD_JOBS = 4;
struct WgradBatch {
    const bf16_t *dy[MAX_WGRAD_JOBS], *x[MAX_WGRAD_JOBS];
    float *dw[MAX_WGRAD_JOBS];
    int lddy[MAX_WGRAD_JOBS], ldx[MAX_WGRAD_JOBS], lddw[MAX_WGRAD_JOBS];
    int tiles_n[MAX_WGRAD_JOBS];
    int first_tile[MAX_WGRAD_JOBS + 1]; // tiles before job j; [count] = all tiles
    int count;
    int k_chunks;            // tokens / 64
    int tiles_a, splits_a;   // group a: tiles [0, tiles_a)
    int tiles_b, splits_b;   // group b: the rest
    int accumulate;
    float *pieces; // BM * BN floats per (tile, split), tile-local row-major, see piece_slot()
};
struct WgradTile {
    int job, m0, n0;
};
struct WgradItem {
    int tile, split, splits, c0, nc;
};
template <int BM, int BN> TG_DEVICE WgradTile wgrad_tile(const WgradBatch &w, int tile) {
    int job = 0;
#pragma unroll
    for (int j = 1; j < MAX_WGRAD_JOBS; ++j)
        if (j < w.count && tile >= w.first_tile[j])
            job = j;
    const int local = tile - w.first_tile[job];
    return {job, (local / w.tiles_n[job]) * BM, (local % w.tiles_n[job]) * BN};
}
TG_DEVICE int piece_slot(const WgradBatch &w, int tile, int split) {
    return (tile < w.tiles_a ? tile * w.splits_a : w.tiles_a * w.splits_a + (tile - w.tiles_a) * w.splits_b) + split;
}
// The block's item of group `group` (0: a, 1: b); false when the group has no item for it.  Consecutive block
// ids sit on consecutive XCDs; an XCD owns a contiguous range of (split, tile), split-major.
TG_DEVICE bool wgrad_item(const WgradBatch &w, int group, int block, WgradItem &item) {
    const int tiles = group ? w.tiles_b : w.tiles_a, splits = group ? w.splits_b : w.splits_a;
    const int n = tiles * splits;
    if (block >= n)
        return false;
    const int logical = (n & 7) == 0 ? (block & 7) * (n >> 3) + (block >> 3) : block;
    item.split = logical / tiles;
    item.tile = (group ? w.tiles_a : 0) + logical - item.split * tiles;
    item.splits = splits;
    item.c0 = item.split * w.k_chunks / splits;
    item.nc = (item.split + 1) * w.k_chunks / splits - item.c0;
    return true;
}
template <int BM, int BN>
__global__ __launch_bounds__(256, 2) void wgrad_batch_kernel(WgradBatch w) {
    using TA = TileKS64<BM>;
    using TB = TileKS64<BN>;
    constexpr int WM = BM / 2, WN = BN / 2, FM = WM / 32, FN = WN / 32;
    constexpr int LA = TA::LOADS, LB = TB::LOADS, LOADS = LA + LB;
    constexpr int SLOT = TA::BYTES + TB::BYTES;
    extern __shared__ __align__(16) unsigned char smem[];
    const uint32_t smem_base = lds_address(smem);
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int wm = (wave >> 1) * WM, wn = (wave & 1) * WN;

    // ---- producer: one stage ahead of the consumer, across the block's (at most two) items --------------
    int p_group = 0, p_left = 0, p_slot = 0;
    const bf16_t *pa[LA], *pb[LB];
    int64_t a_step = 0, b_step = 0;
    auto producer_open = [&]() { // the next group that has an item for this block; false when there is none
        WgradItem item;
        while (p_group < 2 && !wgrad_item(w, p_group, blockIdx.x, item))
            ++p_group;
        if (p_group >= 2)
            return false;
        ++p_group;
        p_left = item.nc;
        const WgradTile t = wgrad_tile<BM, BN>(w, item.tile);
        const int lda = w.lddy[t.job], ldb = w.ldx[t.job];
        a_step = TA::step(lda), b_step = TB::step(ldb);
        const bf16_t *a0 = w.dy[t.job] + TA::origin(t.m0, item.c0 * 64, lda);
        const bf16_t *b0 = w.x[t.job] + TB::origin(t.n0, item.c0 * 64, ldb);
#pragma unroll
        for (int j = 0; j < LA; ++j)
            pa[j] = a0 + TA::source_offset(j, tid, lda);
#pragma unroll
        for (int j = 0; j < LB; ++j)
            pb[j] = b0 + TB::source_offset(j, tid, ldb);
        return true;
    };
    auto copy_one = [&](int n) {
        const uint32_t to = smem_base + uint32_t(p_slot) * SLOT;
        if (n < LA) {
            async_copy16(__builtin_amdgcn_readfirstlane(to + TA::lds_offset(n, tid)), pa[n]);
            pa[n] += a_step;
        } else {
            async_copy16(__builtin_amdgcn_readfirstlane(to + TA::BYTES + TB::lds_offset(n - LA, tid)), pb[n - LA]);
            pb[n - LA] += b_step;
        }
    };
    if (!producer_open())
        return;
#pragma unroll
    for (int n = 0; n < LOADS; ++n)
        copy_one(n);
    --p_left;
    p_slot = 1;

    int c_slot = 0;
    for (int group = 0; group < 2; ++group) {
        WgradItem item;
        if (!wgrad_item(w, group, blockIdx.x, item))
            continue;
        f32x4 acc[FM][FN][2][2];
#pragma unroll
        for (int i = 0; i < FM; ++i)
#pragma unroll
            for (int j = 0; j < FN; ++j)
#pragma unroll
                for (int t = 0; t < 4; ++t)
                    acc[i][j][t >> 1][t & 1] = f32x4{0.f, 0.f, 0.f, 0.f};
        for (int c = 0; c < item.nc; ++c) {
            wait_vmcnt<0>();
            __syncthreads();
            bool copy = true;
            if (p_left == 0)
                copy = producer_open();
            multiply_stage<TA, TB, FM, FN, LOADS>(acc, smem + c_slot * SLOT, wm, wn, lane, copy, copy_one);
            if (copy) {
                --p_left;
                p_slot ^= 1;
            }
            c_slot ^= 1;
        }
        __syncthreads(); // the transposition buffers lie in the stage consumed last
        unsigned char *mine = smem + (c_slot ^ 1) * SLOT + wave * 4096;
        if (item.splits == 1) {
            const WgradTile t = wgrad_tile<BM, BN>(w, item.tile);
            const EpilogueF32 whole{w.dw[t.job], w.lddw[t.job], 0, w.accumulate};
            staged_store_f32<FM, FN>(acc, mine, whole, t.m0 + wm, t.n0 + wn, lane, 0);
        } else {
            const EpilogueF32 piece{w.pieces + size_t(piece_slot(w, item.tile, item.split)) * (BM * BN), BN, 0, 0};
            staged_store_f32<FM, FN>(acc, mine, piece, wm, wn, lane, 0);
        }
    }
    wait_vmcnt<0>();
}
// Sums the pieces of every split tile, in split order, into the gradient.  Four blocks per tile, 32 rows each.
template <int BM, int BN>
__global__ __launch_bounds__(256) void wgrad_batch_fold_kernel(WgradBatch w) {
    const int tile = blockIdx.x >> 2, part = blockIdx.x & 3;
    const int splits = tile < w.tiles_a ? w.splits_a : w.splits_b;
    if (splits == 1)
        return; // the tile's only item wrote the gradient itself
    const WgradTile t = wgrad_tile<BM, BN>(w, tile);
    float *out = w.dw[t.job];
    const int ld = w.lddw[t.job];
    const float *first = w.pieces + size_t(piece_slot(w, tile, 0)) * (BM * BN);
    constexpr int QUADS = BN / 4, ROWS = BM / 4, PER_THREAD = ROWS * QUADS / 256;
    static_assert(ROWS * QUADS % 256 == 0, "a quarter tile is a whole number of float4 per thread");
    const auto finish = [&](int i, float4 sum) {
        const int r = part * ROWS + i / QUADS, c = (i % QUADS) * 4;
        float4 *p = reinterpret_cast<float4 *>(out + size_t(t.m0 + r) * ld + t.n0 + c);
        if (w.accumulate) {
            const float4 old = *p;
            sum.x += old.x, sum.y += old.y, sum.z += old.z, sum.w += old.w;
        }
        __builtin_nontemporal_store(f32x4{sum.x, sum.y, sum.z, sum.w}, reinterpret_cast<f32x4 *>(p));
    };
    const float *mine = first + size_t(part) * ROWS * BN + threadIdx.x * 4; // a quarter tile is contiguous
    if (splits == 2) { // most tiles: every load of the thread is requested before the first sum
        float4 a[PER_THREAD], b[PER_THREAD];
#pragma unroll
        for (int k = 0; k < PER_THREAD; ++k) {
            a[k] = *reinterpret_cast<const float4 *>(mine + k * 1024);
            b[k] = *reinterpret_cast<const float4 *>(mine + k * 1024 + BM * BN);
        }
#pragma unroll
        for (int k = 0; k < PER_THREAD; ++k)
            finish(threadIdx.x + k * 256, make_float4(a[k].x + b[k].x, a[k].y + b[k].y, a[k].z + b[k].z, a[k].w + b[k].w));
        return;
    }
#pragma unroll
    for (int k = 0; k < PER_THREAD; ++k) {
        float4 sum = make_float4(0, 0, 0, 0);
#pragma unroll 4
        for (int split = 0; split < splits; ++split) { // fixed order
            const float4 v = *reinterpret_cast<const float4 *>(mine + k * 1024 + size_t(split) * (BM * BN));
            sum.x += v.x, sum.y += v.y, sum.z += v.z, sum.w += v.w;
        }
        finish(threadIdx.x + k * 256, sum);
    }
}

// ---- every weight gradient of a step in one launch: 256-row tiles, one wave per SIMD ------------------------
// dW_j[N_j][K_j] = dY_j^T X_j for any number of (dY, X) pairs that share the reduced dimension (the tokens).  A
// training step has 4 * depth + 2 of them; taken together they have several tiles per compute unit, so almost every
// tile is reduced over all tokens by one block (no partial sums, no fold) and only the last tiles % blocks tiles are
// cut into token ranges.  The operands of all layers must exist at once: the caller keeps every layer's output
// gradients until the end of the backward pass (a few GB of the 288).
//
// One block of four waves per compute unit, a 256 x BN tile, each wave 128 x BN/2 outputs (accumulators in 256
// registers: a wave owns its SIMD's whole register file).  Per 32 k a wave then reads 16 KB of fragments for 64
// matrix instructions where the 64 x 96 wave tile of gemm64_kernel reads 10 KB for 24, and the block copies 32 KB
// per 4.2 MFLOP where two 128 x 192 blocks copy 40 KB for 3.1: less of everything that is not a matrix instruction
// per flop, which is what the power limit pays for.  With one wave per SIMD nothing else covers a wave's waits, so:
// a ring of four 32-k stages filled three stages ahead (a copy has three stages of matrix instructions to land), the
// fragments of the next stage read into a second register set between the matrix instructions of the current one
// (its data is published one stage early), one barrier per stage, and copies and fragment reads spread evenly
// between the matrix instructions.
struct WgradListJob {
    const bf16_t *dy, *x;
    float *dw;
    int lddy, ldx, lddw, pad;
};
struct WgradList {
    const WgradListJob *jobs; // device memory
    const int4 *tiles;        // device memory: {job, first row, first column, 0} per tile, in processing order
    int rounds;               // whole tiles per block
    int rem_tiles, rem_splits; // the tiles after rounds * blocks, each cut into rem_splits token ranges
    int k_quads;              // tokens / 128
    int accumulate;
    float *pieces; // rem_tiles * rem_splits partial tiles of 256 * BN floats, row major
    float *sumsq;  // optional: sums of squares of the gradients written, four per block of the product launch (one per
                   // wave) followed by one per block of the fold launch
};
struct WgradListItem {
    int tile, q0, nq, piece; // piece < 0: the block reduces over all tokens and writes the gradient itself
};
// The i-th work item of this block.  Consecutive block ids sit on consecutive XCDs; an XCD takes 1/8 of the blocks'
// consecutive tiles in every round, which are neighbours in one job's tile grid and walk the tokens together, so the
// operand panels they share are read into that XCD's L2 once.
TG_DEVICE bool wgrad_list_item(const WgradList &w, int i, WgradListItem &item) {
    const int blocks = gridDim.x, b = blockIdx.x;
    const int logical = (blocks & 7) == 0 ? (b & 7) * (blocks >> 3) + (b >> 3) : b;
    if (i < w.rounds) {
        item = {i * blocks + logical, 0, w.k_quads, -1};
        return true;
    }
    if (i > w.rounds || logical >= w.rem_tiles * w.rem_splits)
        return false;
    const int split = logical / w.rem_tiles, r = logical - split * w.rem_tiles;
    item.tile = w.rounds * blocks + r;
    item.q0 = int(int64_t(split) * w.k_quads / w.rem_splits);
    item.nq = int(int64_t(split + 1) * w.k_quads / w.rem_splits) - item.q0;
    item.piece = w.rem_splits > 1 ? r * w.rem_splits + split : -1;
    return true;
}
TG_DEVICE const char *uniform_pointer(const void *p) {
    const uint64_t v = reinterpret_cast<uint64_t>(p);
    const uint32_t lo = __builtin_amdgcn_readfirstlane(uint32_t(v)), hi = __builtin_amdgcn_readfirstlane(uint32_t(v >> 32));
    return reinterpret_cast<const char *>(uint64_t(hi) << 32 | lo);
}
template <int ROWS> TG_DEVICE uint32_t ks_frag16_offset(int row0, int lane) { // TileKS<ROWS>::frag16's first address, k0 = 0
    const int g = lane >> 4, i = lane & 15;
    const int r = 8 * g + (i >> 2), col = row0 + 4 * (i & 3);
    return uint32_t(r * (ROWS * 2) + (i & 1) * 8 + (((col >> 3) ^ TileKS<ROWS>::swizzle(r)) << 4));
}
template <int ROWS> TG_DEVICE bf16x8 ks_frag16_at(const unsigned char *p) { // k-rows r and r + 4 share a swizzle term
    const s16x4 lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_s16x4 *)(p));
    const s16x4 hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_s16x4 *)(p + 4 * ROWS * 2));
    const s16x8 both = __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7);
    return __builtin_bit_cast(bf16x8, both);
}
template <int BN>
__global__ __launch_bounds__(256, 1) void wgrad_list_kernel(const WgradList w) {
    constexpr int BM = 256, S = 4;
    using TA = TileKS<BM>;
    using TB = TileKS<BN>;
    constexpr int WM = BM / 2, WN = BN / 2, FM = WM / 32, FN = WN / 32, AF = 2 * FM, BF = 2 * FN, MFMAS = AF * BF;
    constexpr int LA = TA::LOADS, LB = TB::LOADS, LOADS = LA + LB;
    constexpr int A_RING = S * TA::BYTES;
    // a fragment read behind every third matrix instruction, a copy behind every eighth (measured: the best of five
    // placements, by 4 %)
    constexpr int READ_EVERY = 3, COPY_EVERY = MFMAS / LOADS, COPY_FIRST = 1;
    extern __shared__ __align__(16) unsigned char smem[];
    const uint32_t smem_base = lds_address(smem);
    const int tid = threadIdx.x, lane = tid & 63, wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int wm = (wave >> 1) * WM, wn = (wave & 1) * WN;

    // ---- producer: one quad (four stages) ahead of the consumer, across item boundaries -----------------------
    int p_index = 0, p_left = 0;
    const char *p_a = nullptr, *p_b = nullptr; // wave-uniform: the operands' first k-row of the stage to copy next
    int64_t a_step = 0, b_step = 0;
    uint32_t la[LA], lb[LB]; // this lane's byte offset inside a stage, per copy
    auto producer_open = [&]() {
        WgradListItem item;
        if (!wgrad_list_item(w, p_index, item)) {
            // Out of work: the copies go on (the loop below is straight-line code), re-reading the last stage into
            // slots nobody consumes.
            p_a -= a_step, p_b -= b_step;
            a_step = b_step = 0;
            p_left = 1 << 30;
            return;
        }
        ++p_index;
        const int4 t = w.tiles[item.tile];
        const WgradListJob job = w.jobs[t.x];
        // the tables are read with vector loads: tell the compiler that the values are the same in every lane
        const int lddy = __builtin_amdgcn_readfirstlane(job.lddy), ldx = __builtin_amdgcn_readfirstlane(job.ldx);
        p_left = __builtin_amdgcn_readfirstlane(item.nq * 4);
        p_a = uniform_pointer(job.dy + int64_t(item.q0) * 128 * job.lddy + t.y);
        p_b = uniform_pointer(job.x + int64_t(item.q0) * 128 * job.ldx + t.z);
        a_step = int64_t(BK) * lddy * 2, b_step = int64_t(BK) * ldx * 2;
#pragma unroll
        for (int j = 0; j < LA; ++j)
            la[j] = uint32_t(TA::source_offset(j, tid, job.lddy) * 2);
#pragma unroll
        for (int j = 0; j < LB; ++j)
            lb[j] = uint32_t(TB::source_offset(j, tid, job.ldx) * 2);
    };
    auto copy_one = [&](int n, int slot) __attribute__((always_inline)) { // n-th of the LOADS copies of a stage
        if (n < LA)
            async_copy16(smem_base + uint32_t(slot * TA::BYTES + (n * 4 + wave) * 1024), p_a, la[n]);
        else
            async_copy16(smem_base + uint32_t(A_RING + slot * TB::BYTES + ((n - LA) * 4 + wave) * 1024), p_b, lb[n - LA]);
    };
    {
        WgradListItem first;
        if (!wgrad_list_item(w, 0, first))
            return;
    }
    producer_open();
#pragma unroll
    for (int s = 0; s < S; ++s) { // every item is a whole number of quads
#pragma unroll
        for (int n = 0; n < LOADS; ++n)
            copy_one(n, s);
        p_a += a_step, p_b += b_step;
    }
    if ((p_left -= S) == 0)
        producer_open();

    // ---- consumer -------------------------------------------------------------------------------------------
    uint32_t fa_at[AF], fb_at[BF]; // this lane's fragment addresses inside a stage
#pragma unroll
    for (int i = 0; i < AF; ++i)
        fa_at[i] = ks_frag16_offset<BM>(wm + i * 16, lane);
#pragma unroll
    for (int j = 0; j < BF; ++j)
        fb_at[j] = A_RING + ks_frag16_offset<BN>(wn + j * 16, lane);
    auto read_fragment = [&](bf16x8 (&fa)[AF], bf16x8 (&fb)[BF], int slot, int f) __attribute__((always_inline)) {
        if (f < AF)
            fa[f] = ks_frag16_at<BM>(smem + fa_at[f] + slot * TA::BYTES);
        else
            fb[f - AF] = ks_frag16_at<BN>(smem + fb_at[f - AF] + slot * TB::BYTES);
    };
    f32x4 acc[FM][FN][2][2];
    // Stage t's fragments are in `cur`; the step publishes stage t + 1, reads its fragments into `next` and copies
    // stage t + 4 into the slot stage t leaves.  Straight-line code: no branch between the matrix instructions.
    auto step = [&](auto slot_tag, const bf16x8 (&cur_a)[AF], const bf16x8 (&cur_b)[BF], bf16x8 (&next_a)[AF],
                    bf16x8 (&next_b)[BF]) __attribute__((always_inline)) {
        constexpr int SLOT = decltype(slot_tag)::value, NEXT = (SLOT + 1) % S;
        wait_vmcnt<(S - 2) * LOADS>(); // stages t + 2 and t + 3 may still be in flight
        __builtin_amdgcn_s_waitcnt(0xc07f); // lgkmcnt(0): this wave's reads of stage t are done, its slot may be overwritten
        __builtin_amdgcn_s_barrier();
        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
        for (int j = 0; j < BF; ++j)
#pragma unroll
            for (int i = 0; i < AF; ++i) {
                // the accumulators fill the accumulation registers exactly, the fragments live in the other 256: left to
                // itself the register allocator mixes the two and spends the loop moving tiles between them
                asm volatile("v_mfma_f32_16x16x32_bf16 %0, %1, %2, %0"
                             : "+a"(acc[i >> 1][j >> 1][i & 1][j & 1])
                             : "v"(cur_b[j]), "v"(cur_a[i]));
                const int q = j * AF + i;
                if (q % READ_EVERY == 0 && q / READ_EVERY < AF + BF)
                    read_fragment(next_a, next_b, NEXT, q / READ_EVERY);
                if (q >= COPY_FIRST && (q - COPY_FIRST) % COPY_EVERY == 0 && (q - COPY_FIRST) / COPY_EVERY < LOADS)
                    copy_one((q - COPY_FIRST) / COPY_EVERY, SLOT);
                __builtin_amdgcn_sched_barrier(0);
            }
        p_a += a_step, p_b += b_step;
    };
    bf16x8 fa0[AF], fb0[BF], fa1[AF], fb1[BF];
    wait_vmcnt<(S - 1) * LOADS>(); // stage 0
    __builtin_amdgcn_s_barrier();
#pragma unroll
    for (int f = 0; f < AF + BF; ++f)
        read_fragment(fa0, fb0, 0, f);
    // Zeroed by the matrix pipe (0 x 0 + 0), in place: an assignment would start a new value in other registers and
    // the allocator would move all 256 into place inside the loop.  64 instructions per 32768.
    const bf16x8 zeros = {0, 0, 0, 0, 0, 0, 0, 0};
    auto clear = [&]() __attribute__((always_inline)) {
#pragma unroll
        for (int i = 0; i < FM; ++i)
#pragma unroll
            for (int j = 0; j < FN; ++j)
#pragma unroll
                for (int t = 0; t < 4; ++t)
                    // The compiler does not know that this is a matrix instruction and leaves no wait states between
                    // the moves that fill `zeros` and the instruction, which then multiplies what the registers held
                    // before: the wait states are part of the statement.
                    asm volatile("s_nop 4\n\tv_mfma_f32_16x16x32_bf16 %0, %1, %1, 0"
                                 : "+a"(acc[i][j][t >> 1][t & 1])
                                 : "v"(zeros));
    };
    // One loop over the quads of all items: the accumulators are carried by a single loop, and an item's end is a
    // (wave-uniform) branch behind the four steps.
    WgradListItem item;
    int index = 0;
    wgrad_list_item(w, 0, item);
    int quads_left = item.nq;
    float squares = 0.f; // of the gradient elements this lane has written (not of pieces: the fold squares their sums)
    clear();
    for (;;) {
        step(std::integral_constant<int, 0>{}, fa0, fb0, fa1, fb1);
        step(std::integral_constant<int, 1>{}, fa1, fb1, fa0, fb0);
        step(std::integral_constant<int, 2>{}, fa0, fb0, fa1, fb1);
        step(std::integral_constant<int, 3>{}, fa1, fb1, fa0, fb0);
        if ((p_left -= S) == 0)
            producer_open();
        if (--quads_left)
            continue;
        // A lane holds 4 consecutive columns of one row per 16 x 16 tile: 16 rows x 64 bytes per store.  One running
        // pointer, hidden from the optimiser between rows: 64 precomputed addresses would not fit beside the fragments.
        const int4 t = w.tiles[item.tile];
        const WgradListJob job = w.jobs[t.x];
        float *out = item.piece < 0 ? job.dw + size_t(t.y) * job.lddw + t.z : w.pieces + size_t(item.piece) * (BM * BN);
        const int ld = item.piece < 0 ? job.lddw : BN;
        out += size_t(wm + (lane & 15)) * ld + wn + 4 * (lane >> 4);
#pragma unroll
        for (int i = 0; i < AF; ++i) {
#pragma unroll
            for (int j = 0; j < BF; ++j)
                *reinterpret_cast<f32x4 *>(out + j * 16) = acc[i >> 1][j >> 1][i & 1][j & 1];
            out += size_t(16) * ld;
            asm volatile("" : "+v"(out));
        }
        // the squares of what went out, one 16 x 16 tile at a time (fenced: all 256 accumulators read at once do not
        // fit beside the fragments)
        if (w.sumsq && item.piece < 0) {
#pragma unroll
            for (int i = 0; i < AF; ++i)
#pragma unroll
                for (int j = 0; j < BF; ++j) {
                    // read through assembly: an accumulator that plain code reads stops being pinned to the
                    // accumulation registers, and the allocation of the whole kernel falls apart (103 spills)
                    float v[4];
#pragma unroll
                    for (int e = 0; e < 4; ++e)
                        asm volatile("v_accvgpr_read_b32 %0, %1" : "=v"(v[e]) : "a"(acc[i >> 1][j >> 1][i & 1][j & 1][e]));
                    squares += (v[0] * v[0] + v[1] * v[1]) + (v[2] * v[2] + v[3] * v[3]);
                    __builtin_amdgcn_sched_barrier(0);
                }
        }
        // the copy counter must hold nothing but the three stages the steps assume: let the stores drain
        wait_vmcnt<0>();
        if (!wgrad_list_item(w, ++index, item))
            break;
        quads_left = item.nq;
        clear();
    }
    wait_vmcnt<0>();
    if (w.sumsq) { // fixed tiles per block, fixed order inside a lane and inside a wave: bit-reproducible
        squares = wave_sum(squares);
        if (lane == 0)
            w.sumsq[blockIdx.x * 4 + wave] = squares;
    }
}
// Sums the pieces of the split tiles, in token order, into the gradient.  Eight blocks per tile.
template <int BN>
__global__ __launch_bounds__(256) void wgrad_list_fold_kernel(const WgradList w, int first_tile, int first_sumsq) {
    constexpr int BM = 256, QUADS = BM * BN / 4 / 8 / 256; // float4 per thread
    __shared__ float waves[4];
    float squares = 0.f;
    const int r = blockIdx.x >> 3, part = blockIdx.x & 7;
    const int4 t = w.tiles[first_tile + r];
    const WgradListJob job = w.jobs[t.x];
    const float *first = w.pieces + size_t(r) * w.rem_splits * (BM * BN);
#pragma unroll
    for (int k = 0; k < QUADS; ++k) {
        const int quad = (part * QUADS + k) * 256 + threadIdx.x;
        const int row = quad / (BN / 4), col = (quad % (BN / 4)) * 4;
        f32x4 sum = {0.f, 0.f, 0.f, 0.f};
        for (int split = 0; split < w.rem_splits; ++split) // fixed order
            sum += *reinterpret_cast<const f32x4 *>(first + size_t(split) * (BM * BN) + size_t(quad) * 4);
        f32x4 *p = reinterpret_cast<f32x4 *>(job.dw + size_t(t.y + row) * job.lddw + t.z + col);
        if (w.accumulate)
            sum += *p;
        __builtin_nontemporal_store(sum, p);
        squares += (sum[0] * sum[0] + sum[1] * sum[1]) + (sum[2] * sum[2] + sum[3] * sum[3]);
    }
    if (w.sumsq) {
        squares = wave_sum(squares);
        if ((threadIdx.x & 63) == 0)
            waves[threadIdx.x >> 6] = squares;
        __syncthreads();
        if (threadIdx.x == 0)
            w.sumsq[first_sumsq + blockIdx.x] = (waves[0] + waves[1]) + (waves[2] + waves[3]);
    }
}

// Sums split-K slabs in a fixed order (deterministic) into the fp32 gradient.
__global__ __launch_bounds__(256) void splitk_reduce_kernel(const float *__restrict__ slabs,
                                                            size_t slab_stride, int splits,
                                                            float *__restrict__ out, int rows,
                                                            int cols, int ld_out, int accumulate) {
    const int cols4 = cols >> 2;
    const size_t total = size_t(rows) * cols4;
    for (size_t i = blockIdx.x * size_t(blockDim.x) + threadIdx.x; i < total;
         i += size_t(gridDim.x) * blockDim.x) {
        const int r = int(i / cols4), c = int(i % cols4) * 4;
        float4 sum = make_float4(0, 0, 0, 0);
        for (int s = 0; s < splits; ++s) {
            const float4 v = *reinterpret_cast<const float4 *>(slabs + s * slab_stride + size_t(r) * cols + c);
            sum.x += v.x, sum.y += v.y, sum.z += v.z, sum.w += v.w;
        }
        float4 *p = reinterpret_cast<float4 *>(out + size_t(r) * ld_out + c);
        if (accumulate) {
            const float4 old = *p;
            sum.x += old.x, sum.y += old.y, sum.z += old.z, sum.w += old.w;
        }
        __builtin_nontemporal_store(f32x4{sum.x, sum.y, sum.z, sum.w}, reinterpret_cast<f32x4 *>(p));
    }
}

// ---- host dispatch -------------------------------------------------------------------------
// Per-device facts are cached per device: several engines may run on different GPUs of one process.
constexpr int MAX_DEVICES = 64;
int current_device() {
    int device = 0;
    check_hip(hipGetDevice(&device));
    if (device < 0 || device >= MAX_DEVICES)
        throw std::runtime_error("gemm: device index out of range");
    return device;
}
int compute_units() {
    static std::atomic<int> cached[MAX_DEVICES];
    const int device = current_device();
    int units = cached[device].load(std::memory_order_relaxed);
    if (!units) {
        hipDeviceProp_t prop{};
        check_hip(hipGetDeviceProperties(&prop, device));
        units = prop.multiProcessorCount > 0 ? prop.multiProcessorCount : 256;
        cached[device].store(units, std::memory_order_relaxed);
    }
    return units;
}

enum Tile { TILE_NONE, TILE_128x128, TILE_128x192 };
// 128x192, 3 stages (60 KiB of LDS, <= 186 VGPRs): two blocks are resident per CU, so one block's
// MFMAs cover the other's epilogue, barrier and copy-issue gaps; at N = 768 / 2304 / 3072 and
// M = 16384 it gives 512 / 1536 / 2048 tiles, whole multiples of the 512 resident blocks.  Measured
// on MI355X it beats a 256x192 single-block-per-CU variant on every training shape.
// 128x128, 4 stages: shapes that 192 does not divide.
Tile choose_tile(int rows, int cols) {
    if (rows % 128 == 0 && cols % 192 == 0)
        return TILE_128x192;
    if (rows % 128 == 0 && cols % 128 == 0)
        return TILE_128x128;
    return TILE_NONE;
}
int tile_rows(Tile) { return 128; }
int tile_cols(Tile t) { return t == TILE_128x128 ? 128 : 192; }
int resident_blocks(Tile) { return compute_units() * 2; }

// How many column groups to cut the tile grid into for the eight XCDs (see locate()).  Estimated
// reads beyond L2: every XCD column group streams all of A once; an XCD re-reads its slice of B once
// per pass over its rows unless the slice stays in its 4 MiB L2 beside the streaming operand.
int xcd_columns(int tiles_m, int tiles_n, int BM, int BN, int K, int blocks) {
    if ((tiles_m * tiles_n) % 8)
        return 1;
    const double a_bytes = 2.0 * tiles_m * BM * K, b_bytes = 2.0 * tiles_n * BN * K;
    const int concurrent = blocks / 8 > 0 ? blocks / 8 : 1; // tiles in flight per XCD
    int best = 1;
    double best_cost = 0;
    for (int columns = 1; columns <= 8; columns *= 2) {
        const int xcd_rows = 8 / columns;
        if (tiles_n % columns || tiles_m % xcd_rows)
            continue;
        const double slice = b_bytes / columns;
        const int cols = tiles_n / columns, rows = tiles_m / xcd_rows;
        const int rows_in_flight = concurrent / cols > 0 ? concurrent / cols : 1;
        const int passes = slice <= 2.5 * 1048576 ? 1 : (rows + rows_in_flight - 1) / rows_in_flight;
        const double cost = a_bytes * columns + 8 * slice * passes;
        if (columns == 1 || cost < best_cost)
            best = columns, best_cost = cost;
    }
    return best;
}

template <int BM, int BN, int S, bool AKC, bool BKC, class Epilogue>
void launch_gemm(hipStream_t stream, const bf16_t *A, int lda, const bf16_t *B, int ldb, int M, int N,
                 int K, int splits, int max_blocks, const Epilogue &epilogue) {
    auto kernel = gemm_kernel<BM, BN, S, AKC, BKC, Epilogue>;
    constexpr size_t lds = lds_bytes<BM, BN, S, Epilogue>();
    static std::atomic<bool> configured[MAX_DEVICES]; // the LDS opt-in is a per-device attribute of the kernel
    const int device = current_device();
    if (!configured[device].load(std::memory_order_acquire)) {
        check_hip(hipFuncSetAttribute(reinterpret_cast<const void *>(kernel),
                                      hipFuncAttributeMaxDynamicSharedMemorySize, int(lds)),
                  "gemm LDS size: ");
        configured[device].store(true, std::memory_order_release);
    }
    const int tiles_m = M / BM, tiles_n = N / BN, tiles = tiles_m * tiles_n, items = tiles * splits;
    const int blocks = items < max_blocks ? items : max_blocks;
    hipLaunchKernelGGL(kernel, dim3(blocks), dim3(256), lds, stream, A, lda, B, ldb, K / BK, splits, tiles_n, tiles,
                       splits == 1 ? xcd_columns(tiles_m, tiles_n, BM, BN, K, blocks) : 1, epilogue);
    check_hip(hipGetLastError(), "gemm launch: ");
}

template <bool AKC, bool BKC, class Epilogue>
void dispatch_gemm(hipStream_t stream, Tile tile, const bf16_t *A, int lda, const bf16_t *B, int ldb, int M,
                   int N, int K, int splits, const Epilogue &epilogue) {
    const int blocks = resident_blocks(tile);
    if (tile == TILE_128x192)
        launch_gemm<128, 192, 3, AKC, BKC>(stream, A, lda, B, ldb, M, N, K, splits, blocks, epilogue);
    else
        launch_gemm<128, 128, 4, AKC, BKC>(stream, A, lda, B, ldb, M, N, K, splits, blocks, epilogue);
}

// A reduced dimension that is a multiple of 64 takes the two-stage 64-k kernel.
bool takes_64(Tile tile, int reduced) { return tile != TILE_NONE && reduced % 64 == 0; }

template <int BN, bool AKC, bool BKC, class Epilogue>
void launch_gemm64_tile(hipStream_t stream, const bf16_t *A, int lda, const bf16_t *B, int ldb, int M, int N, int K,
                        int splits, const Epilogue &epilogue) {
    constexpr int BM = 128;
    auto kernel = gemm64_kernel<BM, BN, AKC, BKC, Epilogue>;
    constexpr size_t lds = 2 * (BM + BN) * 128;
    static std::atomic<bool> configured[MAX_DEVICES];
    const int device = current_device();
    if (!configured[device].load(std::memory_order_acquire)) {
        check_hip(hipFuncSetAttribute(reinterpret_cast<const void *>(kernel),
                                      hipFuncAttributeMaxDynamicSharedMemorySize, int(lds)),
                  "gemm LDS size: ");
        configured[device].store(true, std::memory_order_release);
    }
    const int tiles_m = M / BM, tiles_n = N / BN, tiles = tiles_m * tiles_n, items = tiles * splits;
    const int max_blocks = resident_blocks(TILE_128x192);
    const int blocks = items < max_blocks ? items : max_blocks;
    hipLaunchKernelGGL(kernel, dim3(blocks), dim3(256), lds, stream, A, lda, B, ldb, K / 64, splits, tiles_n, tiles,
                       splits == 1 ? xcd_columns(tiles_m, tiles_n, BM, BN, K, blocks) : 1, epilogue);
    check_hip(hipGetLastError(), "gemm launch: ");
}
template <bool AKC, bool BKC, class Epilogue>
void launch_gemm64(hipStream_t stream, Tile tile, const bf16_t *A, int lda, const bf16_t *B, int ldb, int M, int N,
                   int K, int splits, const Epilogue &epilogue) {
    if (tile == TILE_128x192)
        launch_gemm64_tile<192, AKC, BKC>(stream, A, lda, B, ldb, M, N, K, splits, epilogue);
    else
        launch_gemm64_tile<128, AKC, BKC>(stream, A, lda, B, ldb, M, N, K, splits, epilogue);
}

// The 256-row kernels take products with a plain or residual epilogue whose tiles fill the compute units a whole
// number of times (or nearly): one block per unit, nothing to cover a tail or a long epilogue (the GELU epilogues
// stay with gemm64_kernel, where the second block of a unit multiplies meanwhile).
bool takes_256(int M, int N, int K, int bn, int k_period) {
    if (M % 256 || N % bn || K % k_period)
        return false;
    const int tiles = (M / 256) * (N / bn), units = compute_units();
    const int rounds = (tiles + units - 1) / units;
    return tiles * 10 >= rounds * units * 9; // at least 90 % of the last round filled
}
bool takes_256x192(int M, int N, int K, int mode) {
    return (mode == EPI_PLAIN || mode == EPI_RESIDUAL) && takes_256(M, N, K, 192, 384);
}
// Where the 192-wide tile does not fit, with every epilogue: what the 128-wide tile competes with there is two
// 128 x 128 blocks per unit, and its fewer operand bytes per flop outweigh the uncovered GELU epilogue (measured at
// d_model 1024: +17 % and +19 % on the two GELU launches; at widths the 192-wide tiles take, gemm64_kernel's 128 x 192
// blocks keep them)
bool takes_256x128(int M, int N, int K) {
    return !takes_256(M, N, K, 192, 384) && takes_256(M, N, K, 128, 256);
}
template <int BN = 192, int RA = 3, class Epilogue>
void launch_gemm256(hipStream_t stream, const bf16_t *A, int lda, const bf16_t *B, int ldb, int M, int N, int K,
                    const Epilogue &epilogue) {
    auto kernel = gemm256_kernel<BN, RA, Epilogue>;
    constexpr size_t rings = RA * 256 * 128 + 2 * BN * 128, lds = rings + 4 * 2048 > 160 * 1024 ? rings : rings + 4 * 2048;
    constexpr int P = RA % 2 ? 2 * RA : RA;
    static std::atomic<bool> configured[MAX_DEVICES];
    const int device = current_device();
    if (!configured[device].load(std::memory_order_acquire)) {
        check_hip(hipFuncSetAttribute(reinterpret_cast<const void *>(kernel),
                                      hipFuncAttributeMaxDynamicSharedMemorySize, int(lds)),
                  "gemm LDS size: ");
        configured[device].store(true, std::memory_order_release);
    }
    const int tiles_m = M / 256, tiles_n = N / BN, tiles = tiles_m * tiles_n;
    const int units = compute_units(), blocks = tiles < units ? tiles : units;
    hipLaunchKernelGGL(kernel, dim3(blocks), dim3(256), lds, stream, A, lda, B, ldb, K / (64 * P), tiles_n, tiles,
                       xcd_columns(tiles_m, tiles_n, 256, BN, K, blocks), epilogue);
    check_hip(hipGetLastError(), "gemm launch: ");
}
void launch_gemm256_bf16(hipStream_t stream, const bf16_t *A, int lda, const bf16_t *B, int ldb, int M, int N, int K,
                         const EpilogueBf16 &e) {
    if (e.mode == EPI_RESIDUAL)
        launch_gemm256(stream, A, lda, B, ldb, M, N, K, EpilogueBf16As<EPI_RESIDUAL>{e});
    else
        launch_gemm256(stream, A, lda, B, ldb, M, N, K, EpilogueBf16As<EPI_PLAIN>{e});
}
// 256 x 128 tiles, A ring of four slots (period of four stages: reduced dimensions that 256 divides)
void launch_gemm256x128_bf16(hipStream_t stream, const bf16_t *A, int lda, const bf16_t *B, int ldb, int M, int N, int K,
                             const EpilogueBf16 &e) {
    switch (e.mode) {
    case EPI_RESIDUAL:
        return launch_gemm256<128, 4>(stream, A, lda, B, ldb, M, N, K, EpilogueBf16As<EPI_RESIDUAL>{e});
    case EPI_GELU:
        return launch_gemm256<128, 4>(stream, A, lda, B, ldb, M, N, K, EpilogueBf16As<EPI_GELU>{e});
    case EPI_GELU_BWD:
        return launch_gemm256<128, 4>(stream, A, lda, B, ldb, M, N, K, EpilogueBf16As<EPI_GELU_BWD>{e});
    default:
        return launch_gemm256<128, 4>(stream, A, lda, B, ldb, M, N, K, EpilogueBf16As<EPI_PLAIN>{e});
    }
}

// bf16 epilogues of the 64-k kernel: one instantiation per mode
template <bool AKC, bool BKC>
void launch_gemm64_bf16(hipStream_t stream, Tile tile, const bf16_t *A, int lda, const bf16_t *B, int ldb, int M, int N,
                        int K, const EpilogueBf16 &e) {
    switch (e.mode) {
    case EPI_RESIDUAL:
        return launch_gemm64<AKC, BKC>(stream, tile, A, lda, B, ldb, M, N, K, 1, EpilogueBf16As<EPI_RESIDUAL>{e});
    case EPI_GELU:
        return launch_gemm64<AKC, BKC>(stream, tile, A, lda, B, ldb, M, N, K, 1, EpilogueBf16As<EPI_GELU>{e});
    case EPI_GELU_BWD:
        return launch_gemm64<AKC, BKC>(stream, tile, A, lda, B, ldb, M, N, K, 1, EpilogueBf16As<EPI_GELU_BWD>{e});
    default:
        return launch_gemm64<AKC, BKC>(stream, tile, A, lda, B, ldb, M, N, K, 1, EpilogueBf16As<EPI_PLAIN>{e});
    }
}

void check_operand(const void *p, int ld, const char *name) {
    if (!p || (reinterpret_cast<uintptr_t>(p) & 15) || ld % 8)
        throw std::invalid_argument(std::string("gemm operand ") + name +
                                    " must be non-null, 16-byte aligned, leading dimension % 8 == 0");
}

// wgrad has few output tiles and a very long reduction: split it so the work items fill the GPU
int wgrad_splits(Tile tile, int tiles, int k_tiles) {
    int splits = resident_blocks(tile) / tiles;
    if (splits < 1)
        splits = 1;
    const int max_by_k = k_tiles / 8 > 0 ? k_tiles / 8 : 1; // at least 8 k-tiles (256 tokens) per split
    return splits < max_by_k ? splits : max_by_k;
}

} // namespace

extern "C" int tgk_gemm_fwd(hipStream_t stream, int M, int N, int K, const uint16_t *X, int ldx,
                            const uint16_t *W, int ldw, uint16_t *Y, int ldy,
                            const uint16_t *residual, int ldr, uint16_t *gelu_out, int ldg) {
    return guarded([&] {
        require(M > 0 && N > 0 && K > 0, "gemm_fwd: empty shape");
        require(K % BK == 0, "gemm_fwd: K must be a multiple of 32");
        const Tile tile = choose_tile(M, N);
        require(tile != TILE_NONE, "gemm_fwd: M must be a multiple of 128 and N of 128 or 192");
        require(!(residual && gelu_out), "gemm_fwd: residual and GELU epilogues are exclusive");
        check_operand(X, ldx, "X");
        check_operand(W, ldw, "W");
        check_operand(Y, ldy, "Y");
        EpilogueBf16 e{Y, ldy, nullptr, 0, nullptr, 0, EPI_PLAIN};
        if (residual) {
            check_operand(residual, ldr, "residual");
            e.aux = residual, e.ld_aux = ldr, e.mode = EPI_RESIDUAL;
        } else if (gelu_out) {
            check_operand(gelu_out, ldg, "gelu_out");
            e.out2 = gelu_out, e.ld_out2 = ldg, e.mode = EPI_GELU;
        }
        if (takes_256x192(M, N, K, e.mode))
            launch_gemm256_bf16(stream, X, ldx, W, ldw, M, N, K, e);
        else if (takes_256x128(M, N, K))
            launch_gemm256x128_bf16(stream, X, ldx, W, ldw, M, N, K, e);
        else if (takes_64(tile, K))
            launch_gemm64_bf16<true, true>(stream, tile, X, ldx, W, ldw, M, N, K, e);
        else
            dispatch_gemm<true, true>(stream, tile, X, ldx, W, ldw, M, N, K, 1, e);
    });
}

extern "C" int tgk_gemm_fwd_t(hipStream_t stream, int M, int N, int K, const uint16_t *X, int ldx,
                              const uint16_t *Wt, int ldwt, uint16_t *Y, int ldy, const uint16_t *residual,
                              int ldr, uint16_t *gelu_out, int ldg) {
    return guarded([&] {
        require(M > 0 && N > 0 && K > 0, "gemm_fwd_t: empty shape");
        require(K % BK == 0, "gemm_fwd_t: K must be a multiple of 32");
        const Tile tile = choose_tile(M, N);
        require(tile != TILE_NONE, "gemm_fwd_t: M must be a multiple of 128 and N of 128 or 192");
        require(!(residual && gelu_out), "gemm_fwd_t: residual and GELU epilogues are exclusive");
        check_operand(X, ldx, "X");
        check_operand(Wt, ldwt, "Wt");
        check_operand(Y, ldy, "Y");
        EpilogueBf16 e{Y, ldy, nullptr, 0, nullptr, 0, EPI_PLAIN};
        if (residual) {
            check_operand(residual, ldr, "residual");
            e.aux = residual, e.ld_aux = ldr, e.mode = EPI_RESIDUAL;
        } else if (gelu_out) {
            check_operand(gelu_out, ldg, "gelu_out");
            e.out2 = gelu_out, e.ld_out2 = ldg, e.mode = EPI_GELU;
        }
        // B(n, k) = Wt[k][n]: k-strided, whole 384-byte rows per copy instead of 64-byte pieces
        dispatch_gemm<true, false>(stream, tile, X, ldx, Wt, ldwt, M, N, K, 1, e);
    });
}

extern "C" int tgk_gemm_dgrad(hipStream_t stream, int M, int N, int K, const uint16_t *dY, int lddy,
                              const uint16_t *W, int ldw, uint16_t *dX, int lddx,
                              const uint16_t *gelu_pre, int ldu) {
    return guarded([&] {
        require(M > 0 && N > 0 && K > 0, "gemm_dgrad: empty shape");
        require(N % BK == 0, "gemm_dgrad: N (the reduced dimension) must be a multiple of 32");
        const Tile tile = choose_tile(M, K);
        require(tile != TILE_NONE, "gemm_dgrad: M must be a multiple of 128 and K of 128 or 192");
        check_operand(dY, lddy, "dY");
        check_operand(W, ldw, "W");
        check_operand(dX, lddx, "dX");
        EpilogueBf16 e{dX, lddx, nullptr, 0, nullptr, 0, EPI_PLAIN};
        if (gelu_pre) {
            check_operand(gelu_pre, ldu, "gelu_pre");
            e.aux = gelu_pre, e.ld_aux = ldu, e.mode = EPI_GELU_BWD;
        }
        // C[m][i] = sum_o dY[m][o] W[o][i] : B(n=i, k=o) is stored [k][n]
        dispatch_gemm<true, false>(stream, tile, dY, lddy, W, ldw, M, K, N, 1, e);
    });
}

extern "C" int tgk_gemm_dgrad_t(hipStream_t stream, int M, int N, int K, const uint16_t *dY, int lddy,
                                const uint16_t *Wt, int ldwt, uint16_t *dX, int lddx,
                                const uint16_t *gelu_pre, int ldu) {
    return guarded([&] {
        require(M > 0 && N > 0 && K > 0, "gemm_dgrad_t: empty shape");
        require(N % BK == 0, "gemm_dgrad_t: N (the reduced dimension) must be a multiple of 32");
        const Tile tile = choose_tile(M, K);
        require(tile != TILE_NONE, "gemm_dgrad_t: M must be a multiple of 128 and K of 128 or 192");
        check_operand(dY, lddy, "dY");
        check_operand(Wt, ldwt, "Wt");
        check_operand(dX, lddx, "dX");
        EpilogueBf16 e{dX, lddx, nullptr, 0, nullptr, 0, EPI_PLAIN};
        if (gelu_pre) {
            check_operand(gelu_pre, ldu, "gelu_pre");
            e.aux = gelu_pre, e.ld_aux = ldu, e.mode = EPI_GELU_BWD;
        }
        // C[m][i] = sum_o dY[m][o] Wt[i][o]: the forward product with (rows, reduced) = (K, N)
        if (takes_256x192(M, K, N, e.mode))
            launch_gemm256_bf16(stream, dY, lddy, Wt, ldwt, M, K, N, e);
        else if (takes_256x128(M, K, N))
            launch_gemm256x128_bf16(stream, dY, lddy, Wt, ldwt, M, K, N, e);
        else if (takes_64(tile, N))
            launch_gemm64_bf16<true, true>(stream, tile, dY, lddy, Wt, ldwt, M, K, N, e);
        else
            dispatch_gemm<true, true>(stream, tile, dY, lddy, Wt, ldwt, M, K, N, 1, e);
    });
}

extern "C" size_t tgk_gemm_wgrad_workspace(int M, int N, int K) {
    if (M <= 0 || N <= 0 || K <= 0 || M % BK)
        return 0;
    const Tile tile = choose_tile(N, K);
    if (tile == TILE_NONE)
        return 0;
    const int splits = wgrad_splits(tile, (N / tile_rows(tile)) * (K / tile_cols(tile)), M / BK);
    return splits > 1 ? size_t(splits) * N * K * sizeof(float) : 0;
}

extern "C" int tgk_gemm_wgrad(hipStream_t stream, int M, int N, int K, const uint16_t *dY, int lddy,
                              const uint16_t *X, int ldx, float *dW, int lddw, int accumulate,
                              void *workspace, size_t workspace_bytes) {
    return guarded([&] {
        require(M > 0 && N > 0 && K > 0, "gemm_wgrad: empty shape");
        require(M % BK == 0, "gemm_wgrad: M (the reduced dimension) must be a multiple of 32");
        const Tile tile = choose_tile(N, K);
        require(tile != TILE_NONE, "gemm_wgrad: N must be a multiple of 128 and K of 128 or 192");
        check_operand(dY, lddy, "dY");
        check_operand(X, ldx, "X");
        require(dW && !(reinterpret_cast<uintptr_t>(dW) & 15) && lddw % 4 == 0,
                "gemm_wgrad: dW must be 16-byte aligned with leading dimension % 4 == 0");
        const int splits = wgrad_splits(tile, (N / tile_rows(tile)) * (K / tile_cols(tile)), M / BK);
        if (splits == 1) {
            EpilogueF32 e{dW, lddw, 0, accumulate};
            if (takes_64(tile, M))
                launch_gemm64<false, false>(stream, tile, dY, lddy, X, ldx, N, K, M, 1, e);
            else
                dispatch_gemm<false, false>(stream, tile, dY, lddy, X, ldx, N, K, M, 1, e);
            return;
        }
        const size_t need = size_t(splits) * N * K * sizeof(float);
        require(workspace && workspace_bytes >= need && !(reinterpret_cast<uintptr_t>(workspace) & 15),
                "gemm_wgrad: workspace too small (see tgk_gemm_wgrad_workspace)");
        EpilogueF32 e{static_cast<float *>(workspace), K, size_t(N) * K, 0};
        if (takes_64(tile, M))
            launch_gemm64<false, false>(stream, tile, dY, lddy, X, ldx, N, K, M, splits, e);
        else
            dispatch_gemm<false, false>(stream, tile, dY, lddy, X, ldx, N, K, M, splits, e);
        const size_t quads = size_t(N) * K / 4;
        const int blocks = int((quads + 255) / 256 < 4096 ? (quads + 255) / 256 : 4096);
        hipLaunchKernelGGL(splitk_reduce_kernel, dim3(blocks), dim3(256), 0, stream,
                           static_cast<const float *>(workspace), size_t(N) * K, splits, dW, N, K, lddw,
                           accumulate);
        check_hip(hipGetLastError(), "split-K reduce launch: ");
    });
}

namespace {
// Job table and the two tile groups of a batch.
bool plan_wgrad_batch(int M, int count, const TgkWgradJob *jobs, WgradBatch &w, std::string &why) {
    if (count < 1 || count > MAX_WGRAD_JOBS || !jobs) {
        why = "gemm_wgrad_batch: between 1 and 4 jobs";
        return false;
    }
    if (M <= 0 || M % 64) {
        why = "gemm_wgrad_batch: M (the reduced dimension) must be a multiple of 64";
        return false;
    }
    w = WgradBatch{};
    w.count = count;
    w.k_chunks = M / 64;
    for (int j = 0; j < count; ++j) {
        const TgkWgradJob &job = jobs[j];
        if (job.N <= 0 || job.K <= 0 || job.N % 128 || job.K % 192) {
            why = "gemm_wgrad_batch: every N must be a multiple of 128 and every K of 192";
            return false;
        }
        w.dy[j] = job.dY, w.x[j] = job.X, w.dw[j] = job.dW;
        w.lddy[j] = job.lddy, w.ldx[j] = job.ldx, w.lddw[j] = job.lddw;
        w.tiles_n[j] = job.K / 192;
        w.first_tile[j + 1] = w.first_tile[j] + (job.N / 128) * (job.K / 192);
    }
    // Two groups of tiles, each split so that it makes (up to) one item per resident block: the first
    // blocks / ceil(blocks / tiles) tiles ceil(blocks / tiles) ways, the rest as many ways as fill the blocks
    // again (items of at least four chunks).
    const int tiles = w.first_tile[count], blocks = resident_blocks(TILE_128x192);
    const int max_splits = w.k_chunks / 4 > 0 ? w.k_chunks / 4 : 1;
    int splits_a = (blocks + tiles - 1) / tiles;
    if (splits_a > max_splits)
        splits_a = max_splits;
    int tiles_a = blocks / splits_a;
    if (tiles_a > tiles)
        tiles_a = tiles;
    const int tiles_b = tiles - tiles_a;
    int splits_b = tiles_b ? blocks / tiles_b : 1;
    if (splits_b > max_splits)
        splits_b = max_splits;
    if (splits_b < 1)
        splits_b = 1;
    w.tiles_a = tiles_a, w.splits_a = splits_a, w.tiles_b = tiles_b, w.splits_b = splits_b;
    return true;
}
int wgrad_batch_blocks(const WgradBatch &w) {
    const int a = w.tiles_a * w.splits_a, b = w.tiles_b * w.splits_b;
    return a > b ? a : b;
}
size_t wgrad_batch_pieces(const WgradBatch &w) {
    return size_t(w.tiles_a * w.splits_a + w.tiles_b * w.splits_b) * 128 * 192 * sizeof(float);
}
} // namespace

extern "C" size_t tgk_gemm_wgrad_batch_workspace(int M, int count, const TgkWgradJob *jobs) {
    try {
        WgradBatch w;
        std::string why;
        return plan_wgrad_batch(M, count, jobs, w, why) ? wgrad_batch_pieces(w) : 0;
    } catch (...) {
        return 0;
    }
}

extern "C" int tgk_gemm_wgrad_batch(hipStream_t stream, int M, int count, const TgkWgradJob *jobs, int accumulate,
                                    void *workspace, size_t workspace_bytes) {
    return guarded([&] {
        WgradBatch w;
        std::string why;
        if (!plan_wgrad_batch(M, count, jobs, w, why))
            throw std::invalid_argument(why);
        for (int j = 0; j < count; ++j) {
            check_operand(jobs[j].dY, jobs[j].lddy, "dY");
            check_operand(jobs[j].X, jobs[j].ldx, "X");
            require(jobs[j].lddy >= jobs[j].N && jobs[j].ldx >= jobs[j].K, "gemm_wgrad_batch: leading dimension too small");
            require(jobs[j].dW && !(reinterpret_cast<uintptr_t>(jobs[j].dW) & 15) && jobs[j].lddw % 4 == 0 &&
                        jobs[j].lddw >= jobs[j].K,
                    "gemm_wgrad_batch: dW must be 16-byte aligned with leading dimension % 4 == 0");
        }
        require(workspace && workspace_bytes >= wgrad_batch_pieces(w) && !(reinterpret_cast<uintptr_t>(workspace) & 15),
                "gemm_wgrad_batch: workspace too small (see tgk_gemm_wgrad_batch_workspace)");
        w.accumulate = accumulate;
        w.pieces = static_cast<float *>(workspace);
        auto kernel = wgrad_batch_kernel<128, 192>;
        constexpr size_t lds = 2 * (128 + 192) * 128;
        static std::atomic<bool> configured[MAX_DEVICES];
        const int device = current_device();
        if (!configured[device].load(std::memory_order_acquire)) {
            check_hip(hipFuncSetAttribute(reinterpret_cast<const void *>(kernel),
                                          hipFuncAttributeMaxDynamicSharedMemorySize, int(lds)),
                      "gemm LDS size: ");
            configured[device].store(true, std::memory_order_release);
        }
        hipLaunchKernelGGL(kernel, dim3(wgrad_batch_blocks(w)), dim3(256), lds, stream, w);
        check_hip(hipGetLastError(), "wgrad batch launch: ");
        hipLaunchKernelGGL((wgrad_batch_fold_kernel<128, 192>), dim3(w.first_tile[count] * 4), dim3(256), 0, stream, w);
        check_hip(hipGetLastError(), "wgrad batch fold launch: ");
    });
}

namespace {
// Tables and split of a whole-step weight-gradient launch.
struct WgradListPlan {
    int tiles, blocks, rounds, rem_tiles, rem_splits, launch_blocks, fold_blocks;
    size_t jobs_bytes, table_bytes, pieces_bytes;
};
bool plan_wgrad_list(int M, int count, const TgkWgradJob *jobs, WgradListPlan &plan, std::string &why) {
    if (count < 1 || count > 4096 || !jobs) {
        why = "gemm_wgrad_list: between 1 and 4096 jobs";
        return false;
    }
    if (M <= 0 || M % 128) {
        why = "gemm_wgrad_list: M (the reduced dimension) must be a multiple of 128";
        return false;
    }
    int tiles = 0;
    for (int j = 0; j < count; ++j) {
        if (jobs[j].N <= 0 || jobs[j].K <= 0 || jobs[j].N % 256 || jobs[j].K % 256) {
            why = "gemm_wgrad_list: every N and K must be a multiple of 256";
            return false;
        }
        tiles += (jobs[j].N / 256) * (jobs[j].K / 256);
    }
    plan.tiles = tiles;
    plan.blocks = compute_units();
    plan.rounds = tiles / plan.blocks;
    plan.rem_tiles = tiles % plan.blocks;
    const int k_quads = M / 128;
    plan.rem_splits = plan.rem_tiles ? std::min(plan.blocks / plan.rem_tiles, k_quads) : 1;
    plan.jobs_bytes = (size_t(count) * sizeof(WgradListJob) + 15) / 16 * 16;
    plan.table_bytes = plan.jobs_bytes + size_t(tiles) * sizeof(int4);
    plan.pieces_bytes = plan.rem_splits > 1 ? size_t(plan.rem_tiles) * plan.rem_splits * 256 * 256 * sizeof(float) : 0;
    plan.launch_blocks = plan.rounds ? plan.blocks : plan.rem_tiles * plan.rem_splits;
    plan.fold_blocks = plan.rem_splits > 1 ? plan.rem_tiles * 8 : 0;
    return true;
}
} // namespace

extern "C" size_t tgk_gemm_wgrad_list_table_bytes(int M, int count, const TgkWgradJob *jobs) {
    try {
        WgradListPlan plan;
        std::string why;
        return plan_wgrad_list(M, count, jobs, plan, why) ? plan.table_bytes : 0;
    } catch (...) {
        return 0;
    }
}
extern "C" size_t tgk_gemm_wgrad_list_workspace(int M, int count, const TgkWgradJob *jobs) {
    try {
        WgradListPlan plan;
        std::string why;
        return plan_wgrad_list(M, count, jobs, plan, why) ? plan.pieces_bytes : 0;
    } catch (...) {
        return 0;
    }
}
extern "C" int tgk_gemm_wgrad_list_sumsq_count(int M, int count, const TgkWgradJob *jobs) {
    try {
        WgradListPlan plan;
        std::string why;
        return plan_wgrad_list(M, count, jobs, plan, why) ? 4 * plan.launch_blocks + plan.fold_blocks : 0;
    } catch (...) {
        return 0;
    }
}
extern "C" int tgk_gemm_wgrad_list_prepare(int M, int count, const TgkWgradJob *jobs, void *table, size_t table_bytes) {
    return guarded([&] {
        WgradListPlan plan;
        std::string why;
        if (!plan_wgrad_list(M, count, jobs, plan, why))
            throw std::invalid_argument(why);
        require(table && table_bytes >= plan.table_bytes && !(reinterpret_cast<uintptr_t>(table) & 15),
                "gemm_wgrad_list_prepare: table too small (see tgk_gemm_wgrad_list_table_bytes)");
        std::vector<unsigned char> host(plan.table_bytes, 0);
        WgradListJob *job_table = reinterpret_cast<WgradListJob *>(host.data());
        int4 *tile_table = reinterpret_cast<int4 *>(host.data() + plan.jobs_bytes);
        int tile = 0;
        for (int j = 0; j < count; ++j) {
            const TgkWgradJob &job = jobs[j];
            check_operand(job.dY, job.lddy, "dY");
            check_operand(job.X, job.ldx, "X");
            require(job.lddy >= job.N && job.ldx >= job.K, "gemm_wgrad_list: leading dimension too small");
            require(job.dW && !(reinterpret_cast<uintptr_t>(job.dW) & 15) && job.lddw % 4 == 0 && job.lddw >= job.K,
                    "gemm_wgrad_list: dW must be 16-byte aligned with leading dimension % 4 == 0");
            job_table[j] = {job.dY, job.X, job.dW, job.lddy, job.ldx, job.lddw, 0};
            for (int m = 0; m < job.N; m += 256)
                for (int n = 0; n < job.K; n += 256)
                    tile_table[tile++] = make_int4(j, m, n, 0);
        }
        check_hip(hipMemcpy(table, host.data(), host.size(), hipMemcpyHostToDevice), "wgrad list tables: ");
    });
}
extern "C" int tgk_gemm_wgrad_list(hipStream_t stream, int M, int count, const TgkWgradJob *jobs, const void *table,
                                   int accumulate, void *workspace, size_t workspace_bytes, float *sumsq) {
    return guarded([&] {
        WgradListPlan plan;
        std::string why;
        if (!plan_wgrad_list(M, count, jobs, plan, why))
            throw std::invalid_argument(why);
        require(accumulate == 0, "gemm_wgrad_list: accumulate is not supported (every gradient is written once)");
        require(table && !(reinterpret_cast<uintptr_t>(table) & 15), "gemm_wgrad_list: no table (see tgk_gemm_wgrad_list_prepare)");
        require(plan.pieces_bytes == 0 ||
                    (workspace && workspace_bytes >= plan.pieces_bytes && !(reinterpret_cast<uintptr_t>(workspace) & 15)),
                "gemm_wgrad_list: workspace too small (see tgk_gemm_wgrad_list_workspace)");
        WgradList w{};
        w.jobs = static_cast<const WgradListJob *>(table);
        w.tiles = reinterpret_cast<const int4 *>(static_cast<const unsigned char *>(table) + plan.jobs_bytes);
        w.rounds = plan.rounds, w.rem_tiles = plan.rem_tiles, w.rem_splits = plan.rem_splits;
        w.k_quads = M / 128;
        w.accumulate = accumulate;
        w.pieces = static_cast<float *>(workspace);
        require(!(reinterpret_cast<uintptr_t>(sumsq) & 3), "gemm_wgrad_list: sumsq must be 4-byte aligned");
        w.sumsq = sumsq;
        auto kernel = wgrad_list_kernel<256>;
        constexpr size_t lds = 4 * (256 + 256) * 64;
        static std::atomic<bool> configured[MAX_DEVICES];
        const int device = current_device();
        if (!configured[device].load(std::memory_order_acquire)) {
            check_hip(hipFuncSetAttribute(reinterpret_cast<const void *>(kernel),
                                          hipFuncAttributeMaxDynamicSharedMemorySize, int(lds)),
                      "gemm LDS size: ");
            configured[device].store(true, std::memory_order_release);
        }
        hipLaunchKernelGGL(kernel, dim3(plan.launch_blocks), dim3(256), lds, stream, w);
        check_hip(hipGetLastError(), "wgrad list launch: ");
        if (plan.fold_blocks) {
            hipLaunchKernelGGL((wgrad_list_fold_kernel<256>), dim3(plan.fold_blocks), dim3(256), 0, stream, w,
                               plan.rounds * plan.blocks, 4 * plan.launch_blocks);
            check_hip(hipGetLastError(), "wgrad list fold launch: ");
        }
    });
}
