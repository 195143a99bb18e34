// bf16 MFMA GEMM family for gfx950: forward Y = X W^T, dgrad dX = dY W, wgrad dW = dY^T X.
// Replaces project / matmul+cast_result / weight_gradient of the reference
// (cuda/mma.cuh:77-108, cuda/ops.cuh:30-55, cuda/ops.cuh:83-109).
//
// One kernel template computes C[m][n] = sum_k A(m,k) B(n,k).  Each operand is either
// "k-contiguous" (stored [row][k]) or "k-strided" (stored [k][row]); k-strided tiles are
// transposed in registers on their way into LDS, so the LDS image is always [row][k] and every
// MFMA fragment is one 16-byte LDS read.
//   forward : A = X  [M][K] k-contiguous, B = W  [N][K] k-contiguous
//   dgrad   : A = dY [M][N] k-contiguous, B = W  [N][K] read as (n=K index, k=N index): k-strided
//   wgrad   : A = dY [M][N] k-strided (m = out index), B = X [M][K] k-strided, fp32 out, split-K
//
// Tile: BM x BN x 64 per 256-thread block, 2x2 waves, v_mfma_f32_32x32x16_bf16 with the operands
// swapped (instruction A = our B rows) so that a lane ends up holding 4 consecutive n for one m:
// 8-byte bf16 / 16-byte fp32 stores.  LDS is double buffered, global loads for tile k+1 are in
// flight while tile k is multiplied; one barrier per k-tile.
#include "common.h"
#include "../../include/tgk_kernels.h"

namespace {

constexpr int BK = 64;
constexpr int LDS_STRIDE = BK + 8; // elements; 144-byte rows keep 16-byte reads conflict-free

enum EpilogueMode { EPI_PLAIN = 0, EPI_RESIDUAL = 1, EPI_GELU = 2, EPI_GELU_BWD = 3 };

struct EpilogueBf16 {
    bf16_t *out;
    int ld_out;
    const bf16_t *aux; // residual (EPI_RESIDUAL) or saved pre-activation (EPI_GELU_BWD)
    int ld_aux;
    bf16_t *out2; // GELU output (EPI_GELU)
    int ld_out2;
    int mode;
    int split_stride_unused;
    TG_DEVICE void operator()(int m, int n, const float (&v)[4], int) const {
        u32x2 packed;
        if (mode == EPI_RESIDUAL) {
            // y = RN(RN(acc) + residual): the bf16 add of cuda/mma.cuh:95-97
            const u32x2 r = *reinterpret_cast<const u32x2 *>(aux + size_t(m) * ld_aux + n);
            packed.x = pack_bf16(round_bf16(v[0]) + bf16_lo(r.x), round_bf16(v[1]) + bf16_hi(r.x));
            packed.y = pack_bf16(round_bf16(v[2]) + bf16_lo(r.y), round_bf16(v[3]) + bf16_hi(r.y));
        } else if (mode == EPI_GELU_BWD) {
            // du = RN(RN(acc) * gelu'(u))
            const u32x2 u = *reinterpret_cast<const u32x2 *>(aux + size_t(m) * ld_aux + n);
            packed.x = pack_bf16(round_bf16(v[0]) * gelu_grad_f(bf16_lo(u.x)),
                                 round_bf16(v[1]) * gelu_grad_f(bf16_hi(u.x)));
            packed.y = pack_bf16(round_bf16(v[2]) * gelu_grad_f(bf16_lo(u.y)),
                                 round_bf16(v[3]) * gelu_grad_f(bf16_hi(u.y)));
        } else {
            packed.x = pack_bf16(v[0], v[1]);
            packed.y = pack_bf16(v[2], v[3]);
            if (mode == EPI_GELU) {
                u32x2 g;
                g.x = pack_bf16(gelu_f(bf16_lo(packed.x)), gelu_f(bf16_hi(packed.x)));
                g.y = pack_bf16(gelu_f(bf16_lo(packed.y)), gelu_f(bf16_hi(packed.y)));
                *reinterpret_cast<u32x2 *>(out2 + size_t(m) * ld_out2 + n) = g;
            }
        }
        *reinterpret_cast<u32x2 *>(out + size_t(m) * ld_out + n) = packed;
    }
};

struct EpilogueF32 {
    float *out;
    int ld_out;
    size_t split_stride; // elements between split-K slabs
    int accumulate;      // only honoured when there is a single split
    TG_DEVICE void operator()(int m, int n, const float (&v)[4], int split) const {
        f32x4 *p = reinterpret_cast<f32x4 *>(out + split * split_stride + size_t(m) * ld_out + n);
        f32x4 value = {v[0], v[1], v[2], v[3]};
        if (accumulate)
            value += *p;
        *p = value;
    }
};

// Staging of one ROWS x 64 operand tile: global -> registers -> LDS image [row][k].
// Plain register arrays with compile-time indices only, so they stay in VGPRs.
template <int ROWS, int NT, bool KCONTIG> struct TileShape {
    static constexpr int GROUPS = ROWS / 8 * (BK / 4);         // 8-row x 4-k groups (k-strided)
    static constexpr int GROUP_ITERS = (GROUPS + NT - 1) / NT; // last iteration may be partial
    static constexpr int CHUNKS = KCONTIG ? ROWS * BK / 8 / NT : GROUP_ITERS * 4; // 16-byte chunks
    static_assert(!KCONTIG || ROWS * BK / 8 % NT == 0, "tile must divide over the block");
};

template <int ROWS, int NT, bool KCONTIG, int COUNT>
TG_DEVICE void stage_load(u32x4 (&regs)[COUNT], const bf16_t *base, int ld, int row0, int k0, int tid) {
    using S = TileShape<ROWS, NT, KCONTIG>;
    static_assert(COUNT == S::CHUNKS, "register tile size");
    if constexpr (KCONTIG) {
#pragma unroll
        for (int i = 0; i < S::CHUNKS; ++i) {
            const int c = tid + i * NT, row = c >> 3, kc = c & 7;
            regs[i] = *reinterpret_cast<const u32x4 *>(base + size_t(row0 + row) * ld + k0 + kc * 8);
        }
    } else {
        // group g: 8 rows (m8) x 4 k (k4); k4 varies fastest over lanes so that the transposed
        // 8-byte LDS writes of a half wave fall into distinct banks
#pragma unroll
        for (int i = 0; i < S::GROUP_ITERS; ++i) {
            const int g = tid + i * NT, k4 = g & 15, m8 = g >> 4;
            const bool live = S::GROUPS % NT == 0 || g < S::GROUPS;
#pragma unroll
            for (int kk = 0; kk < 4; ++kk)
                regs[i * 4 + kk] = live ? *reinterpret_cast<const u32x4 *>(
                                              base + size_t(k0 + k4 * 4 + kk) * ld + row0 + m8 * 8)
                                        : u32x4{0, 0, 0, 0};
        }
    }
}

TG_DEVICE void store_transposed_pair(bf16_t *p, uint32_t r0, uint32_t r1, uint32_t r2, uint32_t r3) {
    // r_k holds rows (2j, 2j+1) at k; emit row 2j and row 2j+1 with k = 0..3 contiguous
    u32x2 even, odd;
    even.x = (r0 & 0xffffu) | (r1 << 16);
    even.y = (r2 & 0xffffu) | (r3 << 16);
    odd.x = (r0 >> 16) | (r1 & 0xffff0000u);
    odd.y = (r2 >> 16) | (r3 & 0xffff0000u);
    *reinterpret_cast<u32x2 *>(p) = even;
    *reinterpret_cast<u32x2 *>(p + LDS_STRIDE) = odd;
}

template <int ROWS, int NT, bool KCONTIG, int COUNT>
TG_DEVICE void stage_store(const u32x4 (&regs)[COUNT], bf16_t *lds, int tid) {
    using S = TileShape<ROWS, NT, KCONTIG>;
    static_assert(COUNT == S::CHUNKS, "register tile size");
    if constexpr (KCONTIG) {
#pragma unroll
        for (int i = 0; i < S::CHUNKS; ++i) {
            const int c = tid + i * NT, row = c >> 3, kc = c & 7;
            *reinterpret_cast<u32x4 *>(lds + row * LDS_STRIDE + kc * 8) = regs[i];
        }
    } else {
#pragma unroll
        for (int i = 0; i < S::GROUP_ITERS; ++i) {
            const int g = tid + i * NT, k4 = g & 15, m8 = g >> 4;
            if (S::GROUPS % NT == 0 || g < S::GROUPS) {
                bf16_t *p = lds + (m8 * 8) * LDS_STRIDE + k4 * 4;
                const u32x4 a = regs[i * 4 + 0], b = regs[i * 4 + 1], c = regs[i * 4 + 2], d = regs[i * 4 + 3];
                store_transposed_pair(p + 0 * LDS_STRIDE, a.x, b.x, c.x, d.x);
                store_transposed_pair(p + 2 * LDS_STRIDE, a.y, b.y, c.y, d.y);
                store_transposed_pair(p + 4 * LDS_STRIDE, a.z, b.z, c.z, d.z);
                store_transposed_pair(p + 6 * LDS_STRIDE, a.w, b.w, c.w, d.w);
            }
        }
    }
}

template <int BM, int BN> constexpr size_t gemm_lds_bytes() {
    return size_t(2) * (BM + BN) * LDS_STRIDE * sizeof(bf16_t);
}

template <int BM, int BN, bool AKC, bool BKC, class Epilogue>
__global__ __launch_bounds__(256) void gemm_kernel(const bf16_t *__restrict__ A, int lda,
                                                   const bf16_t *__restrict__ B, int ldb,
                                                   int k_tiles, int splits, int tiles_n,
                                                   int tiles_total, Epilogue epilogue) {
    constexpr int NT = 256, WM = BM / 2, WN = BN / 2, FM = WM / 32, FN = WN / 32;
    extern __shared__ __align__(16) unsigned char smem[];
    bf16_t *const sA = reinterpret_cast<bf16_t *>(smem);    // two stages of BM rows
    bf16_t *const sB = sA + 2 * BM * LDS_STRIDE;             // two stages of BN rows

    // Blocks are dealt round-robin to the 8 XCDs; give each XCD a contiguous run of tiles so
    // that tiles sharing operand rows meet in the same L2.
    const int blocks = gridDim.x;
    int logical = blockIdx.x;
    if ((blocks & 7) == 0)
        logical = (logical & 7) * (blocks >> 3) + (logical >> 3);
    const int split = logical / tiles_total, tile = logical - split * tiles_total;
    const int m0 = (tile / tiles_n) * BM, n0 = (tile % tiles_n) * BN;
    const int kt0 = int(int64_t(split) * k_tiles / splits);
    const int kt1 = int(int64_t(split + 1) * k_tiles / splits);

    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int wm = (wave >> 1) * WM, wn = (wave & 1) * WN;
    const int frag_row = lane & 31, frag_k = (lane >> 5) * 8;

    f32x16 acc[FM][FN];
#pragma unroll
    for (int i = 0; i < FM; ++i)
#pragma unroll
        for (int j = 0; j < FN; ++j)
#pragma unroll
            for (int r = 0; r < 16; ++r)
                acc[i][j][r] = 0.f;

    u32x4 regsA[TileShape<BM, NT, AKC>::CHUNKS], regsB[TileShape<BN, NT, BKC>::CHUNKS];
    if (kt0 < kt1) {
        stage_load<BM, NT, AKC>(regsA, A, lda, m0, kt0 * BK, tid);
        stage_load<BN, NT, BKC>(regsB, B, ldb, n0, kt0 * BK, tid);
        stage_store<BM, NT, AKC>(regsA, sA, tid);
        stage_store<BN, NT, BKC>(regsB, sB, tid);
    }
    __syncthreads();
    for (int kt = kt0; kt < kt1; ++kt) {
        const int cur = (kt - kt0) & 1;
        const bool more = kt + 1 < kt1;
        if (more) {
            stage_load<BM, NT, AKC>(regsA, A, lda, m0, (kt + 1) * BK, tid);
            stage_load<BN, NT, BKC>(regsB, B, ldb, n0, (kt + 1) * BK, tid);
        }
        const bf16_t *a_base = sA + cur * (BM * LDS_STRIDE) + (wm + frag_row) * LDS_STRIDE + frag_k;
        const bf16_t *b_base = sB + cur * (BN * LDS_STRIDE) + (wn + frag_row) * LDS_STRIDE + frag_k;
#pragma unroll
        for (int ks = 0; ks < BK / 16; ++ks) {
            bf16x8 af[FM], bfr[FN];
#pragma unroll
            for (int i = 0; i < FM; ++i)
                af[i] = *reinterpret_cast<const bf16x8 *>(a_base + i * 32 * LDS_STRIDE + ks * 16);
#pragma unroll
            for (int j = 0; j < FN; ++j)
                bfr[j] = *reinterpret_cast<const bf16x8 *>(b_base + j * 32 * LDS_STRIDE + ks * 16);
#pragma unroll
            for (int i = 0; i < FM; ++i)
#pragma unroll
                for (int j = 0; j < FN; ++j)
                    acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(bfr[j], af[i], acc[i][j], 0, 0, 0);
        }
        if (more) {
            stage_store<BM, NT, AKC>(regsA, sA + (cur ^ 1) * (BM * LDS_STRIDE), tid);
            stage_store<BN, NT, BKC>(regsB, sB + (cur ^ 1) * (BN * LDS_STRIDE), tid);
        }
        __syncthreads();
    }

    // accumulator register r of a lane: m = lane%32, n = 8*(r/4) + 4*(lane/32) + r%4
    const int out_m = m0 + wm + frag_row, out_n = n0 + wn + (lane >> 5) * 4;
#pragma unroll
    for (int i = 0; i < FM; ++i)
#pragma unroll
        for (int j = 0; j < FN; ++j)
#pragma unroll
            for (int q = 0; q < 4; ++q) {
                const float v[4] = {acc[i][j][q * 4 + 0], acc[i][j][q * 4 + 1], acc[i][j][q * 4 + 2],
                                    acc[i][j][q * 4 + 3]};
                epilogue(out_m + i * 32, out_n + j * 32 + q * 8, v, split);
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
        *p = sum;
    }
}

// ---- host dispatch -------------------------------------------------------------------------
int compute_units() {
    static int cached = 0;
    if (!cached) {
        int device = 0;
        hipDeviceProp_t prop{};
        check_hip(hipGetDevice(&device));
        check_hip(hipGetDeviceProperties(&prop, device));
        cached = prop.multiProcessorCount > 0 ? prop.multiProcessorCount : 256;
    }
    return cached;
}

struct TileChoice {
    int bm, bn;
};
// Measured on MI355X at the training shapes (M = 16384, N and K in {768, 2304, 3072}).  The
// 128x128 tile keeps two blocks resident per CU, so a co-resident block covers the other's
// prologue, epilogue and global-load latency: it wins whenever the reduction is short (12 k-tiles
// at K = 768).  With a k-strided operand and a long reduction the 256x192 tile's lower LDS and L2
// traffic wins instead.
TileChoice choose_tile(int M, int N, int K, bool kstrided_operand) {
    const bool big_ok = M % 256 == 0 && N % 192 == 0;
    if (big_ok && kstrided_operand && K >= 2048)
        return {256, 192};
    if (M % 128 == 0 && N % 128 == 0)
        return {128, 128};
    if (big_ok)
        return {256, 192};
    return {0, 0};
}

template <int BM, int BN, bool AKC, bool BKC, class Epilogue>
void launch_gemm(hipStream_t stream, const bf16_t *A, int lda, const bf16_t *B, int ldb, int M, int N,
                 int K, int splits, const Epilogue &epilogue) {
    auto kernel = gemm_kernel<BM, BN, AKC, BKC, Epilogue>;
    constexpr size_t lds = gemm_lds_bytes<BM, BN>();
    static bool configured = false;
    if (!configured) {
        check_hip(hipFuncSetAttribute(reinterpret_cast<const void *>(kernel),
                                      hipFuncAttributeMaxDynamicSharedMemorySize, int(lds)),
                  "gemm LDS size: ");
        configured = true;
    }
    const int tiles_n = N / BN, tiles = (M / BM) * tiles_n;
    hipLaunchKernelGGL(kernel, dim3(tiles * splits), dim3(256), lds, stream, A, lda, B, ldb, K / BK,
                       splits, tiles_n, tiles, epilogue);
    check_hip(hipGetLastError(), "gemm launch: ");
}

template <bool AKC, bool BKC, class Epilogue>
void dispatch_gemm(hipStream_t stream, TileChoice tile, const bf16_t *A, int lda, const bf16_t *B,
                   int ldb, int M, int N, int K, int splits, const Epilogue &epilogue) {
    if (tile.bm == 256 && tile.bn == 192)
        launch_gemm<256, 192, AKC, BKC>(stream, A, lda, B, ldb, M, N, K, splits, epilogue);
    else if (tile.bm == 256 && tile.bn == 256)
        launch_gemm<256, 256, AKC, BKC>(stream, A, lda, B, ldb, M, N, K, splits, epilogue);
    else
        launch_gemm<128, 128, AKC, BKC>(stream, A, lda, B, ldb, M, N, K, splits, epilogue);
}

void check_operand(const void *p, int ld, const char *name) {
    if (!p || (reinterpret_cast<uintptr_t>(p) & 15) || ld % 8)
        throw std::invalid_argument(std::string("gemm operand ") + name +
                                    " must be non-null, 16-byte aligned, leading dimension % 8 == 0");
}

int wgrad_splits(int tiles, int k_tiles) {
    const int cus = compute_units();
    int splits = cus / tiles;
    if (splits < 1)
        splits = 1;
    const int max_by_k = k_tiles / 4 > 0 ? k_tiles / 4 : 1; // at least 4 k-tiles per split
    return splits < max_by_k ? splits : max_by_k;
}

TileChoice wgrad_tile(int rows, int cols) {
    // few output tiles and a very long reduction: the big tiles win (measured), split-K fills the CUs
    if (rows % 256 == 0 && cols % 192 == 0)
        return {256, 192};
    if (rows % 256 == 0 && cols % 256 == 0)
        return {256, 256};
    if (rows % 128 == 0 && cols % 128 == 0)
        return {128, 128};
    return {0, 0};
}

} // namespace

extern "C" int tgk_gemm_fwd(hipStream_t stream, int M, int N, int K, const uint16_t *X, int ldx,
                            const uint16_t *W, int ldw, uint16_t *Y, int ldy,
                            const uint16_t *residual, int ldr, uint16_t *gelu_out, int ldg) {
    return guarded([&] {
        require(M > 0 && N > 0 && K > 0, "gemm_fwd: empty shape");
        require(K % BK == 0, "gemm_fwd: K must be a multiple of 64");
        const TileChoice tile = choose_tile(M, N, K, false);
        require(tile.bm != 0, "gemm_fwd: M and N must be multiples of 128 (or of 256 and 192)");
        require(!(residual && gelu_out), "gemm_fwd: residual and GELU epilogues are exclusive");
        check_operand(X, ldx, "X");
        check_operand(W, ldw, "W");
        check_operand(Y, ldy, "Y");
        EpilogueBf16 e{Y, ldy, nullptr, 0, nullptr, 0, EPI_PLAIN, 0};
        if (residual) {
            check_operand(residual, ldr, "residual");
            e.aux = residual, e.ld_aux = ldr, e.mode = EPI_RESIDUAL;
        } else if (gelu_out) {
            check_operand(gelu_out, ldg, "gelu_out");
            e.out2 = gelu_out, e.ld_out2 = ldg, e.mode = EPI_GELU;
        }
        dispatch_gemm<true, true>(stream, tile, X, ldx, W, ldw, M, N, K, 1, e);
    });
}

extern "C" int tgk_gemm_dgrad(hipStream_t stream, int M, int N, int K, const uint16_t *dY, int lddy,
                              const uint16_t *W, int ldw, uint16_t *dX, int lddx,
                              const uint16_t *gelu_pre, int ldu) {
    return guarded([&] {
        require(M > 0 && N > 0 && K > 0, "gemm_dgrad: empty shape");
        require(N % BK == 0, "gemm_dgrad: N (the reduced dimension) must be a multiple of 64");
        const TileChoice tile = choose_tile(M, K, N, true);
        require(tile.bm != 0, "gemm_dgrad: M and K must be multiples of 128 (or of 256 and 192)");
        check_operand(dY, lddy, "dY");
        check_operand(W, ldw, "W");
        check_operand(dX, lddx, "dX");
        EpilogueBf16 e{dX, lddx, nullptr, 0, nullptr, 0, EPI_PLAIN, 0};
        if (gelu_pre) {
            check_operand(gelu_pre, ldu, "gelu_pre");
            e.aux = gelu_pre, e.ld_aux = ldu, e.mode = EPI_GELU_BWD;
        }
        // C[m][i] = sum_o dY[m][o] W[o][i] : B(n=i, k=o) is stored [k][n]
        dispatch_gemm<true, false>(stream, tile, dY, lddy, W, ldw, M, K, N, 1, e);
    });
}

extern "C" size_t tgk_gemm_wgrad_workspace(int M, int N, int K) {
    if (M <= 0 || N <= 0 || K <= 0 || M % BK)
        return 0;
    const TileChoice tile = wgrad_tile(N, K);
    if (!tile.bm)
        return 0;
    const int splits = wgrad_splits((N / tile.bm) * (K / tile.bn), M / BK);
    return splits > 1 ? size_t(splits) * N * K * sizeof(float) : 0;
}

extern "C" int tgk_gemm_wgrad(hipStream_t stream, int M, int N, int K, const uint16_t *dY, int lddy,
                              const uint16_t *X, int ldx, float *dW, int lddw, int accumulate,
                              void *workspace, size_t workspace_bytes) {
    return guarded([&] {
        require(M > 0 && N > 0 && K > 0, "gemm_wgrad: empty shape");
        require(M % BK == 0, "gemm_wgrad: M (the reduced dimension) must be a multiple of 64");
        const TileChoice tile = wgrad_tile(N, K);
        require(tile.bm != 0, "gemm_wgrad: N and K must be multiples of 128 (or of 256 and 192)");
        check_operand(dY, lddy, "dY");
        check_operand(X, ldx, "X");
        require(dW && !(reinterpret_cast<uintptr_t>(dW) & 15) && lddw % 4 == 0,
                "gemm_wgrad: dW must be 16-byte aligned with leading dimension % 4 == 0");
        const int splits = wgrad_splits((N / tile.bm) * (K / tile.bn), M / BK);
        if (splits == 1) {
            EpilogueF32 e{dW, lddw, 0, accumulate};
            dispatch_gemm<false, false>(stream, tile, dY, lddy, X, ldx, N, K, M, 1, e);
            return;
        }
        const size_t need = size_t(splits) * N * K * sizeof(float);
        require(workspace && workspace_bytes >= need && !(reinterpret_cast<uintptr_t>(workspace) & 15),
                "gemm_wgrad: workspace too small (see tgk_gemm_wgrad_workspace)");
        EpilogueF32 e{static_cast<float *>(workspace), K, size_t(N) * K, 0};
        dispatch_gemm<false, false>(stream, tile, dY, lddy, X, ldx, N, K, M, splits, e);
        const size_t quads = size_t(N) * K / 4;
        const int blocks = int((quads + 255) / 256 < 4096 ? (quads + 255) / 256 : 4096);
        hipLaunchKernelGGL(splitk_reduce_kernel, dim3(blocks), dim3(256), 0, stream,
                           static_cast<const float *>(workspace), size_t(N) * K, splits, dW, N, K, lddw,
                           accumulate);
        check_hip(hipGetLastError(), "split-K reduce launch: ");
    });
}
