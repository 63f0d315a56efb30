// bf16 matrix products on the gfx950 matrix cores: C[M,N] (+)= A[M,K] * W[N,K]^T with
// bf16 inputs, float accumulation, and a bf16 or float output.  W is a weight matrix as
// checkpoints store it ([out, in], row-major), so both operands are read along k.
//
// Kernels:
//  * gemm_stream: M <= 16 rows (decode): weight streaming by one resident workgroup per
//    compute unit, weights and activations brought into per-wave LDS rings by direct
//    global-to-LDS loads (described at the kernel).
//  * gemm_tile: LDS-staged tiles for many rows (prompts): 4 waves, each a TM x TN grid of
//    v_mfma_f32_32x32x16_bf16 blocks; global loads of the next k-tile are issued before the
//    current one is multiplied and written to the other LDS buffer after it.
//  * gemm_skinny: M <= 64 rows (decode): pure weight streaming.  A workgroup owns 16*RB
//    weight rows; its 4 waves take interleaved 128-element k-chunks, every lane reading
//    64 contiguous bytes of one weight row per chunk straight into v_mfma_f32_16x16x32_bf16
//    operands (the k-permutation inside a chunk is the same for both operands, so the dot
//    product is unchanged); the waves' partial sums are added in wave order in LDS.
//
// reference: op_linear_proj (GEMV per output row, kernels/megakernel_ops.hip:166-276) for
// what is computed; wmma_gemm_bf16 (kernels/wmma_gemm_bf16.hip:27-82, one wave32 per 16x16
// tile without LDS, used only by its tests) for the matrix-core form on RDNA3.
#include "common.h"

// output modes
#define OUT_BF16 0
#define OUT_F32 1
#define OUT_F32_ACC 2
// SwiGLU epilogue: W holds gate and up rows interleaved in blocks of 16 (8 gate rows, then
// the 8 up rows of the same outputs); the output is bf16 [M, N / 2] with
// out[m][8 b + j] = silu(gate) * up, silu(g) = g / (1 + exp(-g))
// (reference: kernels/megakernel_ops.hip:1538-1544, fused there too, per output row).
#define OUT_SWIGLU 3
#define SSQ_LD 64           // row stride of the sums of squares that a product leaves for the next RMS norm

__device__ __forceinline__ float silu_mul(float g, float u) { return g / (1.f + expf(-g)) * u; }

template <int MODE>
__device__ __forceinline__ void store_out(void* C, size_t idx, float v) {
    if (MODE == OUT_BF16) ((bf16*)C)[idx] = (bf16)v;
    else if (MODE == OUT_F32) ((float*)C)[idx] = v;
    else if (MODE == OUT_F32_ACC) ((float*)C)[idx] += v;
}

__device__ __forceinline__ bf16x8 zero8() {
    bf16x8 z;
#pragma unroll
    for (int i = 0; i < 8; ++i) z[i] = (bf16)0.f;
    return z;
}

// 8 consecutive bf16 of row `row` at k; zeros outside [0,rows) x [0,K).
template <bool ALIGNED>
__device__ __forceinline__ bf16x8 load8(const bf16* __restrict__ base, size_t ld, int row, int rows, int k, int K) {
    if (row >= rows || k >= K) return zero8();
    const bf16* p = base + (size_t)row * ld + k;
    if (ALIGNED) {
        if (k + 8 <= K) return *(const bf16x8*)p;
    }
    bf16x8 v;
#pragma unroll
    for (int i = 0; i < 8; ++i) v[i] = (k + i < K) ? p[i] : (bf16)0.f;
    return v;
}

// Store a wave's TM x TN grid of 32x32 accumulator blocks whose first element is (m1, n1).
// acc[i][j][r]: row = 8 (r / 4) + 4 (lane / 32) + r % 4, column = lane % 32 of the block.
template <int TM, int TN, int MODE>
__device__ __forceinline__ void tile_epilogue(f32x16 (&acc)[TM][TN], void* __restrict__ C, int M, int N, size_t ldc,
                                              int m1, int n1, int lane) {
#pragma unroll
    for (int i = 0; i < TM; ++i)
#pragma unroll
        for (int j = 0; j < TN; ++j) {
            const int n = n1 + j * 32 + (lane & 31);
            if (MODE == OUT_SWIGLU) {
                // the up value of a gate column sits 8 columns on, in lane ^ 8
#pragma unroll
                for (int r = 0; r < 16; ++r) {
                    const float other = __shfl_xor(acc[i][j][r], 8, 64);
                    const int m = m1 + i * 32 + 8 * (r >> 2) + 4 * (lane >> 5) + (r & 3);
                    if ((lane & 8) == 0 && n < N && m < M)
                        ((bf16*)C)[(size_t)m * ldc + (n >> 4) * 8 + (n & 7)] = (bf16)silu_mul(acc[i][j][r], other);
                }
                continue;
            }
            if (n >= N) continue;
            // one 64-bit address per block; the 16 rows of a lane are reached by 32-bit offsets
            const int mb = m1 + i * 32 + 4 * (lane >> 5);
            const size_t base = (size_t)mb * ldc + n;
            const unsigned ld32 = (unsigned)ldc;
#pragma unroll
            for (int r = 0; r < 16; ++r) {
                const int dm = 8 * (r >> 2) + (r & 3);
                if (mb + dm < M) store_out<MODE>(C, base + (size_t)(dm * ld32), acc[i][j][r]);
            }
            // keep the blocks' stores apart: moving every accumulator out of the matrix-core
            // registers at once would not fit the register file of the large tiles
            __builtin_amdgcn_sched_barrier(0);
        }
}

// ------------------------------------------------------------------ gemm_tile -------
template <int BM, int BN, int BK, int WAVES_M, int WAVES_N, int MODE, bool ALIGNED, bool KFULL>
__global__ __launch_bounds__(256) void gemm_tile_kernel(const bf16* __restrict__ A, const bf16* __restrict__ W,
                                                        void* __restrict__ C, int M, int N, int K,
                                                        size_t lda, size_t ldc, int tiles_m, int tiles_n) {
    static_assert(WAVES_M * WAVES_N == 4, "4 waves");
    constexpr int WM = BM / WAVES_M, WN = BN / WAVES_N;      // per-wave tile
    constexpr int TM = WM / 32, TN = WN / 32;
    constexpr int LDS_LD = BK + 8;                           // padded row, in bf16
    constexpr int A_CHUNKS = BM * BK / 8 / 256, B_CHUNKS = BN * BK / 8 / 256;
    constexpr int CPR = BK / 8;                              // 16-byte chunks per tile row
    extern __shared__ __attribute__((aligned(16))) unsigned char smem[];
    bf16* As = (bf16*)smem;                                  // [2][BM][LDS_LD]
    bf16* Bs = As + 2 * BM * LDS_LD;                         // [2][BN][LDS_LD]

    // Workgroups are dealt round-robin to the 8 XCDs; give each XCD a contiguous run of
    // tiles (n-major, m inner) so that the workgroups sharing an L2 share weight tiles.
    const int total = tiles_m * tiles_n;
    int pid = blockIdx.x;
    {
        const int per = total / 8, xcd = pid % 8, idx = pid / 8;
        if (pid < per * 8) pid = xcd * per + idx;
    }
    const int tile_n = pid / tiles_m, tile_m = pid - tile_n * tiles_m;
    const int m0 = tile_m * BM, n0 = tile_n * BN;

    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int wm = (wave / WAVES_N) * WM, wn = (wave % WAVES_N) * WN;
    const int lrow = lane & 31, lk = (lane >> 5) * 8;

    f32x16 acc[TM][TN];
#pragma unroll
    for (int i = 0; i < TM; ++i)
#pragma unroll
        for (int j = 0; j < TN; ++j)
#pragma unroll
            for (int r = 0; r < 16; ++r) acc[i][j][r] = 0.f;

    // Rows beyond M or N are read from the last valid row (and dropped at the store), so a
    // load needs a guard along k only; with K a multiple of BK and 16-byte aligned rows
    // (KFULL) it needs none.
    bf16x8 ra[A_CHUNKS], rb[B_CHUNKS];
    const bf16* ap[A_CHUNKS];
    const bf16* bp[B_CHUNKS];
    int akc[A_CHUNKS], bkc[B_CHUNKS];
#pragma unroll
    for (int c = 0; c < A_CHUNKS; ++c) {
        const int id = tid + c * 256;
        int r = m0 + id / CPR;
        if (r > M - 1) r = M - 1;
        akc[c] = (id % CPR) * 8;
        ap[c] = A + (size_t)r * lda + akc[c];
    }
#pragma unroll
    for (int c = 0; c < B_CHUNKS; ++c) {
        const int id = tid + c * 256;
        int r = n0 + id / CPR;
        if (r > N - 1) r = N - 1;
        bkc[c] = (id % CPR) * 8;
        bp[c] = W + (size_t)r * K + bkc[c];
    }
    auto gload = [&](int k0) {
#pragma unroll
        for (int c = 0; c < A_CHUNKS; ++c) {
            if (KFULL) ra[c] = *(const bf16x8*)(ap[c] + k0);
            else ra[c] = load8<ALIGNED>(ap[c] - akc[c], 0, 0, 1, k0 + akc[c], K);
        }
#pragma unroll
        for (int c = 0; c < B_CHUNKS; ++c) {
            if (KFULL) rb[c] = *(const bf16x8*)(bp[c] + k0);
            else rb[c] = load8<ALIGNED>(bp[c] - bkc[c], 0, 0, 1, k0 + bkc[c], K);
        }
    };
    auto sstore = [&](int buf) {
        bf16* a = As + buf * BM * LDS_LD;
        bf16* b = Bs + buf * BN * LDS_LD;
#pragma unroll
        for (int c = 0; c < A_CHUNKS; ++c) {
            const int id = tid + c * 256, r = id / CPR, kc = (id % CPR) * 8;
            *(bf16x8*)(a + r * LDS_LD + kc) = ra[c];
        }
#pragma unroll
        for (int c = 0; c < B_CHUNKS; ++c) {
            const int id = tid + c * 256, r = id / CPR, kc = (id % CPR) * 8;
            *(bf16x8*)(b + r * LDS_LD + kc) = rb[c];
        }
    };

    const int nk = (K + BK - 1) / BK;
    gload(0);
    sstore(0);
    __syncthreads();
    for (int kt = 0; kt < nk; ++kt) {
        const int buf = kt & 1;
        if (kt + 1 < nk) gload((kt + 1) * BK);
        const bf16* a = As + buf * BM * LDS_LD + (wm + lrow) * LDS_LD + lk;
        const bf16* b = Bs + buf * BN * LDS_LD + (wn + lrow) * LDS_LD + lk;
#pragma unroll
        for (int kk = 0; kk < BK; kk += 16) {
            bf16x8 fa[TM], fb[TN];
#pragma unroll
            for (int i = 0; i < TM; ++i) fa[i] = *(const bf16x8*)(a + i * 32 * LDS_LD + kk);
#pragma unroll
            for (int j = 0; j < TN; ++j) fb[j] = *(const bf16x8*)(b + j * 32 * LDS_LD + kk);
#pragma unroll
            for (int i = 0; i < TM; ++i)
#pragma unroll
                for (int j = 0; j < TN; ++j)
                    acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(fa[i], fb[j], acc[i][j], 0, 0, 0);
        }
        if (kt + 1 < nk) sstore(buf ^ 1);
        __syncthreads();
    }

    tile_epilogue<TM, TN, MODE>(acc, C, M, N, ldc, m0 + wm, n0 + wn, lane);
}

template <int BM, int BN, int BK, int WAVES_M, int WAVES_N>
static int launch_tile(const bf16* A, const bf16* W, void* C, int M, int N, int K, size_t lda, size_t ldc,
                       int mode, bool aligned, hipStream_t s) {
    const int tm = (M + BM - 1) / BM, tn = (N + BN - 1) / BN;
    const long long total = (long long)tm * tn;
    if (total > 0x7fffffffLL) return BR_BAD_ARG;
    const size_t lds = (size_t)2 * (BM + BN) * (BK + 8) * sizeof(bf16);
#define BR_LAUNCH_TILE_(MODE, AL, KF)                                                                    \
    do {                                                                                                \
        auto kern = gemm_tile_kernel<BM, BN, BK, WAVES_M, WAVES_N, MODE, AL, KF>;                       \
        if (lds > 48 * 1024) {                                                                          \
            static bool set = false;                                                                    \
            if (!set) {                                                                                 \
                if (hipFuncSetAttribute((const void*)kern, hipFuncAttributeMaxDynamicSharedMemorySize,  \
                                        (int)lds) != hipSuccess) return BR_LAUNCH_FAILED;               \
                set = true;                                                                             \
            }                                                                                           \
        }                                                                                               \
        kern<<<(unsigned)total, 256, lds, s>>>(A, W, C, M, N, K, lda, ldc, tm, tn);                     \
    } while (0)
#define BR_LAUNCH_TILE(MODE)                                                 \
    do {                                                                     \
        if (aligned && K % BK == 0) BR_LAUNCH_TILE_(MODE, true, true);       \
        else if (aligned) BR_LAUNCH_TILE_(MODE, true, false);                \
        else BR_LAUNCH_TILE_(MODE, false, false);                            \
    } while (0)
    if (mode == OUT_BF16) BR_LAUNCH_TILE(OUT_BF16);
    else if (mode == OUT_F32) BR_LAUNCH_TILE(OUT_F32);
    else if (mode == OUT_F32_ACC) BR_LAUNCH_TILE(OUT_F32_ACC);
    else BR_LAUNCH_TILE(OUT_SWIGLU);
#undef BR_LAUNCH_TILE_
#undef BR_LAUNCH_TILE
    return br_check_launch();
}

// -------------------------------------------------------------- gemm_tile_dma -------
// The tile product for aligned shapes (K a multiple of 64, 16-byte aligned rows): tiles
// go from memory to LDS by direct global-to-LDS loads (global_load_lds_dwordx4: a wave
// writes 1 KB = 8 tile rows of 64 k, no registers, no ds_write), into a ring of S stages.
// A row's eight 16-byte columns are stored XOR-swizzled by (row / 2) % 8, which makes the
// operand reads of 16 consecutive rows conflict-free; the swizzle is applied by choosing
// the global column each lane fetches.  Rows beyond M or N are fetched from the last
// valid row and dropped at the store.
//
// The loads are issued from inline assembly and counted by hand: before a stage is
// read, `s_waitcnt vmcnt(n)` leaves only the younger stages' loads outstanding, then a
// barrier makes every wave's part of the stage visible (and says that the stage about to
// be overwritten has been read by all).  The kernel issues no other vector memory
// operation inside the loop, so the count is exact.
// Weight layouts (`wl`).  0: N rows of K.  1: blocks of 16 rows x 128 k, 4 KB contiguous each, ordered
// [row block][k block], rows padded to a multiple of 16 (K in steps of 128): a 16-row strip is one
// contiguous run along k.  A streaming product then reads 4 KB pieces, in order, instead of 256 bytes
// from every row, which the memory serves faster (bare loads of a 64-row tile by every workgroup: 5.4 to
// 5.9 against 4.1 to 4.6 TB/s; in the products: wide matrices at 17 to 128 rows gain 10 to 15 %, up to
// 16 rows 0 to 5 %, the rest nothing).  Blocks of 64 rows were tried: slower up to 16 rows.
#define WL_ROWS 0
#define WL_BLOCKED 1
#ifndef WL_BLOCK_ROWS
#define WL_BLOCK_ROWS 16
#endif
#define WL_BLOCK_ELEMS (WL_BLOCK_ROWS * 128)
__device__ __forceinline__ size_t w_row_base(int n, int K, int wl) {
    return wl ? (size_t)(n / WL_BLOCK_ROWS) * (size_t)(K >> 7) * WL_BLOCK_ELEMS + (size_t)((n % WL_BLOCK_ROWS) << 7)
              : (size_t)n * K;
}
#define DMA_BK 64
#define DMA_ISSUE(ST, kt)                                                                                      \
    do {                                                                                                       \
        _Pragma("unroll") for (int q = 0; q < INSTR; ++q) {                                                    \
            const unsigned lds_ = __builtin_amdgcn_readfirstlane(                                              \
                (unsigned)(size_t)((__attribute__((address_space(3))) unsigned char*)(ST)) + dst[q]);          \
            if (once[q])                                   /* weights that no other row of tiles reads */      \
                asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, off nt" ::"s"(lds_), "v"(src[q]) \
                             : "m0");                                                                          \
            else                                                                                               \
                asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, off" ::"s"(lds_), "v"(src[q]) \
                             : "m0");                                                                          \
            src[q] += (knext & 1) ? hop[q] : DMA_BK;       /* k-tiles are issued in order, (kt) is the next */ \
        }                                                                                                      \
        if (++knext == kwrap) {                            /* on to the run's first k-tile */                  \
            knext = kt0;                                                                                       \
            _Pragma("unroll") for (int q = 0; q < INSTR; ++q) src[q] -= (size_t)(nk_run >> 1) * (DMA_BK + hop[q]); \
        }                                                                                                      \
    } while (0)
#define DMA_COMPUTE(ST)                                                                                        \
    do {                                                                                                       \
        _Pragma("unroll") for (int kk = 0; kk < 4; ++kk) {                                                     \
            bf16x8 fa[TM], fb[TN];                                                                             \
            const int c = kk * 2 + g;                                                                          \
            _Pragma("unroll") for (int i = 0; i < TM; ++i) {                                                   \
                const int r = wm + i * 32 + lrow;                                                              \
                fa[i] = *(const bf16x8*)((ST) + r * 128 + ((c ^ ((r >> 1) & 7)) * 16));                        \
            }                                                                                                  \
            _Pragma("unroll") for (int j = 0; j < TN; ++j) {                                                   \
                const int r = BM + wn + j * 32 + lrow;                                                         \
                fb[j] = *(const bf16x8*)((ST) + r * 128 + ((c ^ ((r >> 1) & 7)) * 16));                        \
            }                                                                                                  \
            _Pragma("unroll") for (int i = 0; i < TM; ++i)                                                     \
                _Pragma("unroll") for (int j = 0; j < TN; ++j)                                                 \
                    acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(fa[i], fb[j], acc[i][j], 0, 0, 0);     \
        }                                                                                                      \
    } while (0)
#define DMA_WAITBAR(N)                                              \
    do {                                                            \
        asm volatile("s_waitcnt vmcnt(%0)" ::"n"(N) : "memory");    \
        __builtin_amdgcn_s_barrier();                               \
        asm volatile("" ::: "memory");                              \
    } while (0)

template <int BM, int BN, int WAVES_M, int WAVES_N, int S, int MODE>
__global__ __launch_bounds__(64 * WAVES_M * WAVES_N) void gemm_tile_dma_kernel(
    const bf16* __restrict__ A, const bf16* __restrict__ W, void* __restrict__ C_, int M, int N, int K, size_t lda,
    size_t ldc, int tiles_m, int tiles_n, int kt_per_part, size_t part_stride, int wl) {
    constexpr int NW = WAVES_M * WAVES_N;
    constexpr int WM = BM / WAVES_M, WN = BN / WAVES_N, TM = WM / 32, TN = WN / 32;
    constexpr int STAGE_BYTES = (BM + BN) * DMA_BK * 2;
    // blockIdx.y: which run of k-tiles this workgroup sums (one run, or the parts of a split
    // product, each into a float matrix of its own `part_stride` elements on)
    void* C = MODE == OUT_F32 ? (void*)((float*)C_ + blockIdx.y * part_stride) : C_;
    constexpr int INSTR = (BM + BN) / 8 / NW;           // 1 KB wave-loads per wave and stage
    static_assert(S == 2 || S == 3, "2 or 3 stages");
    __shared__ __attribute__((aligned(1024))) unsigned char st0[STAGE_BYTES];
    __shared__ __attribute__((aligned(1024))) unsigned char st1[STAGE_BYTES];
    __shared__ __attribute__((aligned(1024))) unsigned char st2[S >= 3 ? STAGE_BYTES : 16];

    // each XCD takes a contiguous run of tiles, in groups of 8 tile columns by all tile rows
    const int total = tiles_m * tiles_n;
    int pid = blockIdx.x;
    {
        const int per = total / 8, xcd = pid % 8, idx = pid / 8;
        if (pid < per * 8) pid = xcd * per + idx;
    }
    const int grp = pid / (8 * tiles_m), in = pid - grp * 8 * tiles_m;
    int gn = tiles_n - grp * 8;
    if (gn > 8) gn = 8;
    const int tile_n = grp * 8 + in % gn, tile_m = in / gn;
    const int m0 = tile_m * BM, n0 = tile_n * BN;
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int wm = (wave / WAVES_N) * WM, wn = (wave % WAVES_N) * WN;
    const int lrow = lane & 31, g = lane >> 5;

    f32x16 acc[TM][TN];
#pragma unroll
    for (int i = 0; i < TM; ++i)
#pragma unroll
        for (int j = 0; j < TN; ++j)
#pragma unroll
            for (int r = 0; r < 16; ++r) acc[i][j][r] = 0.f;

    // wave-load q of this wave covers rows (q NW + wave) 8 .. + 8 of the stacked tile [A rows | W rows]
    const bf16* src[INSTR];
    int dst[INSTR];
    int hop[INSTR];                                      // elements from an odd k-tile to the next (even) one
    bool once[INSTR];                                    // a load of weight rows that are read this once (non-temporal)
    const int kt0 = (int)blockIdx.y * kt_per_part;       // the run's first k-tile
    int nk_run = K / DMA_BK - kt0;                       // k-tiles of this run
    if (nk_run > kt_per_part) nk_run = kt_per_part;
    // Where in its run a workgroup starts (it wraps round): workgroups that walk k in step ask the same few
    // memory channels at the same time.  Only with a single row of tiles (3 to 6 % on wide matrices at
    // 65 to 128 rows): workgroups that share a tile live on reading the same k-tile at the same time (a start
    // of its own for each made 2,048 rows 50 % slower, one per tile column made 2 rows of tiles 5 to 12 %
    // slower).  An even start in an even run, so that pairs of k-tiles (one 128-wide block of the blocked
    // layout) stay together.
    const int rot = (tiles_m == 1 && nk_run % 2 == 0 && kt0 % 2 == 0)
                        ? 2 * (int)((((unsigned)tile_n * 2654435761u) >> 8) % (unsigned)(nk_run / 2)) : 0;
    const int kwrap = kt0 + nk_run;
    int knext = kt0 + rot;                               // the k-tile that src[] points at
#pragma unroll
    for (int q = 0; q < INSTR; ++q) {
        const int R = (q * NW + wave) * 8 + (lane >> 3);
        const int c = (lane & 7) ^ ((R >> 1) & 7);       // the global 16-byte column this lane fetches
        if (R < BM) {
            int r = m0 + R;
            if (r > M - 1) r = M - 1;
            src[q] = A + (size_t)r * lda + c * 8 + (size_t)(kt0 + rot) * DMA_BK;
            hop[q] = DMA_BK;
        } else {
            int r = n0 + R - BM;
            if (r > N - 1) r = N - 1;
            src[q] = W + w_row_base(r, K, wl) + c * 8 +
                     (wl ? (size_t)((kt0 + rot) >> 1) * WL_BLOCK_ELEMS + (kt0 & 1) * DMA_BK : (size_t)(kt0 + rot) * DMA_BK);
            hop[q] = wl ? WL_BLOCK_ELEMS - DMA_BK : DMA_BK;
        }
        hop[q] = __builtin_amdgcn_readfirstlane(hop[q]);             // the same for the 8 rows of a wave-load
        once[q] = __builtin_amdgcn_readfirstlane((int)((q * NW + wave) * 8 >= BM && tiles_m == 1)) != 0;
        dst[q] = (q * NW + wave) * 1024;
    }
    const int nk = nk_run;
    if (S == 2) {
        DMA_ISSUE(st0, 0);
        for (int kt = 0; kt < nk; kt += 2) {
            DMA_WAITBAR(0);
            if (kt + 1 < nk) DMA_ISSUE(st1, kt + 1);
            DMA_COMPUTE(st0);
            if (kt + 1 >= nk) break;
            DMA_WAITBAR(0);
            if (kt + 2 < nk) DMA_ISSUE(st0, kt + 2);
            DMA_COMPUTE(st1);
        }
    } else {
        DMA_ISSUE(st0, 0);
        if (nk > 1) DMA_ISSUE(st1, 1);
        int kt = 0;
        // steady state: two stages are in flight at every wait, the older one is waited for
        for (; kt + 5 <= nk; kt += 3) {
            DMA_WAITBAR(INSTR);
            DMA_ISSUE(st2, kt + 2);
            DMA_COMPUTE(st0);
            DMA_WAITBAR(INSTR);
            DMA_ISSUE(st0, kt + 3);
            DMA_COMPUTE(st1);
            DMA_WAITBAR(INSTR);
            DMA_ISSUE(st1, kt + 4);
            DMA_COMPUTE(st2);
        }
        // the last tiles: wait for everything in flight
        for (; kt < nk; kt += 3) {
            DMA_WAITBAR(0);
            if (kt + 2 < nk) DMA_ISSUE(st2, kt + 2);
            DMA_COMPUTE(st0);
            if (kt + 1 >= nk) break;
            DMA_WAITBAR(0);
            if (kt + 3 < nk) DMA_ISSUE(st0, kt + 3);
            DMA_COMPUTE(st1);
            if (kt + 2 >= nk) break;
            DMA_WAITBAR(0);
            if (kt + 4 < nk) DMA_ISSUE(st1, kt + 4);
            DMA_COMPUTE(st2);
        }
    }
    tile_epilogue<TM, TN, MODE>(acc, C, M, N, ldc, m0 + wm, n0 + wn, lane);
}

// ------------------------------------------------------------ gemm_tile_quad -------
// A BM x BN tile by four waves (2 x 2, or 4 x 1 for the 256x224 tile), one to a SIMD, each summing a quarter of it in the matrix-core
// registers (256x256: 16 blocks of 32x32, all 256 of them), with the operands of one k-step of 16 in
// vector registers, twice (the set in use and the set being read from LDS).  Per matrix instruction
// half the LDS operand bytes of the 64x64 wave tiles above.  With one wave per SIMD nothing fills a gap
// in that wave's instruction stream, so the order is written out: matrix instructions, LDS reads,
// direct loads and waits are inline assembly in program order.  The compiler keeps volatile statements
// in order, but it neither knows their latencies nor that they are matrix instructions: every wait is
// placed by hand, and so are the idle states that the hardware wants between a register's write and
// a matrix instruction's read of it (and the reverse).
// Each operand has a ring of two or three stages of 64 k (the layout and swizzle of gemm_tile_dma).  One
// barrier per k-tile, before its last k-step of 16: by then every wave has read the stages in use.  An
// operand with two stages is asked for after that barrier, into the stage just read; one with three
// during the k-steps before it, into the stage that the barrier before freed: a compute unit's path into
// LDS takes one 1 KB load per 16 cycles, so a k-tile's loads are spread over it, not bunched (bunched,
// the waves wait at their load instructions with the matrix cores idle behind them).
// The blocks hold the product transposed (weight rows are the instruction's first operand), which
// gives every lane four neighbouring columns of one output row: 16-byte accesses in the epilogue, and
// the up value of a gate column in the same lane.
typedef int i32x4 __attribute__((ext_vector_type(4)));
template <int I, int N_, class F>
__device__ __forceinline__ void static_for(F&& f) {
    if constexpr (I < N_) {
        f(std::integral_constant<int, I>{});
        static_for<I + 1, N_>(f);
    }
}
template <int OFF>
__device__ __forceinline__ void quad_read(i32x4& d, unsigned addr) {
    asm volatile("ds_read_b128 %0, %1 offset:%2" : "=v"(d) : "v"(addr), "n"(OFF));
}
template <int IMM>
__device__ __forceinline__ void quad_load(unsigned lds_base, unsigned voff, unsigned long long sbase) {
    asm volatile("s_add_u32 m0, %0, %1\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %2, %3"
                 ::"s"(lds_base), "n"(IMM), "v"(voff), "s"(sbase)
                 : "m0", "scc", "memory");
}
__device__ __forceinline__ void quad_mfma(f32x16& acc, const i32x4& a, const i32x4& b) {
    asm volatile("v_mfma_f32_32x32x16_bf16 %0, %1, %2, %0" : "+a"(acc) : "v"(a), "v"(b));
}
__device__ __forceinline__ void quad_touch(f32x16& acc) { asm volatile("s_nop 1" : "+a"(acc)); }
template <int N_>
__device__ __forceinline__ void quad_wait_loads() {
    asm volatile("s_waitcnt vmcnt(%0)" ::"n"(N_) : "memory");
}

// acc[i][j][r]: weight row (output column) n1 + 32 i + 8 (r / 4) + 4 (lane / 32) + r % 4, activation
// row m1 + 32 j + lane % 32.  Needs ldc % 4 == 0 and C aligned to 16 bytes.
template <int TI, int TJ, int MODE>
__device__ __forceinline__ void quad_epilogue(f32x16 (&acc)[TI][TJ], void* __restrict__ C, int M, int N, size_t ldc,
                                              int m1, int n1, int lane) {
    typedef float f32x4 __attribute__((ext_vector_type(4)));
    typedef __bf16 bf16x4 __attribute__((ext_vector_type(4)));
#pragma unroll
    for (int j = 0; j < TJ; ++j) {
        const int m = m1 + j * 32 + (lane & 31);
        if (m >= M) continue;
#pragma unroll
        for (int i = 0; i < TI; ++i) {
            const int nb = n1 + i * 32 + 4 * (lane >> 5);
            if (MODE == OUT_SWIGLU) {
#pragma unroll
                for (int h = 0; h < 2; ++h) {
                    const int n = nb + 16 * h;                      // gate columns n .. n + 3, N a multiple of 16
                    if (n >= N) continue;
                    bf16x4 v;
#pragma unroll
                    for (int e = 0; e < 4; ++e) v[e] = (bf16)silu_mul(acc[i][j][8 * h + e], acc[i][j][8 * h + 4 + e]);
                    *(bf16x4*)((bf16*)C + (size_t)m * ldc + (n >> 4) * 8 + (n & 7)) = v;
                }
                continue;
            }
#pragma unroll
            for (int q = 0; q < 4; ++q) {
                const int n = nb + 8 * q;
                const size_t at = (size_t)m * ldc + n;
                if (n + 3 < N) {
                    if (MODE == OUT_BF16) {
                        bf16x4 v;
#pragma unroll
                        for (int e = 0; e < 4; ++e) v[e] = (bf16)acc[i][j][4 * q + e];
                        *(bf16x4*)((bf16*)C + at) = v;
                    } else {
                        f32x4 v;
                        if (MODE == OUT_F32_ACC) v = *(const f32x4*)((float*)C + at);
#pragma unroll
                        for (int e = 0; e < 4; ++e) v[e] = (MODE == OUT_F32_ACC ? v[e] : 0.f) + acc[i][j][4 * q + e];
                        *(f32x4*)((float*)C + at) = v;
                    }
                } else {
#pragma unroll
                    for (int e = 0; e < 4; ++e)
                        if (n + e < N) store_out<MODE>(C, at + e, acc[i][j][4 * q + e]);
                }
            }
        }
    }
}

template <int BM, int BN, int NSA, int NSB, int WVM, int MODE>
__global__ __launch_bounds__(256) void gemm_tile_quad_kernel(const bf16* __restrict__ A, const bf16* __restrict__ W,
                                                              void* __restrict__ C_, int M, int N, int K, size_t lda,
                                                              size_t ldc, int tiles_m, int tiles_n, int kt_per_part,
                                                              size_t part_stride, int wl) {
    constexpr int SA = BM * 128, SB = BN * 128;          // bytes of a stage of activation rows, of weight rows
    constexpr int WVN = 4 / WVM;                         // the four waves: WVM along the activation rows x WVN
    constexpr int TI = BN / WVN / 32, TJ = BM / WVM / 32; // blocks of a wave: weight rows, activation rows
    constexpr int NM = TI * TJ;                          // matrix instructions per k-step of 16
    constexpr int LA = BM / 32, LB = BN / 32;            // wave-loads per wave and stage
    // An operand with three stages is asked for during the first three k-steps of 16 of a k-tile, into the
    // stage that the barrier before freed, and has a whole k-tile more to arrive; one with two stages after
    // the barrier, into the stage just read.  Either way k-tile t asks for k-tile t + 2.
    constexpr bool EARLY_A = NSA == 3, EARLY_B = NSB == 3;
    constexpr int NEARLY = (EARLY_A ? LA : 0) + (EARLY_B ? LB : 0), NLATE = LA + LB - NEARLY;
    static_assert((WVM == 2 || WVM == 4) && BM % (32 * WVM) == 0 && BN % (32 * WVN) == 0 && BM % 32 == 0 && BN % 32 == 0 &&
                      NSA * SA + NSB * SB <= 160 * 1024 && TI * TJ * 16 <= 256, "tile");
    static_assert((NSA == 2 || NSA == 3) && (NSB == 2 || NSB == 3), "two or three stages an operand");
    static_assert(TI + TJ <= NM && NLATE <= 2 * NM, "schedule");
    __shared__ __attribute__((aligned(1024))) unsigned char st[NSA * SA + NSB * SB];
    // blockIdx.y: which run of k-tiles this workgroup sums (one run, or the parts of a split product, each
    // into a float matrix of its own `part_stride` elements on; runs start at an even k-tile)
    void* C = MODE == OUT_F32 ? (void*)((float*)C_ + blockIdx.y * part_stride) : C_;
    const int kt0 = (int)blockIdx.y * kt_per_part;
    const int total = tiles_m * tiles_n;
    int pid = blockIdx.x;
    {
        const int per = total / 8, xcd = pid % 8, idx = pid / 8;
        if (pid < per * 8) pid = xcd * per + idx;
    }
    const int grp = pid / (8 * tiles_m), in = pid - grp * 8 * tiles_m;
    int gn = tiles_n - grp * 8;
    if (gn > 8) gn = 8;
    const int tile_n = grp * 8 + in % gn, tile_m = in / gn;
    const int m0 = tile_m * BM, n0 = tile_n * BN;
    const int tid = threadIdx.x, lane = tid & 63, wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int wm = (wave / WVN) * (BM / WVM), wn = (wave % WVN) * (BN / WVN);
    const int lrow = lane & 31, g = lane >> 5;

    f32x16 acc[TI][TJ];
#pragma unroll
    for (int i = 0; i < TI; ++i)
#pragma unroll
        for (int j = 0; j < TJ; ++j)
#pragma unroll
            for (int r = 0; r < 16; ++r) acc[i][j][r] = 0.f;

    // wave-load q of this wave: rows (4 q + wave) 8 .. + 8 of the operand's tile, reached by a 32-bit byte
    // offset from the matrix's first element (the launcher checks that this suffices)
    unsigned offA[LA], offB[LB];
#pragma unroll
    for (int q = 0; q < (LA > LB ? LA : LB); ++q) {
        const int R = (q * 4 + wave) * 8 + (lane >> 3);
        const int c = (lane & 7) ^ ((R >> 1) & 7);
        if (q < LA) {
            int r = m0 + R;
            if (r > M - 1) r = M - 1;
            offA[q] = (unsigned)((size_t)r * lda * 2 + c * 16);
        }
        if (q < LB) {
            int r = n0 + R;
            if (r > N - 1) r = N - 1;
            offB[q] = (unsigned)(w_row_base(r, K, wl) * 2 + c * 16);
        }
    }
    // at the next k-tile to ask for
    unsigned long long baseA = (unsigned long long)A + (size_t)kt0 * 128;
    unsigned long long baseW = (unsigned long long)W + (wl ? (size_t)(kt0 >> 1) * (WL_BLOCK_ELEMS * 2) : (size_t)kt0 * 128);
    int knext = kt0;
    const unsigned hopW = wl ? WL_BLOCK_ELEMS * 2 - 128 : 128;                        // bytes from an odd k-tile on
    const unsigned lds0 = (unsigned)(size_t)((__attribute__((address_space(3))) unsigned char*)st);
    // where this wave's loads of the next k-tile to ask for land, and which stage that is
    unsigned ldsA = __builtin_amdgcn_readfirstlane(lds0 + wave * 1024);
    unsigned ldsB = __builtin_amdgcn_readfirstlane(lds0 + NSA * SA + wave * 1024);
    int slotA = 0, slotB = 0;
    // LDS addresses of this lane's operand pieces in the stage in use, per k-step of 16, and which stage that is
    unsigned ra[4], rb[4];
    int curA = 0, curB = 0;
#pragma unroll
    for (int kk = 0; kk < 4; ++kk) {
        const int col = ((kk * 2 + g) ^ ((lrow >> 1) & 7)) * 16;
        ra[kk] = lds0 + (wm + lrow) * 128 + col;
        rb[kk] = lds0 + NSA * SA + (wn + lrow) * 128 + col;
    }
    i32x4 fa[2][TJ], fb[2][TI];

    auto loadA = [&](auto q_) {
        constexpr int q = decltype(q_)::value;
        quad_load<q * 4096>(ldsA, offA[q], baseA);
    };
    auto loadB = [&](auto q_) {
        constexpr int q = decltype(q_)::value;
        quad_load<q * 4096>(ldsB, offB[q], baseW);
    };
    // the x-th early load (A's first where both operands are early), the x-th late load
    auto early = [&](auto x_) {
        constexpr int x = decltype(x_)::value;
        if constexpr (EARLY_A && x < LA) loadA(x_);
        else loadB(std::integral_constant<int, x - (EARLY_A ? LA : 0)>{});
    };
    auto late = [&](auto x_) {
        constexpr int x = decltype(x_)::value;
        if constexpr (!EARLY_A && x < LA) loadA(x_);
        else loadB(std::integral_constant<int, x - (!EARLY_A ? LA : 0)>{});
    };
    auto next_tile = [&]() {                       // the pointers and the stages to load go on by a k-tile
        baseA += 128;
        baseW += (knext & 1) ? hopW : 128;
        ++knext;
        ldsA += slotA == NSA - 1 ? (unsigned)(-(NSA - 1) * SA) : (unsigned)SA;
        slotA = slotA == NSA - 1 ? 0 : slotA + 1;
        ldsB += slotB == NSB - 1 ? (unsigned)(-(NSB - 1) * SB) : (unsigned)SB;
        slotB = slotB == NSB - 1 ? 0 : slotB + 1;
    };
    // One k-step of 16 from operand set `use`: NM matrix instructions, and between them the LDS reads of set
    // `use ^ 1` (k-step rk of the stage that ra/rb point into) and the direct loads [E0, E1) of the early
    // ones or [L0, L1) of the late ones, evenly.
    auto substep = [&](auto use_, auto rd_, auto rk_, auto e0_, auto e1_, auto l0_, auto l1_) {
        constexpr int use = decltype(use_)::value, rk = decltype(rk_)::value;
        constexpr bool RD = decltype(rd_)::value;
        constexpr int E0 = decltype(e0_)::value, E1 = decltype(e1_)::value, L0 = decltype(l0_)::value, L1 = decltype(l1_)::value;
        static_for<0, NM>([&](auto n_) {
            constexpr int n = decltype(n_)::value;
            // block (i, j): weight rows i (the instruction's first operand, so the result's rows), activation rows j
            constexpr int i = n / TJ, j = (i & 1) ? TJ - 1 - n % TJ : n % TJ;
            quad_mfma(acc[i][j], fb[use][i], fa[use][j]);
            if constexpr (RD && n < TJ) quad_read<n * 4096>(fa[use ^ 1][n], ra[rk]);
            if constexpr (RD && n >= TJ && n < TJ + TI) quad_read<(n - TJ) * 4096>(fb[use ^ 1][n - TJ], rb[rk]);
            static_for<E0 + n * (E1 - E0) / NM, E0 + (n + 1) * (E1 - E0) / NM>(early);
            static_for<L0 + n * (L1 - L0) / NM, L0 + (n + 1) * (L1 - L0) / NM>(late);
        });
        if constexpr (RD) asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
    };
    using T = std::true_type;
    using F = std::false_type;
    using I0 = std::integral_constant<int, 0>;
    using I1 = std::integral_constant<int, 1>;
    using I2 = std::integral_constant<int, 2>;
    using I3 = std::integral_constant<int, 3>;
    // One k-tile from the stages in use.  Not LAST: before its last k-step every wave waits for its own
    // loads of the next k-tile (the early ones of the one after may be on their way) and for the others at
    // a barrier, which also says that all have read these stages; then it reads the next k-tile's first
    // operands.  LOADS: it asks for the k-tile two on, the early loads before the barrier, the late ones after.
    auto step = [&](auto loads_, auto last_) {
        constexpr bool LOADS = decltype(loads_)::value, LAST = decltype(last_)::value;
        constexpr int NE = LOADS ? NEARLY : 0, NL = LOADS ? NLATE : 0;
        using Z = std::integral_constant<int, 0>;
        substep(I0{}, T{}, I1{}, Z{}, std::integral_constant<int, NE / 3>{}, Z{}, Z{});
        substep(I1{}, T{}, I2{}, std::integral_constant<int, NE / 3>{}, std::integral_constant<int, 2 * NE / 3>{}, Z{}, Z{});
        substep(I0{}, T{}, I3{}, std::integral_constant<int, 2 * NE / 3>{}, std::integral_constant<int, NE>{}, Z{}, Z{});
        if constexpr (LAST) {
            substep(I1{}, F{}, I0{}, Z{}, Z{}, Z{}, Z{});
        } else {
            quad_wait_loads<NE>();
            __builtin_amdgcn_s_barrier();
            asm volatile("" ::: "memory");
            const unsigned da = curA == NSA - 1 ? (unsigned)(-(NSA - 1) * SA) : (unsigned)SA;
            const unsigned db = curB == NSB - 1 ? (unsigned)(-(NSB - 1) * SB) : (unsigned)SB;
#pragma unroll
            for (int kk = 0; kk < 4; ++kk) {                           // reads: the next stages
                ra[kk] += da;
                rb[kk] += db;
            }
            curA = curA == NSA - 1 ? 0 : curA + 1;
            curB = curB == NSB - 1 ? 0 : curB + 1;
            substep(I1{}, T{}, I0{}, Z{}, Z{}, Z{}, std::integral_constant<int, NL>{});
            if constexpr (LOADS) next_tile();
        }
    };

    int nk = K / DMA_BK - kt0;                                         // k-tiles of this run
    if (nk > kt_per_part) nk = kt_per_part;
    static_for<0, LA>(loadA);                                          // the first two k-tiles
    static_for<0, LB>(loadB);
    next_tile();
    if (nk > 1) {
        static_for<0, LA>(loadA);
        static_for<0, LB>(loadB);
        next_tile();
        quad_wait_loads<LA + LB>();
    } else {
        quad_wait_loads<0>();
    }
    __builtin_amdgcn_s_barrier();
    asm volatile("" ::: "memory");
    static_for<0, TJ>([&](auto n_) { quad_read<decltype(n_)::value * 4096>(fa[0][decltype(n_)::value], ra[0]); });
    static_for<0, TI>([&](auto n_) { quad_read<decltype(n_)::value * 4096>(fb[0][decltype(n_)::value], rb[0]); });
    asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
    // Statements that name the accumulators: what the compiler wrote into one (the zeroes) is written before
    // its statement, and a matrix instruction must not read a register in the states right after its write.
    static_for<0, NM>([&](auto n_) { quad_touch(acc[decltype(n_)::value / TJ][decltype(n_)::value % TJ]); });
    int t = 0;
    for (; t + 2 < nk; ++t) step(T{}, F{});
    for (; t + 1 < nk; ++t) step(F{}, F{});
    step(F{}, T{});
    // the last matrix instructions' results are not in their registers yet; the epilogue's reads of an
    // accumulator stay behind the statement that names it
    asm volatile("s_nop 15\n\ts_nop 15" ::: "memory");
    static_for<0, NM>([&](auto n_) { quad_touch(acc[decltype(n_)::value / TJ][decltype(n_)::value % TJ]); });
    quad_epilogue<TI, TJ, MODE>(acc, C, M, N, ldc, m0 + wm, n0 + wn, lane);
}

static int launch_split_sum(const float* scratch, int parts, void* C, int M, int N, size_t ldc, int mode, hipStream_t s);

// What the quad tiles ask of a product beyond K % 64 == 0 and aligned rows: the loads reach a row by a
// 32-bit byte offset from the matrix's first element, and the epilogue stores 16 bytes at a time.
static bool quad_takes(const void* C, int M, int N, int K, size_t lda, size_t ldc) {
    return (unsigned long long)M * lda * 2 < (1ull << 32) && ((unsigned long long)N + 16) * K * 2 < (1ull << 32) &&
           ldc % 4 == 0 && (uintptr_t)C % 16 == 0;
}

// parts > 1: the k-tiles are cut into runs of an even number of k-tiles, every (tile, run) workgroup writes
// its float sums to a matrix of its own in `scratch`, and gemm_split_sum_kernel adds the runs in run order
// and applies the epilogue.
#ifndef QUAD12
#define QUAD12 2, 3
#endif
#ifndef QUAD13
#define QUAD13 3, 3
#endif
#ifndef QUAD14
#define QUAD14 2, 3
#endif
template <int BM, int BN, int NSA, int NSB, int WVM = 2>
static int launch_tile_quad(const bf16* A, const bf16* W, void* C, int M, int N, int K, size_t lda, size_t ldc,
                            int mode, hipStream_t s, int wl, int parts = 1, float* scratch = nullptr) {
    const int tm = (M + BM - 1) / BM, tn = (N + BN - 1) / BN;
    const long long total = (long long)tm * tn;
    if (total > 0x7fffffffLL || !quad_takes(C, M, N, K, lda, ldc)) return BR_BAD_ARG;
    const int nk = K / DMA_BK;
    if (parts > 1) {
        if (N % 4 != 0 || (uintptr_t)scratch % 16 != 0) return BR_BAD_ARG;
        int kpp = (nk + parts - 1) / parts;
        kpp += kpp & 1;
        parts = (nk + kpp - 1) / kpp;                                 // no empty run
        dim3 grid((unsigned)total, (unsigned)parts);
        gemm_tile_quad_kernel<BM, BN, NSA, NSB, WVM, OUT_F32><<<grid, 256, 0, s>>>(A, W, scratch, M, N, K, lda, (size_t)N, tm, tn, kpp,
                                                                        (size_t)M * N, wl);
        int rc = br_check_launch();
        if (rc != BR_OK) return rc;
        return launch_split_sum(scratch, parts, C, M, N, ldc, mode, s);
    }
    if (mode == OUT_BF16)
        gemm_tile_quad_kernel<BM, BN, NSA, NSB, WVM, OUT_BF16><<<(unsigned)total, 256, 0, s>>>(A, W, C, M, N, K, lda, ldc, tm, tn, nk, 0, wl);
    else if (mode == OUT_F32)
        gemm_tile_quad_kernel<BM, BN, NSA, NSB, WVM, OUT_F32><<<(unsigned)total, 256, 0, s>>>(A, W, C, M, N, K, lda, ldc, tm, tn, nk, 0, wl);
    else if (mode == OUT_F32_ACC)
        gemm_tile_quad_kernel<BM, BN, NSA, NSB, WVM, OUT_F32_ACC><<<(unsigned)total, 256, 0, s>>>(A, W, C, M, N, K, lda, ldc, tm, tn, nk, 0, wl);
    else
        gemm_tile_quad_kernel<BM, BN, NSA, NSB, WVM, OUT_SWIGLU><<<(unsigned)total, 256, 0, s>>>(A, W, C, M, N, K, lda, ldc, tm, tn, nk, 0, wl);
    return br_check_launch();
}

// Which quad tile (12: 256x256, 13: 128x256, 14: 256x192, 15: 256x224, whose 128 tile columns over 28,672
// weight rows make whole rounds where 112 of 256 do not) and how many runs of k-tiles: the least time by a
// count in microseconds.  A k-tile takes 1.50, 0.85, 1.20 and 1.39 us with every compute unit at work and 1.08,
// 0.80, 0.92 and 1.00 us with few (measured; in between, the cube of the share at work fits: at half the chip
// the tiles hardly feel each other yet); whole rounds of workgroups over the chip, then the rest of them,
// which after whole rounds take nearly what a whole round takes (2,048 x 28,672 by 896 tiles of 256x256,
// three and a half rounds: 390 us, the half round 1.41 us a k-tile); plus what a launch costs besides and,
// when split along k, the second launch and the traffic of the partial sums.  Returns the count.
static const double QUAD_FULL[4] = {1.50, 0.85, 1.20, 1.39}, QUAD_FEW[4] = {1.08, 0.80, 0.92, 1.00};
static double choose_quad(int M, int N, int K, int mode, int cus, size_t scratch_bytes, int* kernel, int* parts) {
    const int nk = K / DMA_BK;
    static const int bm[4] = {256, 128, 256, 256}, bn[4] = {256, 256, 192, 224};
    double best = 1e30;
    *kernel = 13;
    *parts = 1;
    for (int k = 0; k < 4; ++k) {
        const long long tiles = (long long)((M + bm[k] - 1) / bm[k]) * ((N + bn[k] - 1) / bn[k]);
        for (int p = 1; p <= 16; p *= 2) {
            if (p > 1 && (p * 4 > nk || N % 4 != 0 || (size_t)p * M * N * sizeof(float) > scratch_bytes)) break;
            int kpp = (nk + p - 1) / p;
            kpp += kpp & 1;
            const long long units = tiles * p, whole = units / cus;
            const double share = (double)(units % cus) / cus;
            const double rest = units % cus == 0 ? 0.0
                                : whole        ? QUAD_FULL[k] * (0.9 + 0.1 * share)
                                               : QUAD_FEW[k] + (QUAD_FULL[k] - QUAD_FEW[k]) * share * share * share;
            double t = kpp * ((double)whole * QUAD_FULL[k] + rest) + (mode == OUT_BF16 ? 8.0 : 12.0);
            if (p > 1) t += 5.0 + (double)p * M * N * 8.0 / 4e6;
            if (t < best - 1e-9) { best = t; *kernel = 12 + k; *parts = p; }
        }
    }
    return best;
}

// Weight rows that the 256x256 tile covers in whole rounds of workgroups over the chip, where the count says that
// these rounds and the best tile for the rest (`kernel`, `parts`, chosen over N - n1 weight rows) take less than
// the best single tile over all rows (`single`); 0 where not.  n1 is a multiple of 256.
static int quad_whole_rounds(int M, int N, int K, int mode, int cus, size_t scratch_bytes, double single, int* kernel,
                             int* parts) {
    const int tm = (M + 255) / 256, nk = K / DMA_BK;
    const int cols = cus / tm;                                        // tile columns of one round
    if (cols < 1) return 0;
    const long long rounds = (long long)(N / 256) / cols, n1 = rounds * cols * 256;
    if (rounds < 1 || n1 >= N || (mode == OUT_SWIGLU && (N - n1) % 16 != 0)) return 0;
    const long long used = (long long)tm * cols;                      // workgroups of such a round
    const double share = (double)used / cus;
    const double per = used == cus ? QUAD_FULL[0] : QUAD_FEW[0] + (QUAD_FULL[0] - QUAD_FEW[0]) * share * share * share;
    int k2, p2;
    const double t = (double)rounds * nk * per + (mode == OUT_BF16 ? 8.0 : 12.0) +
                     choose_quad(M, (int)(N - n1), K, mode, cus, scratch_bytes, &k2, &p2);
    if (t >= 0.97 * single) return 0;
    *kernel = k2;
    *parts = p2;
    return (int)n1;
}

// parts > 1: the k-tiles are cut into `parts` runs, every (tile, run) workgroup writes its
// float sums to a matrix of its own in `scratch`, and gemm_split_sum_kernel adds the runs in
// run order and applies the epilogue (for products with too few tiles to fill the chip).
template <int BM, int BN, int WAVES_M, int WAVES_N, int S>
static int launch_tile_dma(const bf16* A, const bf16* W, void* C, int M, int N, int K, size_t lda, size_t ldc,
                           int mode, hipStream_t s, int parts = 1, float* scratch = nullptr, int wl = 0) {
    const int tm = (M + BM - 1) / BM, tn = (N + BN - 1) / BN;
    const long long total = (long long)tm * tn;
    if (total > 0x7fffffffLL) return BR_BAD_ARG;
    constexpr int NT = 64 * WAVES_M * WAVES_N;
    const int nk = K / DMA_BK;
    if (parts > 1) {
        const int kpp = (nk + parts - 1) / parts;
        parts = (nk + kpp - 1) / kpp;                                 // no empty run
        dim3 grid((unsigned)total, (unsigned)parts);
        gemm_tile_dma_kernel<BM, BN, WAVES_M, WAVES_N, S, OUT_F32><<<grid, NT, 0, s>>>(
            A, W, scratch, M, N, K, lda, (size_t)N, tm, tn, kpp, (size_t)M * N, wl);
        int rc = br_check_launch();
        if (rc != BR_OK) return rc;
        return launch_split_sum(scratch, parts, C, M, N, ldc, mode, s);
    }
    if (mode == OUT_BF16)
        gemm_tile_dma_kernel<BM, BN, WAVES_M, WAVES_N, S, OUT_BF16><<<(unsigned)total, NT, 0, s>>>(A, W, C, M, N, K, lda, ldc, tm, tn, nk, 0, wl);
    else if (mode == OUT_F32)
        gemm_tile_dma_kernel<BM, BN, WAVES_M, WAVES_N, S, OUT_F32><<<(unsigned)total, NT, 0, s>>>(A, W, C, M, N, K, lda, ldc, tm, tn, nk, 0, wl);
    else if (mode == OUT_F32_ACC)
        gemm_tile_dma_kernel<BM, BN, WAVES_M, WAVES_N, S, OUT_F32_ACC><<<(unsigned)total, NT, 0, s>>>(A, W, C, M, N, K, lda, ldc, tm, tn, nk, 0, wl);
    else
        gemm_tile_dma_kernel<BM, BN, WAVES_M, WAVES_N, S, OUT_SWIGLU><<<(unsigned)total, NT, 0, s>>>(A, W, C, M, N, K, lda, ldc, tm, tn, nk, 0, wl);
    return br_check_launch();
}

// Which direct-to-LDS tile (5: 128x256, one workgroup per CU; 6: 128x128, two; 10: 256x192, one, two
// stages, not split) and how many runs of k-tiles for a product of more than 64 rows: the least time by
// a rough count in microseconds (rounds of workgroups over the chip times k-tiles times 1.0-1.7 us a
// k-tile, plus, when split, a launch and the traffic of the partial sums), runs of at least 4 k-tiles
// that fit the scratch memory.  The 256x192 tile is there for shapes that it covers in fewer rounds:
// 2,048 x 6,144 is 256 of them, one round, against 384 tiles of 128x256 (measured 103-118 against
// 129-134 us); with equal rounds it loses (two stages, 1.5 times the work a k-tile for 1.5 times the time).
static void choose_tile(int M, int N, int K, int mode, int cus, size_t scratch_bytes, int* kernel, int* parts) {
    const int nk = K / DMA_BK;
    double best = 1e30;
    *kernel = 5;
    *parts = 1;
    {
        const long long tiles = (long long)((M + 255) / 256) * ((N + 191) / 192);
        const double t = (double)((tiles + cus - 1) / cus) * nk * 1.72;
        if (tiles > cus / 2) { best = t; *kernel = 10; }             // with fewer tiles a split product fills the chip better
    }
    if (mode == OUT_SWIGLU) {
        // 256x256, SwiGLU epilogue only (the other epilogues run out of registers around its 128 accumulators a
        // wave): 8 % faster than 128x256 where its rounds fit (4,096 x 28,672: 920 against 1,000 us)
        const long long tiles = (long long)((M + 255) / 256) * ((N + 255) / 256);
        const double t = (double)((tiles + cus - 1) / cus) * nk * 2.1;
        if (tiles > cus / 2 && t < best - 1e-9) { best = t; *kernel = 11; }
    }
    for (int k = 5; k <= 6; ++k) {
        const long long tiles = (long long)((M + 127) / 128) * ((N + (k == 5 ? 255 : 127)) / (k == 5 ? 256 : 128));
        const long long slots = (long long)cus * (k == 5 ? 1 : 2);
        for (int p = 1; p <= 16; p *= 2) {
            if (p > 1 && (p * 4 > nk || (size_t)p * M * N * sizeof(float) > scratch_bytes)) break;
            const long long units = tiles * p, rounds = (units + slots - 1) / slots;
            const int kpp = (nk + p - 1) / p;
            const double per = k == 5 ? 1.14 : (units > cus ? 1.33 : 1.0);
            double t = (double)rounds * kpp * per;
            if (p > 1) t += 5.0 + (double)p * M * N * 8.0 / 4e6;
            if (t < best - 1e-9) { best = t; *kernel = k; *parts = p; }
        }
    }
}

// ----------------------------------------------------------------- gemm_skinny ------
// grid = ceil(N / (16 RB)); block = 64 NW.  Needs K % 8 == 0 and 16-byte aligned rows.
// Every wave keeps U chunks of 128 k in flight (the loads of all U are issued before the
// first product), which is what fills the memory pipeline; rows beyond N or M are read
// from the last valid row instead of being masked, and dropped at the store.
template <int MB, int RB, int U, int NW, int MODE>
__global__ __launch_bounds__(NW * 64) void gemm_skinny_kernel(const bf16* __restrict__ A, const bf16* __restrict__ W,
                                                              void* __restrict__ C, int M, int N, int K,
                                                              size_t lda, size_t ldc) {
    constexpr int ROWS = 16 * RB, COLS = 16 * MB;
    __shared__ float red[NW][ROWS][COLS + 1];
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int r16 = lane & 15, g = lane >> 4;
    const int n0 = blockIdx.x * ROWS;

    f32x4 acc[RB][MB];
#pragma unroll
    for (int i = 0; i < RB; ++i)
#pragma unroll
        for (int j = 0; j < MB; ++j)
#pragma unroll
            for (int r = 0; r < 4; ++r) acc[i][j][r] = 0.f;
    const bf16* wp[RB];
    const bf16* xp[MB];
#pragma unroll
    for (int i = 0; i < RB; ++i) {
        int row = n0 + i * 16 + r16;
        if (row > N - 1) row = N - 1;
        wp[i] = W + (size_t)row * K + g * 8;
    }
#pragma unroll
    for (int j = 0; j < MB; ++j) {
        int row = j * 16 + r16;
        if (row > M - 1) row = M - 1;
        xp[j] = A + (size_t)row * lda + g * 8;
    }
    // lane (row r16, group g) holds k = chunk * 128 + s * 32 + g * 8 + [0, 8) for s = 0..3
    const int nfull = K / 128;
    int c = wave * U;
    for (; c + U <= nfull; c += NW * U) {
        bf16x8 fw[U][RB][4], fx[U][MB][4];
#pragma unroll
        for (int u = 0; u < U; ++u) {
            const int kb = (c + u) * 128;
#pragma unroll
            for (int i = 0; i < RB; ++i)
#pragma unroll
                for (int s = 0; s < 4; ++s) fw[u][i][s] = *(const bf16x8*)(wp[i] + kb + s * 32);
#pragma unroll
            for (int j = 0; j < MB; ++j)
#pragma unroll
                for (int s = 0; s < 4; ++s) fx[u][j][s] = *(const bf16x8*)(xp[j] + kb + s * 32);
        }
#pragma unroll
        for (int u = 0; u < U; ++u)
#pragma unroll
            for (int s = 0; s < 4; ++s)
#pragma unroll
                for (int i = 0; i < RB; ++i)
#pragma unroll
                    for (int j = 0; j < MB; ++j)
                        acc[i][j] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(fw[u][i][s], fx[u][j][s], acc[i][j], 0, 0, 0);
    }
    // this wave's leftover chunks (fewer than U, or the partial last chunk), guarded along k
    const int nch = (K + 127) / 128;
    for (int u = 0; u < U; ++u) {
        const int cc = c + u;
        if (cc >= nch) break;
        const int kb = cc * 128;
#pragma unroll
        for (int s = 0; s < 4; ++s) {
            const bool in = kb + s * 32 + g * 8 + 8 <= K;
#pragma unroll
            for (int i = 0; i < RB; ++i) {
                const bf16x8 a = in ? *(const bf16x8*)(wp[i] + kb + s * 32) : zero8();
#pragma unroll
                for (int j = 0; j < MB; ++j) {
                    const bf16x8 b = in ? *(const bf16x8*)(xp[j] + kb + s * 32) : zero8();
                    acc[i][j] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a, b, acc[i][j], 0, 0, 0);
                }
            }
        }
    }
    // acc[i][j][r]: weight row = 16 i + 4 (lane / 16) + r, batch row = 16 j + lane % 16
#pragma unroll
    for (int i = 0; i < RB; ++i)
#pragma unroll
        for (int j = 0; j < MB; ++j)
#pragma unroll
            for (int r = 0; r < 4; ++r) red[wave][i * 16 + 4 * g + r][j * 16 + r16] = acc[i][j][r];
    __syncthreads();
    if (MODE == OUT_SWIGLU) {
        for (int e = tid; e < (ROWS / 2) * COLS; e += NW * 64) {
            const int m = e / (ROWS / 2), jl = e - m * (ROWS / 2);
            const int gl = (jl >> 3) * 16 + (jl & 7);            // gate row in the tile; its up row is 8 on
            if (m < M && n0 + gl + 8 < N) {
                float gv = 0.f, uv = 0.f;
#pragma unroll
                for (int w = 0; w < NW; ++w) { gv += red[w][gl][m]; uv += red[w][gl + 8][m]; }
                ((bf16*)C)[(size_t)m * ldc + n0 / 2 + jl] = (bf16)silu_mul(gv, uv);
            }
        }
        return;
    }
    for (int e = tid; e < ROWS * COLS; e += NW * 64) {
        const int m = e / ROWS, nl = e - m * ROWS;   // consecutive threads: consecutive weight rows
        const int n = n0 + nl;
        if (m < M && n < N) {
            float v = 0.f;
#pragma unroll
            for (int w = 0; w < NW; ++w) v += red[w][nl][m];     // in wave order, always
            store_out<MODE>(C, (size_t)m * ldc + n, v);
        }
    }
}

template <int MB, int RB, int U, int NW>
static int launch_skinny(const bf16* A, const bf16* W, void* C, int M, int N, int K, size_t lda, size_t ldc,
                         int mode, hipStream_t s) {
    const unsigned grid = (unsigned)((N + 16 * RB - 1) / (16 * RB));
    if (mode == OUT_BF16)
        gemm_skinny_kernel<MB, RB, U, NW, OUT_BF16><<<grid, NW * 64, 0, s>>>(A, W, C, M, N, K, lda, ldc);
    else if (mode == OUT_SWIGLU)
        gemm_skinny_kernel<MB, RB, U, NW, OUT_SWIGLU><<<grid, NW * 64, 0, s>>>(A, W, C, M, N, K, lda, ldc);
    else if (mode == OUT_F32)
        gemm_skinny_kernel<MB, RB, U, NW, OUT_F32><<<grid, NW * 64, 0, s>>>(A, W, C, M, N, K, lda, ldc);
    else
        gemm_skinny_kernel<MB, RB, U, NW, OUT_F32_ACC><<<grid, NW * 64, 0, s>>>(A, W, C, M, N, K, lda, ldc);
    return br_check_launch();
}

// ------------------------------------------------------------- gemm_skinny_lds ------
// 16 < M <= 64: the activations of a 512-wide k-slab are staged in LDS once per workgroup
// with direct global-to-LDS loads (one 1 KB row per wave-load, no registers), because at
// these M the activation fragments, not the weights, dominate the load instructions.
// A row's 16-byte columns are stored XOR-swizzled by the row number, so that the 16 rows
// an operand read touches fall into different banks; the swizzle is applied by choosing
// which global column each lane fetches.  Weights stream from memory into the operands
// as in gemm_skinny; the 4 waves split the slab's k and are added in wave order.
#define SLAB_K 512
template <int MB, int RB, int MODE>
__global__ __launch_bounds__(256) void gemm_skinny_lds_kernel(const bf16* __restrict__ A, const bf16* __restrict__ W,
                                                              void* __restrict__ C_, int M, int N, int K,
                                                              size_t lda, size_t ldc, int slabs_per_part,
                                                              size_t part_stride) {
    constexpr int ROWS = 16 * RB, COLS = 16 * MB;
    constexpr int SLAB_BYTES = COLS * SLAB_K * 2;
    constexpr int RED_BYTES = 4 * ROWS * (COLS + 1) * 4;
    __shared__ __attribute__((aligned(1024))) unsigned char smem[SLAB_BYTES > RED_BYTES ? SLAB_BYTES : RED_BYTES];
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int r16 = lane & 15, g = lane >> 4;
    const int n0 = blockIdx.x * ROWS;
    f32x4 acc[RB][MB];
#pragma unroll
    for (int i = 0; i < RB; ++i)
#pragma unroll
        for (int j = 0; j < MB; ++j)
#pragma unroll
            for (int r = 0; r < 4; ++r) acc[i][j][r] = 0.f;
    const bf16* wp[RB];
#pragma unroll
    for (int i = 0; i < RB; ++i) {
        int row = n0 + i * 16 + r16;
        if (row > N - 1) row = N - 1;
        wp[i] = W + (size_t)row * K + wave * 128 + g * 8;
    }
    // blockIdx.y: which run of k-slabs this workgroup sums (one run, or the parts of a split
    // product, each into its own float matrix `part_stride` elements on)
    const int nslab = (K + SLAB_K - 1) / SLAB_K;
    const int sl0 = blockIdx.y * slabs_per_part;
    const int sl1 = sl0 + slabs_per_part < nslab ? sl0 + slabs_per_part : nslab;
    void* C = MODE == OUT_F32 ? (void*)((float*)C_ + blockIdx.y * part_stride) : C_;
    for (int sl = sl0; sl < sl1; ++sl) {
        const int k0 = sl * SLAB_K;
        bf16x8 fw[RB][4];                                  // this wave's weight fragments of the slab
#pragma unroll
        for (int i = 0; i < RB; ++i)
#pragma unroll
            for (int s = 0; s < 4; ++s) {
                const int k = k0 + wave * 128 + s * 32 + g * 8;
                fw[i][s] = (k + 8 <= K) ? *(const bf16x8*)(wp[i] + k0 + s * 32) : zero8();
            }
#pragma unroll
        for (int rr = 0; rr < COLS / 4; ++rr) {
            const int row = rr * 4 + wave;                 // slab row = batch row; lane l fetches column l ^ (row & 15)
            int grow = row;
            if (grow > M - 1) grow = M - 1;
            int kk = k0 + ((lane ^ (row & 15)) * 8);
            if (kk + 8 > K) kk = 0;                        // never multiplied: the weight fragment there is zero
            __builtin_amdgcn_global_load_lds((const __attribute__((address_space(1))) void*)(A + (size_t)grow * lda + kk),
                                             (__attribute__((address_space(3))) void*)(smem + row * 1024), 16, 0, 0);
        }
        __syncthreads();
#pragma unroll
        for (int s = 0; s < 4; ++s) {
            const int c = wave * 16 + s * 4 + g;
#pragma unroll
            for (int j = 0; j < MB; ++j) {
                const bf16x8 fx = *(const bf16x8*)(smem + (j * 16 + r16) * 1024 + ((c ^ r16) * 16));
#pragma unroll
                for (int i = 0; i < RB; ++i)
                    acc[i][j] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(fw[i][s], fx, acc[i][j], 0, 0, 0);
            }
        }
        __syncthreads();
    }
    float (*red)[ROWS][COLS + 1] = (float (*)[ROWS][COLS + 1])smem;
#pragma unroll
    for (int i = 0; i < RB; ++i)
#pragma unroll
        for (int j = 0; j < MB; ++j)
#pragma unroll
            for (int r = 0; r < 4; ++r) red[wave][i * 16 + 4 * g + r][j * 16 + r16] = acc[i][j][r];
    __syncthreads();
    if (MODE == OUT_SWIGLU) {
        for (int e = tid; e < (ROWS / 2) * COLS; e += 256) {
            const int m = e / (ROWS / 2), jl = e - m * (ROWS / 2);
            const int gl = (jl >> 3) * 16 + (jl & 7);
            if (m < M && n0 + gl + 8 < N) {
                float gv = 0.f, uv = 0.f;
#pragma unroll
                for (int w = 0; w < 4; ++w) { gv += red[w][gl][m]; uv += red[w][gl + 8][m]; }
                ((bf16*)C)[(size_t)m * ldc + n0 / 2 + jl] = (bf16)silu_mul(gv, uv);
            }
        }
        return;
    }
    for (int e = tid; e < ROWS * COLS; e += 256) {
        const int m = e / ROWS, nl = e - m * ROWS;
        const int n = n0 + nl;
        if (m < M && n < N) {
            float v = 0.f;
#pragma unroll
            for (int w = 0; w < 4; ++w) v += red[w][nl][m];
            store_out<MODE>(C, (size_t)m * ldc + n, v);
        }
    }
}

template <int MB, int RB>
static int launch_skinny_lds(const bf16* A, const bf16* W, void* C, int M, int N, int K, size_t lda, size_t ldc,
                             int mode, hipStream_t s) {
    const unsigned grid = (unsigned)((N + 16 * RB - 1) / (16 * RB));
    const int nslab = (K + SLAB_K - 1) / SLAB_K;
    if (mode == OUT_BF16) gemm_skinny_lds_kernel<MB, RB, OUT_BF16><<<grid, 256, 0, s>>>(A, W, C, M, N, K, lda, ldc, nslab, 0);
    else if (mode == OUT_F32) gemm_skinny_lds_kernel<MB, RB, OUT_F32><<<grid, 256, 0, s>>>(A, W, C, M, N, K, lda, ldc, nslab, 0);
    else if (mode == OUT_F32_ACC) gemm_skinny_lds_kernel<MB, RB, OUT_F32_ACC><<<grid, 256, 0, s>>>(A, W, C, M, N, K, lda, ldc, nslab, 0);
    else gemm_skinny_lds_kernel<MB, RB, OUT_SWIGLU><<<grid, 256, 0, s>>>(A, W, C, M, N, K, lda, ldc, nslab, 0);
    return br_check_launch();
}

// ---------------------------------------------------------------- split product ------
// 16 < M <= 64 and so few weight rows that 64-row workgroups would leave most of the chip
// idle (N = 4096: 64 of them): the k-slabs are cut into `parts` runs, every (tile, run)
// workgroup writes its sums to a float matrix of its own in `scratch`, and a second kernel
// adds the runs in run order and applies the epilogue.  Nothing is added atomically: the
// result does not depend on which workgroup finishes first.
template <int MODE>
__global__ void gemm_split_sum_kernel(const float* __restrict__ part, int parts, size_t part_stride, void* __restrict__ C,
                                      int M, int N, size_t ldc) {
    const size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (MODE == OUT_SWIGLU) {
        // output j of a row: gate column 16 (j / 8) + j % 8, its up value 8 columns on
        const size_t half = (size_t)N / 2;
        if (i >= (size_t)M * half) return;
        const size_t m = i / half, j = i - m * half;
        const size_t gc = m * N + (j >> 3) * 16 + (j & 7);
        float gv = 0.f, uv = 0.f;
        for (int p = 0; p < parts; ++p) { gv += part[p * part_stride + gc]; uv += part[p * part_stride + gc + 8]; }
        ((bf16*)C)[m * ldc + j] = (bf16)silu_mul(gv, uv);
        return;
    }
    if (i >= (size_t)M * N) return;
    float v = 0.f;
    for (int p = 0; p < parts; ++p) v += part[p * part_stride + i];
    const size_t m = i / N, n = i - m * N;
    store_out<MODE>(C, m * ldc + n, v);
}

// The sum of the runs added into the residual rows C, with the next RMS norm prepared as by
// gemm_stream's NORM = 1 form: a workgroup takes 256 consecutive columns of one row (N in
// steps of 256), writes h = C + sum back, bf16(h * gain) to xg, and the sum of its 256
// squares to ssq[(column / 256) * SSQ_LD + row].
__global__ __launch_bounds__(256) void gemm_split_sum_prep_kernel(const float* __restrict__ part, int parts,
                                                                  size_t part_stride, float* __restrict__ C, int N,
                                                                  size_t ldc, const float* __restrict__ gain,
                                                                  bf16* __restrict__ xg, size_t ldx,
                                                                  float* __restrict__ ssq) {
    __shared__ float red[16];
    const size_t i = (size_t)blockIdx.x * 256 + threadIdx.x;
    const size_t m = i / N, n = i - m * N;
    float v = 0.f;
    for (int p = 0; p < parts; ++p) v += part[p * part_stride + i];
    const float h = C[m * ldc + n] + v;
    C[m * ldc + n] = h;
    xg[m * ldx + n] = (bf16)(h * gain[n]);
    const float tot = block_sum(h * h, red);
    if (threadIdx.x == 0) ssq[(n / 256) * SSQ_LD + m] = tot;
}

static int launch_split_sum(const float* scratch, int parts, void* C, int M, int N, size_t ldc, int mode, hipStream_t s) {
    const size_t stride = (size_t)M * N;
    const unsigned blocks = (unsigned)((stride + 255) / 256);
    if (mode == OUT_BF16) gemm_split_sum_kernel<OUT_BF16><<<blocks, 256, 0, s>>>(scratch, parts, stride, C, M, N, ldc);
    else if (mode == OUT_F32) gemm_split_sum_kernel<OUT_F32><<<blocks, 256, 0, s>>>(scratch, parts, stride, C, M, N, ldc);
    else if (mode == OUT_F32_ACC) gemm_split_sum_kernel<OUT_F32_ACC><<<blocks, 256, 0, s>>>(scratch, parts, stride, C, M, N, ldc);
    else gemm_split_sum_kernel<OUT_SWIGLU><<<blocks, 256, 0, s>>>(scratch, parts, stride, C, M, N, ldc);
    return br_check_launch();
}

template <int MB>
static int launch_split(const bf16* A, const bf16* W, void* C, int M, int N, int K, size_t lda, size_t ldc, int mode,
                        int parts, float* scratch, hipStream_t s) {
    constexpr int RB = 4;
    const int nslab = (K + SLAB_K - 1) / SLAB_K;
    const int spp = (nslab + parts - 1) / parts;
    parts = (nslab + spp - 1) / spp;                                   // no empty run
    const size_t stride = (size_t)M * N;
    dim3 grid((unsigned)((N + 16 * RB - 1) / (16 * RB)), (unsigned)parts);
    gemm_skinny_lds_kernel<MB, RB, OUT_F32><<<grid, 256, 0, s>>>(A, W, scratch, M, N, K, lda, (size_t)N, spp, stride);
    int rc = br_check_launch();
    if (rc != BR_OK) return rc;
    return launch_split_sum(scratch, parts, C, M, N, ldc, mode, s);
}

// How many runs of k-slabs a product of 16 < M <= 64 rows is cut into when the caller gives
// scratch memory: enough (tile, run) workgroups of 64 weight rows for the chip, at least two
// slabs a run; 1 = not split.
static int split_parts(int M, int N, int K, int mode, size_t scratch_bytes) {
    if (M <= 16 || M > 64 || mode == OUT_SWIGLU) return 1;
    const int tiles = (N + 63) / 64, nslab = (K + SLAB_K - 1) / SLAB_K;
    int parts = 256 / tiles;
    if (parts > nslab / 2) parts = nslab / 2;
    if (parts > 8) parts = 8;
    if (parts < 2 || (size_t)parts * M * N * sizeof(float) > scratch_bytes) return 1;
    return parts;
}

// ------------------------------------------------------------------ gemm_stream ------
// M <= 16, K in steps of 128: weight streaming by workgroups that stay.  One workgroup per
// compute unit walks over tiles of 16 weight rows (tile t of workgroup b is b + t * grid);
// its 8 waves take the tile's 128-wide k-chunks in turn.  A wave brings a chunk of the
// tile (16 rows x 256 bytes) and the same chunk of the activations (8 or 16 rows) into a
// ring of LDS stages of its own with direct global-to-LDS loads: whole 256-byte row
// pieces per request, no registers, and the loads of the next chunk (of the next tile,
// at a tile's end) are in flight while this one is multiplied.  No wave waits for another
// inside a tile; at a tile's end the waves' sums meet in LDS (one barrier, two buffers)
// and are added in wave order.  The 16-byte columns of a row are XOR-swizzled by the row
// number through the choice of the global column a lane fetches.
//
// Two forms serve the RMS norm between a product that adds into the residual stream and the
// product that reads the normed rows, so that single-token steps launch no norm kernel
// (reference: op_rmsnorm, kernels/megakernel_ops.hip:1421-1446, a step of its own there):
//  * NORM = 1, the producer (with the accumulate epilogue): it reads the element it adds to,
//    writes the sum h back, writes bf16(h * g) (g: the next norm's weights) to `xg`, and the
//    sum of h^2 over its tile's 16 columns to ssq[tile * SSQ_LD + row].
//  * NORM = 2, the consumer: its activations are those bf16(h * g) rows; before its first
//    tile it adds the `ssq_tiles` sums of every row in a fixed order, and 1 / rms, the same
//    for a whole row, multiplies the sums at a tile's end:
//    y = rsqrt(mean(h^2) + eps) * sum_k W[n,k] (h[k] g[k]).
struct StreamNorm {
    const float* gain;     // producer: the next norm's weights [N]
    bf16* xg;              // producer: [M, ldx]
    size_t ldx;
    float* ssq;            // producer writes, consumer reads: [tiles, SSQ_LD]
    int ssq_tiles;         // consumer: tiles of the producer
    float inv_k, eps;      // consumer: 1 / width of the normed rows, the norm's eps
};

template <int RT, int XR, int KC, int S, int NW, int MODE, int NORM>
__global__ __launch_bounds__(NW * 64) void gemm_stream_kernel(const bf16* __restrict__ A, const bf16* __restrict__ W,
                                                              void* __restrict__ C, int M, int N, int K, size_t lda,
                                                              size_t ldc, int ntiles, StreamNorm nrm, int wl) {
    static_assert(NORM == 0 || (NORM == 1 && MODE == OUT_F32_ACC) || (NORM == 2 && MODE != OUT_F32_ACC), "norm forms");
    constexpr int STEPS = KC / 32;
    constexpr int ROWB = KC * 2;
    constexpr int STAGE = (RT + XR) * ROWB;
    constexpr int WDMA = RT * ROWB / 1024;
    constexpr int NDMA = STAGE / 1024;
    constexpr int CPL = ROWB / 16;          // 16-byte columns per row
    constexpr int RPI = 64 / CPL;           // rows per DMA instruction
    constexpr int LPI = NDMA;
    constexpr int D = S - 1;
    static_assert(RPI >= 1 && (D - 1) * LPI <= 63, "wait count");
    extern __shared__ __attribute__((aligned(1024))) unsigned char smem[];
    float* red = (float*)(smem + NW * S * STAGE);       // [2][NW][16][17]
    float* rstd = red + 2 * NW * 16 * 17;               // NORM 2: [16]
    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int r16 = lane & 15, g = lane >> 4;
    unsigned char* ring = smem + wave * (S * STAGE);
    const unsigned ring_lds = (unsigned)(size_t)((__attribute__((address_space(3))) unsigned char*)ring);

    const int nch = K / KC;
    const int ncw = (nch - wave + NW - 1) / NW;
    // Where in k this workgroup starts: workgroups that walk their rows in step ask the same few memory
    // channels at the same time; a start of its own for each spreads them (measured: 4 to 9 % on the
    // products of 4,096 to 6,144 weight rows).  The order of a column's sum depends on the column only.
    const int rot = (int)(((unsigned)blockIdx.x * 2654435761u) >> 8) % nch;
    const int my_tiles = (ntiles - (int)blockIdx.x + (int)gridDim.x - 1) / (int)gridDim.x;
    const int nitems = my_tiles * ncw;

    // DMA lane mapping
    const int drow = lane / CPL, dcol = lane % CPL;
    const int wstep = wl ? WL_BLOCK_ELEMS : KC;        // elements from a chunk of a weight row to the next
    f32x4 acc = {0.f, 0.f, 0.f, 0.f}, acc1 = {0.f, 0.f, 0.f, 0.f};

    int is_t = 0, is_c = 0;      // issue cursor: local tile index, local chunk index
    int cp_t = 0, cp_c = 0;      // compute cursor
    int buf = 0;

#define ISSUE(J)                                                                                         \
    do {                                                                                                 \
        int chunk_ = wave + is_c * NW + rot;                                                             \
        if (chunk_ >= nch) chunk_ -= nch;                                                                \
        const int n0_ = ((int)blockIdx.x + is_t * (int)gridDim.x) * RT;                                  \
        _Pragma("unroll") for (int q_ = 0; q_ < NDMA; ++q_) {                                            \
            const int row_ = q_ * RPI + drow;                                                            \
            const bf16* gp_;                                                                             \
            if (q_ < WDMA) {                                                                             \
                int nrow_ = n0_ + row_;                                                                  \
                if (nrow_ > N - 1) nrow_ = N - 1;                                                        \
                gp_ = W + w_row_base(nrow_, K, wl) + (size_t)chunk_ * wstep + ((dcol ^ (row_ & 7)) * 8);  \
            } else {                                                                                     \
                int m_ = row_ - RT;                                                                      \
                if (m_ > M - 1) m_ = M - 1;                                                              \
                gp_ = A + (size_t)m_ * lda + (size_t)chunk_ * KC + ((dcol ^ (row_ & 7)) * 8);            \
            }                                                                                            \
            const unsigned lds_ = __builtin_amdgcn_readfirstlane(ring_lds + (J) * STAGE + q_ * 1024);    \
            if (q_ < WDMA)                              /* weights pass once: non-temporal */            \
                asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, off nt" ::"s"(lds_), "v"(gp_) : "m0"); \
            else                                        /* activations are every workgroup's: they stay cached */ \
                asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, off" ::"s"(lds_), "v"(gp_) : "m0"); \
        }                                                                                                \
        if (++is_c == ncw) { is_c = 0; ++is_t; }                                                         \
    } while (0)

    // prologue
#pragma unroll
    for (int j = 0; j < D; ++j)
        if (j < nitems) ISSUE(j);
    // NORM 2: row m = tid / 32, its 32 lanes take the tiles' sums in turn.  The first eight a lane are requested
    // here and added at the first tile's end, so that their way from memory runs under the first tile.
    float ssq_pre[8];
    if constexpr (NORM == 2) {
        const int m = tid >> 5, l = tid & 31;
#pragma unroll
        for (int j = 0; j < 8; ++j)
            ssq_pre[j] = (m < M && l + 32 * j < nrm.ssq_tiles) ? nrm.ssq[(size_t)(l + 32 * j) * SSQ_LD + m] : 0.f;
    }

    for (int base = 0; base < nitems; base += S) {
#pragma unroll
        for (int j = 0; j < S; ++j) {
            const int it = base + j;
            if (it < nitems) {
                // wait for item `it`
                if (it + D - 1 < nitems) asm volatile("s_waitcnt vmcnt(%0)" ::"n"((D - 1) * LPI) : "memory");
                else asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
                if (it + D < nitems) ISSUE((j + D) % S);
                // compute
                const unsigned char* st = ring + j * STAGE;
                const int rr = RT == 8 ? (r16 & 7) : r16;
                const int xr = XR == 8 ? (r16 & 7) : r16;
                bf16x8 wf[STEPS], xv[STEPS];
#pragma unroll
                for (int s = 0; s < STEPS; ++s) {
                    wf[s] = *(const bf16x8*)(st + rr * ROWB + (((4 * s + g) ^ (rr & 7)) * 16));
                    xv[s] = *(const bf16x8*)(st + (RT + xr) * ROWB + (((4 * s + g) ^ (xr & 7)) * 16));
                }
#pragma unroll
                for (int s = 0; s < STEPS; s += 2) {
                    acc = __builtin_amdgcn_mfma_f32_16x16x32_bf16(wf[s], xv[s], acc, 0, 0, 0);
                    acc1 = __builtin_amdgcn_mfma_f32_16x16x32_bf16(wf[s + 1], xv[s + 1], acc1, 0, 0, 0);
                }
                if (++cp_c == ncw) {
                    cp_c = 0;
                    const int n0 = ((int)blockIdx.x + cp_t * (int)gridDim.x) * RT;
                    ++cp_t;
                    float* rb = red + buf * (NW * 16 * 17);
                    if (NORM == 2 && cp_t == 1) {
                        const int m = tid >> 5, l = tid & 31;
                        float t = 0.f;
#pragma unroll
                        for (int j = 0; j < 8; ++j) t += ssq_pre[j];
                        if (m < M)
                            for (int c = l + 256; c < nrm.ssq_tiles; c += 32) t += nrm.ssq[(size_t)c * SSQ_LD + m];
#pragma unroll
                        for (int o = 16; o > 0; o >>= 1) t += __shfl_xor(t, o, 64);
                        if (l == 0) rstd[m] = m < M ? rsqrtf(t * nrm.inv_k + nrm.eps) : 0.f;
                    }
#pragma unroll
                    for (int r = 0; r < 4; ++r) rb[(wave * 16 + 4 * g + r) * 17 + r16] = acc[r] + acc1[r];
                    acc = {0.f, 0.f, 0.f, 0.f};
                    acc1 = {0.f, 0.f, 0.f, 0.f};
                    asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
                    __builtin_amdgcn_s_barrier();
                    asm volatile("" ::: "memory");
                    if (MODE == OUT_SWIGLU) {
                        for (int e = tid; e < 8 * 16; e += NW * 64) {
                            const int m = e >> 3, jl = e & 7;
                            if (m < M && n0 + jl + 8 < N) {
                                float gv = 0.f, uv = 0.f;
#pragma unroll
                                for (int w = 0; w < NW; ++w) { gv += rb[(w * 16 + jl) * 17 + m]; uv += rb[(w * 16 + jl + 8) * 17 + m]; }
                                if (NORM == 2) { gv *= rstd[m]; uv *= rstd[m]; }
                                ((bf16*)C)[(size_t)m * ldc + n0 / 2 + jl] = (bf16)silu_mul(gv, uv);
                            }
                        }
                    } else if (NORM == 1) {
                        // whole waves (16 lanes a row): the row's 16 squares of this tile are added by shuffles
                        if (tid < 16 * XR) {
                            const int m = tid >> 4, nl = tid & 15, n = n0 + nl;
                            const bool ok = m < M && n < N;
                            float h = 0.f;
                            if (ok) {
                                float v = 0.f;
#pragma unroll
                                for (int w = 0; w < NW; ++w) v += rb[(w * 16 + nl) * 17 + m];
                                const size_t idx = (size_t)m * ldc + n;
                                h = ((float*)C)[idx] + v;
                                ((float*)C)[idx] = h;
                                nrm.xg[(size_t)m * nrm.ldx + n] = (bf16)(h * nrm.gain[n]);
                            }
                            float sq = h * h;
#pragma unroll
                            for (int o = 8; o > 0; o >>= 1) sq += __shfl_xor(sq, o, 64);
                            if (nl == 0 && m < M) nrm.ssq[(size_t)(n0 / 16) * SSQ_LD + m] = sq;
                        }
                    } else {
                        for (int e = tid; e < RT * 16; e += NW * 64) {
                            const int m = e / RT, nl = e % RT, n = n0 + nl;
                            if (m < M && n < N) {
                                float v = 0.f;
#pragma unroll
                                for (int w = 0; w < NW; ++w) v += rb[(w * 16 + nl) * 17 + m];
                                if (NORM == 2) v *= rstd[m];
                                const size_t idx = (size_t)m * ldc + n;
                                if (MODE == OUT_BF16) ((bf16*)C)[idx] = (bf16)v;
                                else if (MODE == OUT_F32) ((float*)C)[idx] = v;
                                // one add per element and product, without a read that this wave would
                                // have to wait for behind its loads in flight
                                else unsafeAtomicAdd((float*)C + idx, v);
                            }
                        }
                    }
                    buf ^= 1;
                }
            }
        }
    }
#undef ISSUE
}



#define STREAM_KC 128
#define STREAM_NW 8
template <int XR, int NORM>
static int launch_stream(const bf16* A, const bf16* W, void* C, int M, int N, int K, size_t lda, size_t ldc,
                         int mode, hipStream_t s, StreamNorm nrm = StreamNorm{}, int wl = 0) {
    constexpr int RT = 16, KC = STREAM_KC, S = 2, NW = STREAM_NW;
    static_assert(KC == 128, "the blocked weight layout has 128 k a block");
    const int cus = br_device_cus();
    if (!cus) return BR_LAUNCH_FAILED;
    const int ntiles = (N + RT - 1) / RT;
    const int grid = ntiles < cus ? ntiles : cus;
    constexpr size_t lds = (size_t)NW * S * (RT + XR) * KC * 2 + 2 * NW * 16 * 17 * 4 + 16 * 4;
#define BR_STREAM(MODE_)                                                                                        \
    do {                                                                                                        \
        auto kern = gemm_stream_kernel<RT, XR, KC, S, NW, MODE_, NORM>;                                         \
        static bool set = false;                                                                                \
        if (!set) {                                                                                             \
            if (hipFuncSetAttribute((const void*)kern, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds) != \
                hipSuccess)                                                                                     \
                return BR_LAUNCH_FAILED;                                                                        \
            set = true;                                                                                         \
        }                                                                                                       \
        kern<<<grid, NW * 64, lds, s>>>(A, W, C, M, N, K, lda, ldc, ntiles, nrm, wl);                           \
    } while (0)
    if constexpr (NORM == 1) {
        BR_STREAM(OUT_F32_ACC);
    } else {
        if (mode == OUT_BF16) BR_STREAM(OUT_BF16);
        else if (mode == OUT_F32) BR_STREAM(OUT_F32);
        else if (mode == OUT_SWIGLU) BR_STREAM(OUT_SWIGLU);
        else if constexpr (NORM == 0) BR_STREAM(OUT_F32_ACC);
        else return BR_BAD_ARG;
    }
#undef BR_STREAM
    return br_check_launch();
}

// ------------------------------------------------------------- gemm_stream_wide ------
// 16 < M <= 64, K in steps of 128: the same streaming by workgroups that stay, with the
// activations shared.  A unit of work is a tile of 16 HB weight rows (64 to 128) over one run of
// k-chunks (the whole K, or one of `parts` runs); height and runs are chosen so that the units
// fill the compute units in whole rounds (wide_shape below: 28,672 rows are 256 tiles of 112).
// Unit u of workgroup b is b + u * grid.  A stage of the workgroup's 3-stage LDS ring holds one
// 128-wide chunk of the tile and of the activations (16 MB rows), brought by all 8 waves with
// direct global-to-LDS loads, two chunks ahead; one barrier per chunk.  Wave w multiplies the
// weight rows 16 (w % 4) .. + 16 (and 64 + 16 (w % 4) .. + 16 where the tile has them) with
// k-steps 2 (w / 4), 2 (w / 4) + 1 of the chunk; the two k-halves are added in LDS at the
// unit's end (half 0 + half 1), in the stage that was multiplied last.  With `parts` > 1 the
// unit's float sums go to a matrix of its run (`part_stride` elements apart) for
// gemm_split_sum_kernel; else the epilogue (`mode`) is applied here.  The epilogue's form is
// chosen at run time: it runs once per unit, the chunk loop is the same for all.
// scale: the activations are the bf16(h * g) rows that the product before left for an RMS norm
// (see gemm_stream's NORM forms); the sums are multiplied by 1 / rms of their row, run by run.
#define WIDE_S 3
template <int MB, int HB>
__global__ __launch_bounds__(512) void gemm_stream_wide_kernel(const bf16* __restrict__ A, const bf16* __restrict__ W,
                                                               void* __restrict__ C, int M, int N, int K, size_t lda,
                                                               size_t ldc, int mode, int partial, int scale,
                                                               int ntiles, int parts, int cpp, size_t part_stride,
                                                               StreamNorm nrm, int wl) {
    constexpr int S = WIDE_S, D = S - 1, NW = 8, H = 16 * HB;
    constexpr int ROWS = H + 16 * MB;                // stacked rows of a stage: weights, then activations
    constexpr int STAGE = ROWS * 256;
    constexpr int NLD = ROWS / 4;                    // wave-loads of a chunk: 4 rows of 256 bytes each
    constexpr int NDMA = (NLD + NW - 1) / NW;        // of each wave; surplus ones repeat the chunk's last load
    constexpr int RLD = 16 * MB + 1;
    constexpr bool TWO = HB > 4;
    static_assert(HB >= 4 && HB <= 8 && (D - 1) * NDMA <= 63 && H * RLD * 4 <= STAGE, "stage");
    extern __shared__ __attribute__((aligned(1024))) unsigned char smem[];
    float* rstd = (float*)(smem + S * STAGE);        // scale: [64]
    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int r16 = lane & 15, g = lane >> 4;
    const int rb = wave & 3, khalf = wave >> 2;
    const bool has1 = TWO && rb + 4 < HB;
    const unsigned ring_lds = (unsigned)(size_t)((__attribute__((address_space(3))) unsigned char*)smem);
    const int nch = K / 128;
    const int nunits = ntiles * parts;
    const int my_units = (nunits - (int)blockIdx.x + (int)gridDim.x - 1) / (int)gridDim.x;

    f32x4 acc[TWO ? 2 : 1][MB];
#pragma unroll
    for (int t = 0; t < (TWO ? 2 : 1); ++t)
#pragma unroll
        for (int j = 0; j < MB; ++j) acc[t][j] = f32x4{0.f, 0.f, 0.f, 0.f};

    // Cursors over this workgroup's chunks in order.  What depends on the unit only (its tile, its run
    // of chunks, each lane's addresses) is worked out once per unit, so that a chunk costs each wave its
    // loads, an address step and a count.
    int is_u = 0, is_left = 0, cp_u = 0, cp_left = 0;       // units begun, chunks of the current one to go
    int is_wrap = 0, is_len = 0;                            // chunks to go before the run's first chunk is next; the run's length
    // Where in its run of chunks a workgroup starts (it wraps round to the run's first chunk): workgroups
    // that walk their rows in step ask the same few memory channels at the same time.
    const unsigned start_hash = ((unsigned)blockIdx.x * 2654435761u) >> 8;
    int issued = 0, done = 0;
    unsigned is_off = 0, cp_off = 0;                        // the ring's stage to fill, to multiply (bytes)
    const bf16* src[NDMA];                                  // this lane's 16 bytes of each of its loads
    const int wstep = wl ? WL_BLOCK_ELEMS : 128;                      // elements from a chunk of a weight row to the next
#define WIDE_RUN_LENGTH(U, LEN)                                                                               \
    do {                                                                                                      \
        const int c0_ = (((int)blockIdx.x + (U) * (int)gridDim.x) % parts) * cpp;                             \
        LEN = (c0_ + cpp < nch ? c0_ + cpp : nch) - c0_;                                                      \
    } while (0)
#define WIDE_LOAD_INDEX(Q) ((wave * NDMA + (Q)) < NLD - 1 ? (wave * NDMA + (Q)) : NLD - 1)
#define WIDE_SETUP()                                                                                          \
    do {                                                                                                      \
        const int unit_ = (int)blockIdx.x + is_u * (int)gridDim.x;                                            \
        const int tile_ = unit_ / parts, c0_ = (unit_ % parts) * cpp;                                         \
        is_left = (c0_ + cpp < nch ? c0_ + cpp : nch) - c0_;                                                  \
        is_len = is_left;                                                                                     \
        const int rot_ = (int)(start_hash % (unsigned)is_left);                                               \
        is_wrap = is_left - rot_;                                                                             \
        _Pragma("unroll") for (int q_ = 0; q_ < NDMA; ++q_) {                                                 \
            const int row_ = WIDE_LOAD_INDEX(q_) * 4 + (lane >> 4);                                           \
            const bf16* gp_;                                                                                  \
            if (row_ < H) {                                                                                   \
                int n_ = tile_ * H + row_;                                                                    \
                if (n_ > N - 1) n_ = N - 1;                                                                   \
                gp_ = W + w_row_base(n_, K, wl) + (size_t)(c0_ + rot_) * wstep;                               \
            } else {                                                                                          \
                int m_ = row_ - H;                                                                            \
                if (m_ > M - 1) m_ = M - 1;                                                                   \
                gp_ = A + (size_t)m_ * lda + (size_t)(c0_ + rot_) * 128;                                      \
            }                                                                                                 \
            src[q_] = gp_ + (((lane & 15) ^ (row_ & 7)) * 8);                                                 \
        }                                                                                                     \
    } while (0)
#define WIDE_ISSUE()                                                                                          \
    do {                                                                                                      \
        _Pragma("unroll") for (int q_ = 0; q_ < NDMA; ++q_) {                                                 \
            const unsigned lds_ = __builtin_amdgcn_readfirstlane(ring_lds + is_off + WIDE_LOAD_INDEX(q_) * 1024); \
            if (WIDE_LOAD_INDEX(q_) * 4 < H)                /* weights pass once: non-temporal */             \
                asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, off nt" ::"s"(lds_), "v"(src[q_]) : "m0"); \
            else                                                                                              \
                asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, off" ::"s"(lds_), "v"(src[q_]) : "m0"); \
            src[q_] += WIDE_LOAD_INDEX(q_) * 4 < H ? wstep : 128;                                             \
        }                                                                                                     \
        if (--is_wrap == 0) {                              /* on to the run's first chunk */                  \
            _Pragma("unroll") for (int q_ = 0; q_ < NDMA; ++q_)                                               \
                src[q_] -= (size_t)is_len * (WIDE_LOAD_INDEX(q_) * 4 < H ? wstep : 128);                      \
        }                                                                                                     \
        ++issued;                                                                                             \
        is_off = is_off + STAGE == S * STAGE ? 0 : is_off + STAGE;                                            \
        if (--is_left == 0 && ++is_u < my_units) WIDE_SETUP();                                                \
    } while (0)

    if (my_units > 0) WIDE_SETUP();
    for (int j = 0; j < D; ++j)
        if (is_u < my_units) WIDE_ISSUE();
    if (scale) {
        // row m = tid / 8: its 8 lanes take the tiles' sums in turn, then a butterfly; read at the first unit's end
        const int m = tid >> 3, l = tid & 7;
        float t = 0.f;
        if (m < M)
            for (int c = l; c < nrm.ssq_tiles; c += 8) t += nrm.ssq[(size_t)c * SSQ_LD + m];
#pragma unroll
        for (int o = 4; o > 0; o >>= 1) t += __shfl_xor(t, o, 64);
        if (l == 0) rstd[m] = m < M ? rsqrtf(t * nrm.inv_k + nrm.eps) : 0.f;
    }
    if (my_units > 0) WIDE_RUN_LENGTH(0, cp_left);
    while (cp_u < my_units) {
        // the chunk to multiply has landed when at most the loads of the chunks issued after it are in flight
        if (issued - done - 1 >= 1) asm volatile("s_waitcnt vmcnt(%0)" ::"n"(NDMA) : "memory");
        else asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
        __builtin_amdgcn_s_barrier();            // every wave's part of it is there; the chunk before is done with
        asm volatile("" ::: "memory");
        if (is_u < my_units) WIDE_ISSUE();
        unsigned char* st = smem + cp_off;
        cp_off = cp_off + STAGE == S * STAGE ? 0 : cp_off + STAGE;
#pragma unroll
        for (int ks = 0; ks < 2; ++ks) {
            const int col = 4 * (2 * khalf + ks) + g;
            const int wr = 16 * rb + r16;
            const bf16x8 wf0 = *(const bf16x8*)(st + wr * 256 + ((col ^ (wr & 7)) * 16));
            bf16x8 wf1 = wf0;
            if (TWO && has1) wf1 = *(const bf16x8*)(st + (64 + wr) * 256 + ((col ^ (wr & 7)) * 16));
#pragma unroll
            for (int j = 0; j < MB; ++j) {
                const int xr = H + 16 * j + r16;
                const bf16x8 xv = *(const bf16x8*)(st + xr * 256 + ((col ^ (xr & 7)) * 16));
                acc[0][j] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(wf0, xv, acc[0][j], 0, 0, 0);
                if (TWO && has1) acc[TWO ? 1 : 0][j] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(wf1, xv, acc[TWO ? 1 : 0][j], 0, 0, 0);
            }
        }
        ++done;
        if (--cp_left > 0) continue;
        // The unit's end: acc[t][j][r] is weight row 64 t + 16 rb + 4 g + r of the tile, batch row 16 j + r16.
        // The sums meet in the stage that was multiplied last: the next loads into it are issued after
        // the next chunk's barrier, which a wave reaches after its part of the epilogue.
        const int unit = (int)blockIdx.x + cp_u * (int)gridDim.x;
        const int part = unit % parts;
        const int n0 = (unit / parts) * H;
        if (++cp_u < my_units) WIDE_RUN_LENGTH(cp_u, cp_left);
        float* red = (float*)st;                 // [H][RLD]
        __builtin_amdgcn_s_barrier();            // every wave has read its operands of the stage
        asm volatile("" ::: "memory");
        if (khalf == 1) {
#pragma unroll
            for (int t = 0; t < (TWO ? 2 : 1); ++t)
                if (t == 0 || has1)
#pragma unroll
                    for (int j = 0; j < MB; ++j)
#pragma unroll
                        for (int r = 0; r < 4; ++r) red[(64 * t + 16 * rb + 4 * g + r) * RLD + 16 * j + r16] = acc[t][j][r];
        }
        asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
        __builtin_amdgcn_s_barrier();
        asm volatile("" ::: "memory");
        if (khalf == 0) {
#pragma unroll
            for (int t = 0; t < (TWO ? 2 : 1); ++t)
                if (t == 0 || has1)
#pragma unroll
                    for (int j = 0; j < MB; ++j)
#pragma unroll
                        for (int r = 0; r < 4; ++r) {
                            float* p = red + (64 * t + 16 * rb + 4 * g + r) * RLD + 16 * j + r16;
                            *p = acc[t][j][r] + *p;
                        }
        }
#pragma unroll
        for (int t = 0; t < (TWO ? 2 : 1); ++t)
#pragma unroll
            for (int j = 0; j < MB; ++j) acc[t][j] = f32x4{0.f, 0.f, 0.f, 0.f};
        asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
        __builtin_amdgcn_s_barrier();
        asm volatile("" ::: "memory");
        if (mode == OUT_SWIGLU && !partial) {
            // blocks of 16 tile rows: 8 gates, then the 8 up values of the same outputs
            for (int e = tid; e < (H / 2) * 16 * MB; e += 512) {
                const int m = e / (H / 2), jl = e % (H / 2);
                const int gr = (jl >> 3) * 16 + (jl & 7);
                if (m < M && n0 + gr + 8 < N) {
                    float gv = red[gr * RLD + m];
                    float uv = red[(gr + 8) * RLD + m];
                    if (scale) { gv *= rstd[m]; uv *= rstd[m]; }
                    ((bf16*)C)[(size_t)m * ldc + n0 / 2 + jl] = (bf16)silu_mul(gv, uv);
                }
            }
        } else {
            for (int e = tid; e < H * 16 * MB; e += 512) {
                const int m = e / H, nl = e % H, n = n0 + nl;
                if (m < M && n < N) {
                    float v = red[nl * RLD + m];
                    if (scale) v *= rstd[m];
                    const size_t idx = (size_t)m * ldc + n;
                    if (partial) ((float*)C)[part * part_stride + (size_t)m * N + n] = v;
                    else if (mode == OUT_BF16) ((bf16*)C)[idx] = (bf16)v;
                    else if (mode == OUT_F32) ((float*)C)[idx] = v;
                    else unsafeAtomicAdd((float*)C + idx, v);         // one add per element, no read to wait for
                }
            }
        }
    }
#undef WIDE_ISSUE
#undef WIDE_SETUP
#undef WIDE_LOAD_INDEX
#undef WIDE_RUN_LENGTH
}

// The shape of gemm_stream_wide's units: tile height (64 to 128 rows in steps of 16) and runs
// along k (1 to 8), the least time by a simple count: rounds of units over the compute
// units, times the run's chunks, times what a chunk costs (its weight rows and a constant for
// the activations, which come from the L2, and the barrier), plus the traffic of the partial
// sums.  Ties go to fewer runs, then to lower tiles.
static void wide_shape(int M, int N, int K, int mode, int cus, size_t scratch_bytes, int* hb_out, int* parts_out) {
    const int nch = K / 128;
    double best_cost = 1e30;
    *hb_out = 4;
    *parts_out = 1;
    for (int parts = 1; parts <= 8; ++parts) {
        if (parts > 1 && (mode == OUT_SWIGLU || parts * 2 > nch || (size_t)parts * M * N * sizeof(float) > scratch_bytes))
            break;
        const int cpp = (nch + parts - 1) / parts;
        if ((nch + cpp - 1) / cpp != parts) continue;                // it would leave a run empty
        for (int hb = 4; hb <= 8; ++hb) {
            const int h = 16 * hb;
            const long long tiles = (N + h - 1) / h;
            const long long rounds = (tiles * parts + cus - 1) / cus;
            double cost = (double)rounds * cpp * (h + 16.0);
            if (parts > 1) cost *= 1.0 + 4.0 * parts * M / K;
            if (cost < best_cost * (1.0 - 1e-9)) { best_cost = cost; *hb_out = hb; *parts_out = parts; }
        }
    }
}

// norm: 0 none; 1 the product is added into the residual rows C and prepares the next RMS norm
// (needs a split product: the sum kernel does it; refused otherwise); 2 the activations were so
// prepared and the sums are scaled (modes 0, 1, 3).  force_hb, force_parts: a tile height (in
// blocks of 16 rows) and a number of runs other than wide_shape's (tests and measurements).
// leave: the runs' sums stay in `scratch` ([runs][M][N] floats) for a consumer that adds them
// in run order itself, and *leave says how many runs; refused (nothing launched) when the
// product is not cut.
template <int MB>
static int launch_stream_wide(const bf16* A, const bf16* W, void* C, int M, int N, int K, size_t lda, size_t ldc,
                              int mode, float* scratch, size_t scratch_bytes, hipStream_t s, int norm = 0,
                              StreamNorm nrm = StreamNorm{}, int force_hb = 0, int force_parts = 0, int wl = 0,
                              int* leave = nullptr) {
    const int cus = br_device_cus();
    if (!cus) return BR_LAUNCH_FAILED;
    const int nch = K / 128;
    int hb, parts;
    wide_shape(M, N, K, mode, cus, scratch ? scratch_bytes : 0, &hb, &parts);
    if (leave && (parts < 2 || norm == 1 || force_hb || force_parts)) return BR_BAD_ARG;
    if (force_hb) {
        if (force_hb < 4 || force_hb > 8) return BR_BAD_ARG;
        hb = force_hb;
    }
    if (force_parts) {
        const int cpp_ = (nch + force_parts - 1) / force_parts;
        if (force_parts > 1 && (!scratch || mode == OUT_SWIGLU || force_parts > 8 || force_parts * 2 > nch ||
                                (nch + cpp_ - 1) / cpp_ != force_parts ||
                                (size_t)force_parts * M * N * sizeof(float) > scratch_bytes))
            return BR_BAD_ARG;
        parts = force_parts;
    }
    if (norm == 1 && (parts < 2 || N % 256 || mode != OUT_F32_ACC)) return BR_BAD_ARG;
    if (norm == 2 && mode == OUT_F32_ACC) return BR_BAD_ARG;
    const int cpp = (nch + parts - 1) / parts;
    const int h = 16 * hb, ntiles = (N + h - 1) / h;
    const long long nunits = (long long)ntiles * parts;
    const int grid = nunits < cus ? (int)nunits : cus;
    const size_t stride = (size_t)M * N;
    const int partial = parts > 1;
    void* out = partial ? (void*)scratch : C;
#define BR_WIDE(HB_)                                                                                            \
    do {                                                                                                        \
        auto kern = gemm_stream_wide_kernel<MB, HB_>;                                                           \
        constexpr size_t lds = (size_t)WIDE_S * (16 * HB_ + 16 * MB) * 256 + 64 * 4;                            \
        static_assert(lds <= 160 * 1024, "LDS of a compute unit");                                              \
        static bool set = false;                                                                                \
        if (!set) {                                                                                             \
            if (hipFuncSetAttribute((const void*)kern, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds) != \
                hipSuccess)                                                                                     \
                return BR_LAUNCH_FAILED;                                                                        \
            set = true;                                                                                         \
        }                                                                                                       \
        kern<<<grid, 512, lds, s>>>(A, W, out, M, N, K, lda, ldc, mode, partial, norm == 2, ntiles, parts, cpp, \
                                    stride, nrm, wl);                                                           \
    } while (0)
    switch (hb) {
        case 4: BR_WIDE(4); break;
        case 5: BR_WIDE(5); break;
        case 6: BR_WIDE(6); break;
        case 7: BR_WIDE(7); break;
        default: BR_WIDE(8); break;
    }
#undef BR_WIDE
    int rc = br_check_launch();
    if (rc != BR_OK || !partial) return rc;
    if (leave) {
        *leave = parts;
        return rc;
    }
    if (norm == 1) {
        gemm_split_sum_prep_kernel<<<(unsigned)(stride / 256), 256, 0, s>>>(scratch, parts, stride, (float*)C, N, ldc,
                                                                            nrm.gain, nrm.xg, nrm.ldx, nrm.ssq);
        return br_check_launch();
    }
    return launch_split_sum(scratch, parts, C, M, N, ldc, mode, s);
}

// kernel: 0 = choose, 1 = tile 128x128 through registers (any shape), 2 = the same 256x128,
// 3 = skinny (M <= 64), 4..6 = direct-to-LDS tiles 256x128, 128x256, 128x128 (K a multiple
// of 64, aligned rows), 7 = stream (M <= 16, K a multiple of 128 and at least 1024, aligned
// rows), 8 = stream wide (16 < M <= 64, K a multiple of 128), 9 = direct-to-LDS tile 64x128
// (M <= 64), 10 = direct-to-LDS tile 256x192, 11 = the same 256x256 (SwiGLU epilogue only), 12..15 = the tiles of
// four waves, one to a SIMD: 256x256, 128x256, 256x192, 256x224 (K a multiple of 64, aligned rows, output rows in steps
// of 16 bytes; plus 16 p: with p runs along k); tests force one.  (A 256x256 tile of 8 waves for every epilogue
// was tried: it runs out of registers in three of the four and was no faster in the fourth.)
// `wl`: the layout of W (see WL_BLOCKED; K in steps of 128 then, kernels 4 to 15).
// `scratch` (float, `scratch_bytes`; may be null) lets a product of 16 < M <= 64 rows with few
// weight rows be split along k (see gemm_split_sum_kernel); BR_GEMM_SCRATCH_BYTES always suffices.
extern "C" int br_gemm_bf16_ex(const void* A_, const void* W_, void* C, int M, int N, int K, size_t lda,
                               size_t ldc, int mode, int kernel, void* scratch, size_t scratch_bytes, int wl,
                               hipStream_t s) {
    if (M <= 0 || N <= 0) return BR_OK;
    if (K <= 0 || lda < (size_t)K || mode < 0 || mode > 3) return BR_BAD_ARG;
    if (mode == OUT_SWIGLU ? (N % 16 != 0 || ldc < (size_t)N / 2) : ldc < (size_t)N) return BR_BAD_ARG;
    // kernel / 16: a forced number of runs along k for kernels 5 and 6, or for kernel 8 a forced tile
    // height in blocks of 16 rows plus 16 times a forced number of runs (measurements and tests), 0 = by shape
    const int forced_parts = kernel >= 16 ? kernel / 16 : 0;
    kernel %= 16;
    const bf16* A = (const bf16*)A_;
    const bf16* W = (const bf16*)W_;
    const bool aligned = (K % 8 == 0) && (lda % 8 == 0) && (((uintptr_t)A | (uintptr_t)W) % 16 == 0);
    if (kernel == 3 && (!aligned || M > 64)) return BR_BAD_ARG;
    const bool dma_ok = aligned && K % DMA_BK == 0;
    const bool stream_ok = aligned && M <= 16 && K % STREAM_KC == 0 && K / STREAM_KC >= STREAM_NW;
    if (kernel >= 4 && kernel <= 6 && !dma_ok) return BR_BAD_ARG;
    const bool wide_ok = aligned && M > 16 && M <= 64 && K % 128 == 0 && K >= 256 &&
                         (!scratch || (uintptr_t)scratch % 16 == 0);
    if ((kernel == 7 && !stream_ok) || (kernel == 8 && !wide_ok) || kernel > 15 || kernel < 0 || (kernel >= 10 && !dma_ok) ||
        (kernel == 11 && mode != OUT_SWIGLU) ||
        (kernel == 9 && (!dma_ok || M > 64)))
        return BR_BAD_ARG;
    if (wl != WL_ROWS) {
        if (wl != WL_BLOCKED || !aligned || K % 128 || (kernel != 0 && kernel < 4)) return BR_BAD_ARG;
        if (kernel == 0 && M <= 16 && !stream_ok) return BR_BAD_ARG;      // blocked weights have K from 1024
    }
    const bool chosen = kernel == 0;
    if (kernel == 0)
        kernel = stream_ok ? 7
                 : wide_ok ? 8
                 : (aligned && M <= 64) ? (wl ? 9 : 3) : (!dma_ok ? 1 : (N > 128 ? 5 : 6));
    if (kernel == 9) return launch_tile_dma<64, 128, 1, 4, 3>(A, W, C, M, N, K, lda, ldc, mode, s, 1, nullptr, wl);
    if (kernel == 8) {
        const int fh = chosen ? 0 : forced_parts % 16, fp = chosen ? 0 : forced_parts / 16;
        return M <= 32 ? launch_stream_wide<2>(A, W, C, M, N, K, lda, ldc, mode, (float*)scratch, scratch_bytes, s, 0,
                                               StreamNorm{}, fh, fp, wl)
                       : launch_stream_wide<4>(A, W, C, M, N, K, lda, ldc, mode, (float*)scratch, scratch_bytes, s, 0,
                                               StreamNorm{}, fh, fp, wl);
    }
    if (kernel == 7) return M <= 8 ? launch_stream<8, 0>(A, W, C, M, N, K, lda, ldc, mode, s, StreamNorm{}, wl)
                                   : launch_stream<16, 0>(A, W, C, M, N, K, lda, ldc, mode, s, StreamNorm{}, wl);
    int parts = 1;
    if (chosen && M > 128 && (kernel == 5 || kernel == 6) && quad_takes(C, M, N, K, lda, ldc)) {
        // More than 128 rows, K in steps of 64: the tiles of one wave per SIMD, where the product's addresses
        // allow.  (Up to 128 rows the tiles of eight waves below stream the weights faster: 7B shapes at 128
        // rows, gate/up 59 against 69 us, the 32,768-row head 71 against 85, down 39 against 45.)
        const int cus = br_device_cus();
        const size_t room = (scratch && (uintptr_t)scratch % 16 == 0) ? scratch_bytes : 0;
        if (cus > 0) {
            const double single = choose_quad(M, N, K, mode, cus, room, &kernel, &parts);
            int k2, p2;
            const int n1 = quad_whole_rounds(M, N, K, mode, cus, room, single, &k2, &p2);
            if (n1 > 0) {
                // whole rounds of the 256x256 tile over the first n1 weight rows, then the rest; n1 rows on
                // is the same number of elements in either weight layout (n1 is a multiple of 16)
                int rc = launch_tile_quad<256, 256, QUAD12>(A, W, C, M, n1, K, lda, ldc, mode, s, wl);
                if (rc != BR_OK) return rc;
                const bf16* W2 = W + (size_t)n1 * K;
                void* C2 = mode == OUT_SWIGLU ? (void*)((bf16*)C + n1 / 2)
                           : mode == OUT_BF16 ? (void*)((bf16*)C + n1) : (void*)((float*)C + n1);
                const int N2 = N - n1;
                if (k2 == 12) return launch_tile_quad<256, 256, QUAD12>(A, W2, C2, M, N2, K, lda, ldc, mode, s, wl, p2, (float*)scratch);
                if (k2 == 13) return launch_tile_quad<128, 256, QUAD13>(A, W2, C2, M, N2, K, lda, ldc, mode, s, wl, p2, (float*)scratch);
                if (k2 == 15) return launch_tile_quad<256, 224, 2, 3, 4>(A, W2, C2, M, N2, K, lda, ldc, mode, s, wl, p2, (float*)scratch);
                return launch_tile_quad<256, 192, QUAD14>(A, W2, C2, M, N2, K, lda, ldc, mode, s, wl, p2, (float*)scratch);
            }
        }
    }
    if (chosen && (kernel == 5 || kernel == 6)) {
        const int cus = br_device_cus();
        if (cus > 0) choose_tile(M, N, K, mode, cus, (scratch && (uintptr_t)scratch % 16 == 0) ? scratch_bytes : 0, &kernel, &parts);
    }
    if (chosen && mode == OUT_SWIGLU && kernel == 5 && parts == 1) {
        // The 256x256 tile over as many weight rows as make whole rounds of it, the 128x256 tile over the rest,
        // where the count says that this is faster than 128x256 over all of them (2,048 x 28,672: three
        // rounds of 256x256 over 24,576 rows and one round of 128x256 over 4,096, instead of seven of 128x256).
        const int cus = br_device_cus();
        const int tm11 = (M + 255) / 256, nk = K / DMA_BK;
        const int cols = cus > 0 ? cus / tm11 : 0;                   // tile columns of one round
        if (cols > 0) {
            const long long n_round = (long long)cols * 256;
            const long long r11 = N / n_round, n1 = r11 * n_round, n2 = N - n1;
            const long long t5_all = ((long long)((M + 127) / 128) * ((N + 255) / 256) + cus - 1) / cus;
            const long long t5_rest = ((long long)((M + 127) / 128) * ((n2 + 255) / 256) + cus - 1) / cus;
            const double whole = (double)t5_all * nk * 1.14;
            const double split = (double)r11 * nk * 2.05 + (double)t5_rest * nk * 1.14 + 5.0;
            if (r11 >= 1 && n2 > 0 && n2 % 16 == 0 && split < 0.97 * whole) {
                gemm_tile_dma_kernel<256, 256, 2, 4, 2, OUT_SWIGLU><<<(unsigned)(tm11 * (int)(n1 / 256)), 512, 0, s>>>(
                    A, W, C, M, (int)n1, K, lda, ldc, tm11, (int)(n1 / 256), nk, 0, wl);
                int rc = br_check_launch();
                if (rc != BR_OK) return rc;
                // n1 rows on: the same number of elements in either weight layout (n1 is a multiple of 16)
                return launch_tile_dma<128, 256, 2, 4, 3>(A, W + (size_t)n1 * K, (bf16*)C + n1 / 2, M, (int)n2, K, lda, ldc,
                                                          mode, s, 1, nullptr, wl);
            }
        }
    }
    if (kernel >= 12 && forced_parts > 1) {
        if (!scratch || (uintptr_t)scratch % 16 || (size_t)forced_parts * M * N * sizeof(float) > scratch_bytes ||
            forced_parts * 2 > K / DMA_BK)
            return BR_BAD_ARG;
        parts = forced_parts;
    }
    if (kernel == 12) return launch_tile_quad<256, 256, QUAD12>(A, W, C, M, N, K, lda, ldc, mode, s, wl, parts, (float*)scratch);
    if (kernel == 13) return launch_tile_quad<128, 256, QUAD13>(A, W, C, M, N, K, lda, ldc, mode, s, wl, parts, (float*)scratch);
    if (kernel == 14) return launch_tile_quad<256, 192, QUAD14>(A, W, C, M, N, K, lda, ldc, mode, s, wl, parts, (float*)scratch);
    if (kernel == 15) return launch_tile_quad<256, 224, 2, 3, 4>(A, W, C, M, N, K, lda, ldc, mode, s, wl, parts, (float*)scratch);
    if (kernel == 10) return launch_tile_dma<256, 192, 4, 2, 2>(A, W, C, M, N, K, lda, ldc, mode, s, 1, nullptr, wl);
    if (kernel == 11) {
        gemm_tile_dma_kernel<256, 256, 2, 4, 2, OUT_SWIGLU><<<(unsigned)(((M + 255) / 256) * ((N + 255) / 256)), 512, 0, s>>>(
            A, W, C, M, N, K, lda, ldc, (M + 255) / 256, (N + 255) / 256, K / DMA_BK, 0, wl);
        return br_check_launch();
    }
    if (forced_parts > 1 && (kernel == 5 || kernel == 6)) {
        if (!scratch || (uintptr_t)scratch % 16 || (size_t)forced_parts * M * N * sizeof(float) > scratch_bytes ||
            forced_parts > K / DMA_BK)
            return BR_BAD_ARG;
        parts = forced_parts;
    }
    if (kernel == 4) return launch_tile_dma<256, 128, 4, 2, 3>(A, W, C, M, N, K, lda, ldc, mode, s, 1, nullptr, wl);
    if (kernel == 5) return launch_tile_dma<128, 256, 2, 4, 3>(A, W, C, M, N, K, lda, ldc, mode, s, parts, (float*)scratch, wl);
    if (kernel == 6) return launch_tile_dma<128, 128, 2, 2, 2>(A, W, C, M, N, K, lda, ldc, mode, s, parts, (float*)scratch, wl);
    if (kernel == 3) {
        // shapes measured on cold weights (cycled through more than the 256 MB cache)
        const bool wide = N >= 16384;
        if (M <= 16) return (wide && M > 4) ? launch_skinny<1, 1, 2, 8>(A, W, C, M, N, K, lda, ldc, mode, s)
                                            : launch_skinny<1, 1, 4, 8>(A, W, C, M, N, K, lda, ldc, mode, s);
        const int parts = (scratch && (uintptr_t)scratch % 16 == 0) ? split_parts(M, N, K, mode, scratch_bytes) : 1;
        if (parts > 1)
            return M <= 32 ? launch_split<2>(A, W, C, M, N, K, lda, ldc, mode, parts, (float*)scratch, s)
                           : launch_split<4>(A, W, C, M, N, K, lda, ldc, mode, parts, (float*)scratch, s);
        if (M <= 32) return wide ? launch_skinny_lds<2, 4>(A, W, C, M, N, K, lda, ldc, mode, s)
                                 : launch_skinny_lds<2, 1>(A, W, C, M, N, K, lda, ldc, mode, s);
        if (wide) return dma_ok ? launch_tile_dma<64, 128, 1, 4, 3>(A, W, C, M, N, K, lda, ldc, mode, s)
                                : launch_skinny_lds<4, 4>(A, W, C, M, N, K, lda, ldc, mode, s);
        return (N >= 6144) ? launch_skinny_lds<4, 2>(A, W, C, M, N, K, lda, ldc, mode, s)
                           : launch_skinny_lds<4, 1>(A, W, C, M, N, K, lda, ldc, mode, s);
    }
    if (kernel == 2) return launch_tile<256, 128, 32, 2, 2>(A, W, C, M, N, K, lda, ldc, mode, aligned, s);
    return launch_tile<128, 128, 64, 2, 2>(A, W, C, M, N, K, lda, ldc, mode, aligned, s);
}

extern "C" int br_gemm_bf16(const void* A, const void* W, void* C, int M, int N, int K, size_t lda, size_t ldc,
                            int mode, hipStream_t s) {
    return br_gemm_bf16_ex(A, W, C, M, N, K, lda, ldc, mode, 0, nullptr, 0, WL_ROWS, s);
}

// What br_gemm_bf16_ex picks for a product of more than 64 rows with K in steps of 64, aligned rows and a
// contiguous, aligned output (tests and benchmarks ask): the kernel and its runs along k; and, where the product is
// cut along its weight rows, `n1` > 0 rows by the 256x256 tile first and `kernel`, `parts` for the rest.
extern "C" int br_gemm_bf16_tile_choice(int M, int N, int K, int mode, size_t scratch_bytes, int* kernel, int* parts,
                                        int* n1) {
    const int cus = br_device_cus();
    if (!cus) return BR_LAUNCH_FAILED;
    *n1 = 0;
    if (M > 128 && quad_takes(nullptr, M, N, K, (size_t)K, (size_t)(mode == OUT_SWIGLU ? N / 2 : N))) {
        const double single = choose_quad(M, N, K, mode, cus, scratch_bytes, kernel, parts);
        int k2, p2;
        const int rows = quad_whole_rounds(M, N, K, mode, cus, scratch_bytes, single, &k2, &p2);
        if (rows > 0) {
            *n1 = rows;
            *kernel = k2;
            *parts = p2;
        }
        return BR_OK;
    }
    choose_tile(M, N, K, mode, cus, scratch_bytes, kernel, parts);
    return BR_OK;
}

static bool stream_takes(const void* A, const void* W, int M, int K, size_t lda) {
    return M > 0 && M <= 16 && K % STREAM_KC == 0 && K / STREAM_KC >= STREAM_NW && lda % 8 == 0 && lda >= (size_t)K &&
           ((uintptr_t)A | (uintptr_t)W) % 16 == 0;
}
static bool wide_takes(const void* A, const void* W, int M, int K, size_t lda) {
    return M > 16 && M <= 64 && K % 128 == 0 && K >= 256 && lda % 8 == 0 && lda >= (size_t)K &&
           ((uintptr_t)A | (uintptr_t)W) % 16 == 0;
}

// C += A W^T through the streaming products, which then also prepare the RMS norm that reads C
// next: xg[M, ldx] = bf16(C * gain) and sums of squares in ssq[tiles, SSQ_LD] (see the kernels);
// *ssq_tiles says how many.  Up to 16 rows: gemm_stream (N in steps of 16).  17 to 64 rows:
// gemm_stream_wide cut along k, the preparation in the sum kernel (N in steps of 256, scratch
// needed).  Refuses (BR_BAD_ARG) anything else: the caller then runs the norm itself.
extern "C" int br_gemm_bf16_norm_prepare(const void* A, const void* W, float* C, int M, int N, int K, size_t lda,
                                         size_t ldc, const float* gain, void* xg, size_t ldx, float* ssq,
                                         int* ssq_tiles, void* scratch, size_t scratch_bytes, int wl, hipStream_t s) {
    if (M <= 0 || N <= 0 || (wl != WL_ROWS && wl != WL_BLOCKED)) return BR_BAD_ARG;
    if (ldc < (size_t)N || ldx < (size_t)N || !gain || !xg || !ssq || !ssq_tiles) return BR_BAD_ARG;
    StreamNorm nrm{gain, (bf16*)xg, ldx, ssq, 0, 0.f, 0.f};
    if (stream_takes(A, W, M, K, lda) && N % 16 == 0) {
        *ssq_tiles = N / 16;
        return M <= 8 ? launch_stream<8, 1>((const bf16*)A, (const bf16*)W, C, M, N, K, lda, ldc, OUT_F32_ACC, s, nrm, wl)
                      : launch_stream<16, 1>((const bf16*)A, (const bf16*)W, C, M, N, K, lda, ldc, OUT_F32_ACC, s, nrm, wl);
    }
    if (wide_takes(A, W, M, K, lda) && N % 256 == 0 && scratch && (uintptr_t)scratch % 16 == 0) {
        *ssq_tiles = N / 256;
        return M <= 32 ? launch_stream_wide<2>((const bf16*)A, (const bf16*)W, C, M, N, K, lda, ldc, OUT_F32_ACC,
                                               (float*)scratch, scratch_bytes, s, 1, nrm, 0, 0, wl)
                       : launch_stream_wide<4>((const bf16*)A, (const bf16*)W, C, M, N, K, lda, ldc, OUT_F32_ACC,
                                               (float*)scratch, scratch_bytes, s, 1, nrm, 0, 0, wl);
    }
    return BR_BAD_ARG;
}

// C = rsqrt(sum of the ssq tiles / norm_width + eps) * (XG W^T), XG and ssq from br_gemm_bf16_norm_prepare:
// the product of the normed rows.  mode: 0 bf16, 1 float, 3 SwiGLU.
extern "C" int br_gemm_bf16_norm_scaled(const void* XG, const void* W, void* C, int M, int N, int K, size_t lda,
                                        size_t ldc, int mode, const float* ssq, int ssq_tiles, int norm_width,
                                        float eps, void* scratch, size_t scratch_bytes, int wl, hipStream_t s) {
    if (M <= 0 || N <= 0) return BR_OK;
    if (wl != WL_ROWS && wl != WL_BLOCKED) return BR_BAD_ARG;
    if (!ssq || ssq_tiles <= 0 || norm_width <= 0 || (mode != OUT_BF16 && mode != OUT_F32 && mode != OUT_SWIGLU))
        return BR_BAD_ARG;
    if (mode == OUT_SWIGLU ? (N % 16 != 0 || ldc < (size_t)N / 2) : ldc < (size_t)N) return BR_BAD_ARG;
    StreamNorm nrm{nullptr, nullptr, 0, (float*)ssq, ssq_tiles, 1.f / (float)norm_width, eps};
    if (stream_takes(XG, W, M, K, lda))
        return M <= 8 ? launch_stream<8, 2>((const bf16*)XG, (const bf16*)W, C, M, N, K, lda, ldc, mode, s, nrm, wl)
                      : launch_stream<16, 2>((const bf16*)XG, (const bf16*)W, C, M, N, K, lda, ldc, mode, s, nrm, wl);
    if (wide_takes(XG, W, M, K, lda)) {
        float* sc = (scratch && (uintptr_t)scratch % 16 == 0) ? (float*)scratch : nullptr;
        return M <= 32 ? launch_stream_wide<2>((const bf16*)XG, (const bf16*)W, C, M, N, K, lda, ldc, mode, sc,
                                               scratch_bytes, s, 2, nrm, 0, 0, wl)
                       : launch_stream_wide<4>((const bf16*)XG, (const bf16*)W, C, M, N, K, lda, ldc, mode, sc,
                                               scratch_bytes, s, 2, nrm, 0, 0, wl);
    }
    return BR_BAD_ARG;
}

// The float sums of the runs of A W^T (17 to 64 rows, bf16 result meant), left in `scratch` as
// [*parts][M][N] for a consumer that adds them in run order and rounds, which gives the bits of
// br_gemm_bf16 (or, with ssq, of br_gemm_bf16_norm_scaled) without the sum kernel's launch.
// Refuses (BR_BAD_ARG, nothing launched) where those would not cut the product.
extern "C" int br_gemm_bf16_wide_partial(const void* A, const void* W, int M, int N, int K, size_t lda,
                                         const float* ssq, int ssq_tiles, int norm_width, float eps, void* scratch,
                                         size_t scratch_bytes, int wl, int* parts, hipStream_t s) {
    if (M <= 16 || M > 64 || N <= 0 || !parts || (wl != WL_ROWS && wl != WL_BLOCKED)) return BR_BAD_ARG;
    if (!scratch || (uintptr_t)scratch % 16 || !wide_takes(A, W, M, K, lda)) return BR_BAD_ARG;
    if (ssq && (ssq_tiles <= 0 || norm_width <= 0)) return BR_BAD_ARG;
    StreamNorm nrm{};
    if (ssq) nrm = StreamNorm{nullptr, nullptr, 0, (float*)ssq, ssq_tiles, 1.f / (float)norm_width, eps};
    const int norm = ssq ? 2 : 0;
    return M <= 32 ? launch_stream_wide<2>((const bf16*)A, (const bf16*)W, nullptr, M, N, K, lda, (size_t)N, OUT_BF16,
                                           (float*)scratch, scratch_bytes, s, norm, nrm, 0, 0, wl, parts)
                   : launch_stream_wide<4>((const bf16*)A, (const bf16*)W, nullptr, M, N, K, lda, (size_t)N, OUT_BF16,
                                           (float*)scratch, scratch_bytes, s, norm, nrm, 0, 0, wl, parts);
}

// into how many runs along k br_gemm_bf16_ex and br_gemm_bf16_norm_prepare cut a product of 17 to 64 rows
extern "C" int br_gemm_bf16_wide_parts(int M, int N, int K, int mode, size_t scratch_bytes) {
    const int cus = br_device_cus();
    if (!cus || M <= 16 || M > 64 || K % 128 || K < 256) return 0;
    int hb, parts;
    wide_shape(M, N, K, mode, cus, scratch_bytes, &hb, &parts);
    return parts;
}

// rows of a block of the blocked weight layout (the host lays weights out by it)
extern "C" int br_gemm_bf16_block_rows() { return WL_BLOCK_ROWS; }
