// Attention over the paged bf16 cache on the gfx950 matrix cores: a flash kernel for
// steps with several tokens per sequence (prompts, chunks) and a split-context kernel
// for single-token steps.  Both compute, per (query row, kv head), the online softmax
// of the reference (m' = max(m, s), c = exp(m - m'), d = d c + w, acc = acc c + w v;
// kernels/megakernel_ops.hip:2310-2342) in float, with kv head = q head / (nq / nkv)
// (:2192), scores scaled by `scale` (:2194), causality as a bound on the key index and a
// window i - W < j <= i.
//
// Operand layout.  A page of one kv head holds keys row-major [token][hd] and values
// transposed [hd][token].  Scores are computed transposed, S^T = K Q^T, so that the
// accumulator of the first product (a lane holds one query column and several keys) is,
// after exp and rounding to bf16, exactly the B operand of the second, O^T = V^T P^T,
// with V^T rows read as the A operand: no shuffle and no LDS between the two products.
// For that, the rows of the first product are a fixed permutation of a block's keys, chosen
// so that the accumulator registers of a lane hold 8 consecutive keys: then the k-slots of
// the second product are in key order and V^T is read 16 contiguous bytes at a time.
#include "common.h"
#include "no_alloc.h"

#define PAGE 64
#define LOG2E 1.4426950408889634f

// 2^x by the hardware's v_exp_f32 (2^-inf = 0).  The softmax of these kernels runs in
// base 2: scores are scaled by scale * log2(e) once, and exp(s - m) becomes 2^(s' - m').
__device__ __forceinline__ float fast_exp2(float x) { return __builtin_amdgcn_exp2f(x); }

__device__ __forceinline__ bf16x8 zero8() {
    bf16x8 z;
#pragma unroll
    for (int i = 0; i < 8; ++i) z[i] = (bf16)0.f;
    return z;
}
// 8 values V^T[dim][k .. k+7] of a page; keys at or beyond `limit` read as zero
__device__ __forceinline__ bf16x8 load_vt8(const bf16* __restrict__ vrow, int k, int limit_local) {
    bf16x8 v = *(const bf16x8*)(vrow + k);
    if (k + 8 > limit_local) {
#pragma unroll
        for (int i = 0; i < 8; ++i) if (k + i >= limit_local) v[i] = (bf16)0.f;
    }
    return v;
}
// Row c (0..31) of a 32-key score block stands for this key of the block; lane (column, g)
// then holds in acc[r] the key 16 (r / 8) + 8 g + r % 8.
__device__ __forceinline__ int key_of_row32(int c) { return 16 * (c >> 4) + 8 * ((c >> 2) & 1) + 4 * ((c >> 3) & 1) + (c & 3); }

// --------------------------------------------------------------------- prefill ------
// grid = (row tiles of 128, nkv, sequences), block = 256.  A row is a (token, q head of
// the group) pair: row = token * G + head.  Each wave owns 32 rows and walks the key
// blocks of 32 its rows can see; NB = ceil(hd / 32).
template <int NB>
__global__ __launch_bounds__(256) void attn_prefill_kernel(
    const bf16* __restrict__ q, size_t q_stride, bf16* __restrict__ out, const int* __restrict__ cu_seqlens,
    const int* __restrict__ slots, const int* __restrict__ ctx_lens, const int* __restrict__ block_table,
    int table_stride, const bf16* __restrict__ cache, int nq, int nkv, int hd, int window, float scale) {
    const int b = blockIdx.z, kvh = blockIdx.y;
    const int slot = slots[b];
    const int t0 = cu_seqlens[b], n_new = cu_seqlens[b + 1] - t0;
    const int G = nq / nkv;
    const int rows_total = n_new * G;
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int row0 = blockIdx.x * 128 + wave * 32;
    if (row0 >= rows_total) return;
    const int c = lane & 31, g = lane >> 5;
    const int row = row0 + c;
    const bool row_ok = row < rows_total;
    const int rr = row_ok ? row : rows_total - 1;
    const int tok = rr / G, head = kvh * G + rr % G;
    bf16* orow = out + ((size_t)(t0 + tok) * nq + head) * hd;
    if (slot < 0) {       // padding: no cache behind it
        if (row_ok && g == 0) for (int d = 0; d < hd; ++d) orow[d] = (bf16)0.f;
        return;
    }
    const int ctx = ctx_lens[b], start = ctx - n_new;
    const int pq = start + tok;
    const int pq_min = start + row0 / G;
    const int last_row = (row0 + 31 < rows_total ? row0 + 31 : rows_total - 1);
    const int pq_max = start + last_row / G;

    const bf16* qrow = q + (size_t)(t0 + tok) * q_stride + (size_t)head * hd;
    bf16x8 qf[2 * NB];
#pragma unroll
    for (int s = 0; s < 2 * NB; ++s) {
        const int d = s * 16 + 8 * g;
        qf[s] = (d < hd) ? *(const bf16x8*)(qrow + d) : zero8();
    }
    f32x16 acc_o[NB];
#pragma unroll
    for (int i = 0; i < NB; ++i)
#pragma unroll
        for (int r = 0; r < 16; ++r) acc_o[i][r] = 0.f;
    float m = -INFINITY, lsum = 0.f;
    const float scale2 = scale * LOG2E;

    const int* bt = block_table + (size_t)slot * table_stride;
    const size_t page_elems = (size_t)2 * nkv * PAGE * hd;
    const size_t k_off = (size_t)kvh * PAGE * hd, v_off = ((size_t)nkv + kvh) * PAGE * hd;
    int lo = 0;
    if (window > 0 && pq_min - window + 1 > 0) lo = pq_min - window + 1;
    for (int kb = (lo / 32) * 32; kb <= pq_max; kb += 32) {
        const bf16* pg = cache + (size_t)bt[kb / PAGE] * page_elems;
        const int kl = kb % PAGE;                       // 0 or 32: the block's place in its page
        const bf16* krow = pg + k_off + (size_t)(kl + key_of_row32(c)) * hd;
        f32x16 s_acc;
#pragma unroll
        for (int r = 0; r < 16; ++r) s_acc[r] = 0.f;
#pragma unroll
        for (int s = 0; s < 2 * NB; ++s) {
            const int d = s * 16 + 8 * g;
            const bf16x8 kf = (d < hd) ? *(const bf16x8*)(krow + d) : zero8();
            s_acc = __builtin_amdgcn_mfma_f32_32x32x16_bf16(kf, qf[s], s_acc, 0, 0, 0);
        }
        // s_acc[r]: key kb + 16 (r / 8) + 8 g + r % 8, query row = this lane's column
        float sv[16];
        float mx = -INFINITY;
#pragma unroll
        for (int r = 0; r < 16; ++r) {
            const int key = kb + 16 * (r >> 3) + 8 * g + (r & 7);
            const bool ok = row_ok && key <= pq && (window <= 0 || key > pq - window);
            sv[r] = ok ? s_acc[r] * scale2 : -INFINITY;
            mx = fmaxf(mx, sv[r]);
        }
        mx = fmaxf(mx, __shfl_xor(mx, 32, 64));
        const float m_new = fmaxf(m, mx);
        const float m_use = (m_new == -INFINITY) ? 0.f : m_new;
        const float corr = fast_exp2(m - m_use);
        float psum = 0.f;
        bf16x8 p1, p2;
#pragma unroll
        for (int r = 0; r < 16; ++r) {
            const float p = fast_exp2(sv[r] - m_use);
            psum += p;
            if (r < 8) p1[r] = (bf16)p; else p2[r - 8] = (bf16)p;
        }
        lsum = lsum * corr + psum;
        m = m_new;
        const int limit_local = ctx - (kb - kl);        // keys of this page at or beyond it are not written yet
#pragma unroll
        for (int i = 0; i < NB; ++i) {
#pragma unroll
            for (int r = 0; r < 16; ++r) acc_o[i][r] *= corr;
            const int dim = i * 32 + c;
            bf16x8 v1 = zero8(), v2 = zero8();
            if (dim < hd) {
                const bf16* vrow = pg + v_off + (size_t)dim * PAGE;
                v1 = load_vt8(vrow, kl + 8 * g, limit_local);
                v2 = load_vt8(vrow, kl + 16 + 8 * g, limit_local);
            }
            acc_o[i] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(v1, p1, acc_o[i], 0, 0, 0);
            acc_o[i] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(v2, p2, acc_o[i], 0, 0, 0);
        }
    }
    lsum += __shfl_xor(lsum, 32, 64);
    if (!row_ok) return;
    const float inv = lsum > 0.f ? 1.f / lsum : 0.f;
#pragma unroll
    for (int i = 0; i < NB; ++i)
#pragma unroll
        for (int r4 = 0; r4 < 4; ++r4) {
            const int d = i * 32 + 8 * r4 + 4 * g;      // acc_o[i][4 r4 + e]: dim d + e
            if (d < hd) {
                bf16x4 o;
#pragma unroll
                for (int e = 0; e < 4; ++e) o[e] = (bf16)(acc_o[i][4 * r4 + e] * inv);
                *(bf16x4*)(orow + d) = o;
            }
        }
}

// ----------------------------------------------------------- prefill through LDS ----
// The same computation with the keys and values of a page staged in LDS once per
// workgroup: grid = (row tiles of 32 NW, nkv, sequences), block = 64 NW (NW waves of 32 rows).
// The page after the current one is fetched into registers while the current one is
// multiplied, and written to the other LDS buffer afterwards.  Tiles are taken from the
// last (most keys) to the first so the long workgroups start first.
#define KPAD 8
#define VLD 72
template <int NB, int NW>
__global__ __launch_bounds__(NW * 64) __attribute__((amdgpu_waves_per_eu(NW == 4 ? 2 : 1, 2))) void attn_prefill_lds_kernel(
    const bf16* __restrict__ q, size_t q_stride, bf16* __restrict__ out, const int* __restrict__ cu_seqlens,
    const int* __restrict__ slots, const int* __restrict__ ctx_lens, const int* __restrict__ block_table,
    int table_stride, const bf16* __restrict__ cache, int nq, int nkv, int hd, int window, float scale, int pair) {
    extern __shared__ __attribute__((aligned(16))) unsigned char smem_raw[];
    const int b = blockIdx.z, kvh = blockIdx.y;
    const int slot = slots[b];
    const int t0 = cu_seqlens[b], n_new = cu_seqlens[b + 1] - t0;
    const int G = nq / nkv;
    const int rows_total = n_new * G;
    // Long tiles first when the workgroups run in several rounds; when all are resident at once
    // (`pair`), the second half of the kv heads goes from short to long, so that the two workgroups of a
    // compute unit are a long and a short one (measured at 2,048 tokens: 113 -> 99 us).
    const int tile = (pair && ((blockIdx.y * 2 / gridDim.y) & 1)) ? blockIdx.x : gridDim.x - 1 - blockIdx.x;
    if (tile * (NW * 32) >= rows_total) return;                 // the whole workgroup leaves together
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int row0 = tile * (NW * 32) + wave * 32;
    const bool wave_ok = row0 < rows_total;
    const int c = lane & 31, g = lane >> 5;
    const int row = row0 + c;
    const bool row_ok = row < rows_total;
    const int rr = row_ok ? row : rows_total - 1;
    const int tok = rr / G, head = kvh * G + rr % G;
    bf16* orow = out + ((size_t)(t0 + tok) * nq + head) * hd;
    if (slot < 0) {
        if (row_ok && g == 0) for (int d = 0; d < hd; ++d) orow[d] = (bf16)0.f;
        return;
    }
    const int ctx = ctx_lens[b], start = ctx - n_new;
    const int pq = start + tok;
    // per wave and per workgroup: the positions of the first and last query row
    const int w_last_row = (row0 + 31 < rows_total ? row0 + 31 : rows_total - 1);
    const int pq_min_w = start + (wave_ok ? row0 : rows_total - 1) / G, pq_max_w = start + w_last_row / G;
    const int g_last_row = (tile * (NW * 32) + NW * 32 - 1 < rows_total ? tile * (NW * 32) + NW * 32 - 1 : rows_total - 1);
    const int pq_min_g = start + (tile * (NW * 32)) / G, pq_max_g = start + g_last_row / G;

    const int kld = hd + KPAD;
    bf16* Ks = (bf16*)smem_raw;                          // [2][64][kld]
    bf16* Vs = Ks + 2 * PAGE * kld;                      // [2][NB * 32][VLD]

    const bf16* qrow = q + (size_t)(t0 + tok) * q_stride + (size_t)head * hd;
    bf16x8 qf[2 * NB];
#pragma unroll
    for (int s = 0; s < 2 * NB; ++s) {
        const int d = s * 16 + 8 * g;
        qf[s] = (d < hd) ? *(const bf16x8*)(qrow + d) : zero8();
    }
    f32x16 acc_o[NB];
#pragma unroll
    for (int i = 0; i < NB; ++i)
#pragma unroll
        for (int r = 0; r < 16; ++r) acc_o[i][r] = 0.f;
    float m = -INFINITY, lsum = 0.f;
    const float scale2 = scale * LOG2E;

    const int* bt = block_table + (size_t)slot * table_stride;
    const size_t page_elems = (size_t)2 * nkv * PAGE * hd;
    const size_t k_off = (size_t)kvh * PAGE * hd, v_off = ((size_t)nkv + kvh) * PAGE * hd;
    int lo = 0;
    if (window > 0 && pq_min_g - window + 1 > 0) lo = pq_min_g - window + 1;
    const int pg_first = lo / PAGE, pg_last = pq_max_g / PAGE;

    // cooperative loads: chunk id -> 8 consecutive elements of the page's K part / V^T part
    constexpr int NT = NW * 64;
    constexpr int CH = (NB * 32 * PAGE / 8 + NT - 1) / NT;  // 16-byte chunks per thread and part (NB * 32 >= hd)
    bf16x8 rk[CH], rv[CH];
    const int kchunks = PAGE * hd / 8;                   // chunks that exist in each part
    auto gload = [&](int pi) {
        const bf16* pg = cache + (size_t)bt[pi] * page_elems;
        const int limit_local = ctx - pi * PAGE;
#pragma unroll
        for (int j = 0; j < CH; ++j) {
            const int id = tid + j * NT;
            if (id < kchunks) {
                rk[j] = *(const bf16x8*)(pg + k_off + (size_t)id * 8);
                bf16x8 v = *(const bf16x8*)(pg + v_off + (size_t)id * 8);
                const int key0 = (id * 8) % PAGE;        // V^T: [dim][key]
                if (key0 + 8 > limit_local) {
#pragma unroll
                    for (int e = 0; e < 8; ++e) if (key0 + e >= limit_local) v[e] = (bf16)0.f;
                }
                rv[j] = v;
            }
        }
    };
    auto sstore = [&](int buf) {
        bf16* ks = Ks + buf * PAGE * kld;
        bf16* vs = Vs + buf * NB * 32 * VLD;
#pragma unroll
        for (int j = 0; j < CH; ++j) {
            const int id = tid + j * NT;
            if (id < kchunks) {
                const int e0 = id * 8;
                *(bf16x8*)(ks + (e0 / hd) * kld + (e0 % hd)) = rk[j];
                *(bf16x8*)(vs + (e0 / PAGE) * VLD + (e0 % PAGE)) = rv[j];
            }
        }
    };

    gload(pg_first);
    sstore(0);
    __syncthreads();
    for (int pi = pg_first; pi <= pg_last; ++pi) {
        const int buf = (pi - pg_first) & 1;
        if (pi < pg_last) gload(pi + 1);
        const bf16* ks = Ks + buf * PAGE * kld;
        const bf16* vs = Vs + buf * NB * 32 * VLD;
#pragma unroll
        for (int half = 0; half < 2; ++half) {
            const int kl = half * 32, kb = pi * PAGE + kl;
            // blocks no row of this wave can see are skipped
            if (!wave_ok || kb > pq_max_w || (window > 0 && kb + 31 <= pq_min_w - window)) continue;
            const bf16* krow = ks + (kl + key_of_row32(c)) * kld;
            f32x16 s_acc;
#pragma unroll
            for (int r = 0; r < 16; ++r) s_acc[r] = 0.f;
#pragma unroll
            for (int s = 0; s < 2 * NB; ++s) {
                const int d = s * 16 + 8 * g;
                const bf16x8 kf = (d < hd) ? *(const bf16x8*)(krow + d) : zero8();
                s_acc = __builtin_amdgcn_mfma_f32_32x32x16_bf16(kf, qf[s], s_acc, 0, 0, 0);
            }
            float sv[16];
            float mx = -INFINITY;
            // a block every row of the wave sees whole (below the diagonal, inside the window)
            // needs no mask
            const bool whole = row0 + 31 < rows_total && kb + 31 <= pq_min_w &&
                               (window <= 0 || kb > pq_max_w - window);
            // the scale is positive: the largest raw score is the largest scaled one, and the scaling rides
            // on the subtraction of the maximum (one fused multiply-add per score)
            if (whole) {
#pragma unroll
                for (int r = 0; r < 16; ++r) { sv[r] = s_acc[r]; mx = fmaxf(mx, sv[r]); }
            } else {
#pragma unroll
                for (int r = 0; r < 16; ++r) {
                    const int key = kb + 16 * (r >> 3) + 8 * g + (r & 7);
                    const bool ok = row_ok && key <= pq && (window <= 0 || key > pq - window);
                    sv[r] = ok ? s_acc[r] : -INFINITY;
                    mx = fmaxf(mx, sv[r]);
                }
            }
            mx = fmaxf(mx, __shfl_xor(mx, 32, 64)) * scale2;
            const float m_new = fmaxf(m, mx);
            const float m_use = (m_new == -INFINITY) ? 0.f : m_new;
            // the accumulators are rescaled only when some row's maximum moved
            const bool moved = __any(m_new > m);
            if (moved) {
                const float corr = fast_exp2(m - m_use);
                lsum *= corr;
#pragma unroll
                for (int i = 0; i < NB; ++i)
#pragma unroll
                    for (int r = 0; r < 16; ++r) acc_o[i][r] *= corr;
            }
            float psum = 0.f;
            bf16x8 p1, p2;
#pragma unroll
            for (int r = 0; r < 16; ++r) {
                const float p = fast_exp2(fmaf(sv[r], scale2, -m_use));
                psum += p;
                if (r < 8) p1[r] = (bf16)p; else p2[r - 8] = (bf16)p;
            }
            lsum += psum;
            m = m_new;
#pragma unroll
            for (int i = 0; i < NB; ++i) {
                const bf16* vrow = vs + (i * 32 + c) * VLD + kl + 8 * g;   // rows at or beyond hd are never filled
                bf16x8 v1 = zero8(), v2 = zero8();
                if (i * 32 + c < hd) {
                    v1 = *(const bf16x8*)(vrow);
                    v2 = *(const bf16x8*)(vrow + 16);
                }
                acc_o[i] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(v1, p1, acc_o[i], 0, 0, 0);
                acc_o[i] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(v2, p2, acc_o[i], 0, 0, 0);
            }
        }
        if (pi < pg_last) sstore(buf ^ 1);
        __syncthreads();
    }
    lsum += __shfl_xor(lsum, 32, 64);
    if (!row_ok) return;
    const float inv = lsum > 0.f ? 1.f / lsum : 0.f;
#pragma unroll
    for (int i = 0; i < NB; ++i)
#pragma unroll
        for (int r4 = 0; r4 < 4; ++r4) {
            const int d = i * 32 + 8 * r4 + 4 * g;
            if (d < hd) {
                bf16x4 o;
#pragma unroll
                for (int e = 0; e < 4; ++e) o[e] = (bf16)(acc_o[i][4 * r4 + e] * inv);
                *(bf16x4*)(orow + d) = o;
            }
        }
}

// ------------------------------------------------- prefill through an LDS ring ----
// Head sizes 64 and 128: the same computation by workgroups of 4 waves (128 rows), two to a compute
// unit, with the pages brought into a ring of two LDS stages by direct global-to-LDS loads: the page
// after the current one is in flight while this one is multiplied, nothing passes through registers and
// nothing is stored to LDS by the waves.  A stage holds the page's keys [64][HD] and values [HD][64] as
// they lie in the cache; 16-byte columns are XOR-swizzled by the row (through the choice of the global
// column a lane fetches) so that the operand reads of 16 consecutive lanes spread over the banks.  The
// workgroup's page numbers are kept in LDS (at most PF_MAX_RUN): no wave waits for a read of the block
// table behind its loads in flight.  One barrier per page.
#define PF_MAX_RUN 2048
template <int HD>
__global__ __launch_bounds__(256) __attribute__((amdgpu_waves_per_eu(2, 2))) void attn_prefill_dma_kernel(
    const bf16* __restrict__ q, size_t q_stride, bf16* __restrict__ out, const int* __restrict__ cu_seqlens,
    const int* __restrict__ slots, const int* __restrict__ ctx_lens, const int* __restrict__ block_table,
    int table_stride, const bf16* __restrict__ cache, int nq, int nkv, int window, float scale, int pair) {
    constexpr int NB = HD / 32, NW = 4;
    constexpr int KROWB = HD * 2, KCOLS = KROWB / 16;       // a key row in bytes, in 16-byte columns
    constexpr int KB = PAGE * KROWB, STAGE = 2 * KB;        // keys, then values [HD][128 bytes]
    constexpr int KINSTR = KB / 1024, NDMA = STAGE / 1024 / NW;   // wave-loads: of the keys; per wave and page
    constexpr int KROWS = 1024 / KROWB;                     // key rows per wave-load
    extern __shared__ __attribute__((aligned(1024))) unsigned char dsm[];
    int* bts = (int*)(dsm + 2 * STAGE);
    const int b = blockIdx.z, kvh = blockIdx.y;
    const int slot = slots[b];
    const int t0 = cu_seqlens[b], n_new = cu_seqlens[b + 1] - t0;
    const int G = nq / nkv;
    const int rows_total = n_new * G;
    const int tile = (pair && ((blockIdx.y * 2 / gridDim.y) & 1)) ? blockIdx.x : gridDim.x - 1 - blockIdx.x;
    if (tile * (NW * 32) >= rows_total) return;           // the whole workgroup leaves together
    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int row0 = tile * (NW * 32) + wave * 32;
    const bool wave_ok = row0 < rows_total;
    const int c = lane & 31, g = lane >> 5;
    const int row = row0 + c;
    const bool row_ok = row < rows_total;
    const int rr = row_ok ? row : rows_total - 1;
    const int tok = rr / G, head = kvh * G + rr % G;
    bf16* orow = out + ((size_t)(t0 + tok) * nq + head) * HD;
    if (slot < 0) {
        if (row_ok && g == 0) for (int d = 0; d < HD; ++d) orow[d] = (bf16)0.f;
        return;
    }
    const int ctx = ctx_lens[b], start = ctx - n_new;
    const int pq = start + tok;
    const int w_last_row = (row0 + 31 < rows_total ? row0 + 31 : rows_total - 1);
    const int pq_min_w = start + (wave_ok ? row0 : rows_total - 1) / G, pq_max_w = start + w_last_row / G;
    const int g_last_row = (tile * (NW * 32) + NW * 32 - 1 < rows_total ? tile * (NW * 32) + NW * 32 - 1 : rows_total - 1);
    const int pq_min_g = start + (tile * (NW * 32)) / G, pq_max_g = start + g_last_row / G;
    int lo = 0;
    if (window > 0 && pq_min_g - window + 1 > 0) lo = pq_min_g - window + 1;
    const int pg_first = lo / PAGE, pg_last = pq_max_g / PAGE;
    const int n_run = pg_last - pg_first + 1;               // at most PF_MAX_RUN (the launcher checks)
    const int* bt = block_table + (size_t)slot * table_stride;
    for (int i = tid; i < n_run; i += NW * 64) bts[i] = bt[pg_first + i];

    const bf16* qrow = q + (size_t)(t0 + tok) * q_stride + (size_t)head * HD;
    bf16x8 qf[2 * NB];
#pragma unroll
    for (int s = 0; s < 2 * NB; ++s) qf[s] = *(const bf16x8*)(qrow + s * 16 + 8 * g);
    f32x16 acc_o[NB];
#pragma unroll
    for (int i = 0; i < NB; ++i)
#pragma unroll
        for (int r = 0; r < 16; ++r) acc_o[i][r] = 0.f;
    float m = -INFINITY, lsum = 0.f;
    const float scale2 = scale * LOG2E;
    const size_t page_elems = (size_t)2 * nkv * PAGE * HD;
    const size_t k_off = (size_t)kvh * PAGE * HD, v_off = ((size_t)nkv + kvh) * PAGE * HD;
    // the query has arrived before the loop: a wait for it inside would also wait for the page in flight
#pragma unroll
    for (int s = 0; s < 2 * NB; ++s) asm volatile("" ::"v"(qf[s]));
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    __syncthreads();                                        // the page numbers are in LDS

    const unsigned ring_lds = (unsigned)(size_t)((__attribute__((address_space(3))) unsigned char*)dsm);
    // this lane's part of each of its wave-loads: offset in the page (elements) and in the stage (bytes)
    int goff[NDMA];
#pragma unroll
    for (int q_ = 0; q_ < NDMA; ++q_) {
        const int in_ = wave * NDMA + q_;
        if (in_ < KINSTR) {
            const int row_ = in_ * KROWS + lane / KCOLS;
            const int swz_ = KCOLS == 16 ? (row_ & 15) : ((row_ >> 1) & 7);
            goff[q_] = (int)k_off + row_ * HD + (((lane % KCOLS) ^ swz_) * 8);
        } else {
            const int row_ = (in_ - KINSTR) * 8 + (lane >> 3);
            goff[q_] = (int)v_off + row_ * PAGE + (((lane & 7) ^ ((row_ >> 1) & 7)) * 8);
        }
    }
#define PF_ISSUE(I)                                                                                          \
    do {                                                                                                     \
        const bf16* pg_ = cache + (size_t)bts[I] * page_elems;                                               \
        _Pragma("unroll") for (int q_ = 0; q_ < NDMA; ++q_) {                                                \
            const unsigned lds_ = __builtin_amdgcn_readfirstlane(ring_lds + ((I) & 1) * STAGE + (wave * NDMA + q_) * 1024); \
            asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, off" ::"s"(lds_), "v"(pg_ + goff[q_]) : "m0"); \
        }                                                                                                    \
    } while (0)

    PF_ISSUE(0);
    for (int i = 0; i < n_run; ++i) {
        const int pi = pg_first + i;
        asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
        __builtin_amdgcn_s_barrier();                 // every wave's part of page i is there; page i - 1 is done with
        asm volatile("" ::: "memory");
        if (i + 1 < n_run) PF_ISSUE(i + 1);
        const unsigned char* st = dsm + (i & 1) * STAGE;
        const bool tail_page = (pi + 1) * PAGE > ctx;      // values beyond the context are stale: read them as zero
#pragma unroll
        for (int half = 0; half < 2; ++half) {
            const int kl = half * 32, kb = pi * PAGE + kl;
            // blocks no row of this wave can see are skipped
            if (!wave_ok || kb > pq_max_w || (window > 0 && kb + 31 <= pq_min_w - window)) continue;
            const int krow = kl + key_of_row32(c);
            const int kswz_ = KCOLS == 16 ? (krow & 15) : ((krow >> 1) & 7);
            const unsigned char* kp = st + krow * KROWB;
            f32x16 sv;
#pragma unroll
            for (int r = 0; r < 16; ++r) sv[r] = 0.f;
            __builtin_amdgcn_s_setprio(1);
#pragma unroll
            for (int s = 0; s < 2 * NB; ++s) {
                const bf16x8 kf = *(const bf16x8*)(kp + (((2 * s + g) ^ kswz_) * 16));
                sv = __builtin_amdgcn_mfma_f32_32x32x16_bf16(kf, qf[s], sv, 0, 0, 0);
            }
            __builtin_amdgcn_s_setprio(0);
            const bool whole = row0 + 31 < rows_total && kb + 31 <= pq_min_w &&
                               (window <= 0 || kb > pq_max_w - window);
            if (!whole) {                                  // masked in place: only blocks at the diagonal and the window's edge
#pragma unroll
                for (int r = 0; r < 16; ++r) {
                    const int key = kb + 16 * (r >> 3) + 8 * g + (r & 7);
                    const bool ok = row_ok && key <= pq && (window <= 0 || key > pq - window);
                    sv[r] = ok ? sv[r] : -INFINITY;
                }
            }
            float mx = fmaxf(fmaxf(sv[0], sv[1]), sv[2]);
#pragma unroll
            for (int r = 3; r < 15; r += 2) mx = fmaxf(fmaxf(mx, sv[r]), sv[r + 1]);
            mx = fmaxf(mx, sv[15]);
            mx = fmaxf(mx, __shfl_xor(mx, 32, 64)) * scale2;      // the scale is positive
            const float m_new = fmaxf(m, mx);
            const float m_use = (m_new == -INFINITY) ? 0.f : m_new;
            const bool moved = __any(m_new > m);
            if (moved) {
                const float corr = fast_exp2(m - m_use);
                lsum *= corr;
#pragma unroll
                for (int i2 = 0; i2 < NB; ++i2)
#pragma unroll
                    for (int r = 0; r < 16; ++r) acc_o[i2][r] *= corr;
            }
            float ps0 = 0.f, ps1 = 0.f;
            bf16x8 p1, p2;
#pragma unroll
            for (int r = 0; r < 16; r += 2) {
                const float pa = fast_exp2(fmaf(sv[r], scale2, -m_use));
                const float pb = fast_exp2(fmaf(sv[r + 1], scale2, -m_use));
                ps0 += pa;
                ps1 += pb;
                if (r < 8) { p1[r] = (bf16)pa; p1[r + 1] = (bf16)pb; }
                else { p2[r - 8] = (bf16)pa; p2[r - 7] = (bf16)pb; }
            }
            lsum += ps0 + ps1;
            m = m_new;
            __builtin_amdgcn_s_setprio(1);
#pragma unroll
            for (int i2 = 0; i2 < NB; ++i2) {
                const int vrow = i2 * 32 + c;
                const unsigned char* vp = st + KB + vrow * 128;
                const int vswz = (vrow >> 1) & 7;
                bf16x8 v1 = *(const bf16x8*)(vp + (((kl / 8 + g) ^ vswz) * 16));
                bf16x8 v2 = *(const bf16x8*)(vp + (((kl / 8 + g + 2) ^ vswz) * 16));
                if (tail_page) {
                    // keys of this lane's two value fragments that lie inside the context; the count is made
                    // opaque here so that its compares stay inside the branch (they were computed for every page)
                    int live = ctx - (kb + 8 * g);
                    asm volatile("" : "+v"(live));
#pragma unroll
                    for (int e = 0; e < 8; ++e) {
                        if (e >= live) v1[e] = (bf16)0.f;
                        if (e + 16 >= live) v2[e] = (bf16)0.f;
                    }
                }
                acc_o[i2] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(v1, p1, acc_o[i2], 0, 0, 0);
                acc_o[i2] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(v2, p2, acc_o[i2], 0, 0, 0);
            }
            __builtin_amdgcn_s_setprio(0);
        }
    }
#undef PF_ISSUE
    lsum += __shfl_xor(lsum, 32, 64);
    if (!row_ok) return;
    const float inv = lsum > 0.f ? 1.f / lsum : 0.f;
#pragma unroll
    for (int i = 0; i < NB; ++i)
#pragma unroll
        for (int r4 = 0; r4 < 4; ++r4) {
            const int d = i * 32 + 8 * r4 + 4 * g;
            bf16x4 o;
#pragma unroll
            for (int e = 0; e < 4; ++e) o[e] = (bf16)(acc_o[i][4 * r4 + e] * inv);
            *(bf16x4*)(orow + d) = o;
        }
}

// ---------------------------------------------------------------------- decode ------
// One token per sequence.  grid = (splits, nkv * head blocks, sequences), block = 256.
// The pages a query sees are cut into `nsplit` runs; the 4 waves of a workgroup take a
// run's pages in turn and are combined in LDS in wave order.  With one split the
// workgroup writes the output; otherwise it writes (m, l, unnormalised O) for its split
// and attn_decode_combine_kernel adds the splits in split order.  NB = ceil(hd / 32).
template <int NB>
__global__ __launch_bounds__(256) __attribute__((amdgpu_waves_per_eu(NB <= 4 ? 3 : 1, NB <= 4 ? 3 : 2))) void attn_decode_kernel(
    const bf16* __restrict__ q, size_t q_stride, bf16* __restrict__ out, const int* __restrict__ slots,
    const int* __restrict__ ctx_lens, const int* __restrict__ block_table, int table_stride,
    const bf16* __restrict__ cache, int nq, int nkv, int hd, int window, float scale, int nsplit,
    float* __restrict__ part_o, float* __restrict__ part_ml) {
    extern __shared__ float lds[];
    const int G = nq / nkv, nhb = (G + 15) / 16;
    const int split = blockIdx.x, kvh = blockIdx.y / nhb, hb = blockIdx.y % nhb, b = blockIdx.z;
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int c = lane & 15, g = lane >> 4;
    const int nheads = (G - hb * 16 < 16) ? G - hb * 16 : 16;     // heads of this block
    const int head0 = kvh * G + hb * 16;
    const int slot = slots[b];
    const int ctx = slot < 0 ? 0 : ctx_lens[b];
    int lo = 0;
    if (window > 0 && ctx - window > 0) lo = ctx - window;         // the query sits at ctx - 1
    const int pg_lo = lo / PAGE, npg = ctx > 0 ? (ctx - 1) / PAGE - pg_lo + 1 : 0;
    const int pps = (npg + nsplit - 1) / nsplit;
    const int pg_begin = pg_lo + split * pps;
    int pg_end = pg_begin + pps;
    if (pg_end > pg_lo + npg) pg_end = pg_lo + npg;

    const bool head_ok = c < nheads;
    const bf16* qrow = q + (size_t)b * q_stride + (size_t)(head0 + (head_ok ? c : 0)) * hd;
    bf16x8 qf[NB];
#pragma unroll
    for (int s = 0; s < NB; ++s) {
        const int d = s * 32 + 8 * g;
        qf[s] = (head_ok && d < hd) ? *(const bf16x8*)(qrow + d) : zero8();
    }
    f32x4 acc_o[2 * NB];
#pragma unroll
    for (int i = 0; i < 2 * NB; ++i)
#pragma unroll
        for (int r = 0; r < 4; ++r) acc_o[i][r] = 0.f;
    float m = -INFINITY, lsum = 0.f;
    const float scale2 = scale * LOG2E;
    const int* bt = block_table + (size_t)(slot < 0 ? 0 : slot) * table_stride;
    const size_t page_elems = (size_t)2 * nkv * PAGE * hd;
    const size_t k_off = (size_t)kvh * PAGE * hd, v_off = ((size_t)nkv + kvh) * PAGE * hd;

    for (int pi = pg_begin + wave; pi < pg_end; pi += 4) {
        const bf16* pg = cache + (size_t)bt[pi] * page_elems;
        const int pos0 = pi * PAGE;
        const int limit_local = ctx - pos0;
#pragma unroll
        for (int half = 0; half < 2; ++half) {
            const int kl = half * 32, kb = pos0 + kl;
            if (kb >= ctx || kb + 32 <= lo) continue;
            // every load of the block is issued before the first product: keys and values
            // arrive in one memory round trip instead of two
            bf16x8 kf[2][NB], vf[2 * NB];
#pragma unroll
            for (int j = 0; j < 2; ++j) {
                // row c of score block j stands for key 8 (c / 4) + 4 j + c % 4 of the 32
                const bf16* krow = pg + k_off + (size_t)(kl + 8 * (c >> 2) + 4 * j + (c & 3)) * hd;
#pragma unroll
                for (int s = 0; s < NB; ++s) {
                    const int d = s * 32 + 8 * g;
                    kf[j][s] = (d < hd) ? *(const bf16x8*)(krow + d) : zero8();
                }
            }
#pragma unroll
            for (int i = 0; i < 2 * NB; ++i) {
                const int dim = i * 16 + c;
                vf[i] = zero8();
                if (dim < hd) {
                    const bf16* vrow = pg + v_off + (size_t)dim * PAGE;
                    vf[i] = load_vt8(vrow, kl + 8 * g, limit_local);
                }
            }
            f32x4 s_acc[2];
#pragma unroll
            for (int j = 0; j < 2; ++j) {
#pragma unroll
                for (int r = 0; r < 4; ++r) s_acc[j][r] = 0.f;
#pragma unroll
                for (int s = 0; s < NB; ++s)
                    s_acc[j] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(kf[j][s], qf[s], s_acc[j], 0, 0, 0);
            }
            // s_acc[j][r]: key kb + 8 g + 4 j + r, head = this lane's column
            float sv[8];
            float mx = -INFINITY;
#pragma unroll
            for (int e = 0; e < 8; ++e) {
                const int key = kb + 8 * g + e;
                const bool ok = key >= lo && key < ctx;
                sv[e] = ok ? s_acc[e >> 2][e & 3] * scale2 : -INFINITY;
                mx = fmaxf(mx, sv[e]);
            }
            mx = fmaxf(mx, __shfl_xor(mx, 16, 64));
            mx = fmaxf(mx, __shfl_xor(mx, 32, 64));
            const float m_new = fmaxf(m, mx);           // finite: the block holds at least one visible key
            const float corr = fast_exp2(m - m_new);
            float psum = 0.f;
            bf16x8 pf;
#pragma unroll
            for (int e = 0; e < 8; ++e) {
                const float p = fast_exp2(sv[e] - m_new);
                psum += p;
                pf[e] = (bf16)p;
            }
            lsum = lsum * corr + psum;
            m = m_new;
#pragma unroll
            for (int i = 0; i < 2 * NB; ++i) {
#pragma unroll
                for (int r = 0; r < 4; ++r) acc_o[i][r] *= corr;
                acc_o[i] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(vf[i], pf, acc_o[i], 0, 0, 0);
            }
        }
    }
    lsum += __shfl_xor(lsum, 16, 64);
    lsum += __shfl_xor(lsum, 32, 64);
    // LDS: per wave [16 heads][hd] O, then [16] m, [16] l
    const int wstride = 16 * hd + 32;
    float* my = lds + wave * wstride;
#pragma unroll
    for (int i = 0; i < 2 * NB; ++i)
#pragma unroll
        for (int r = 0; r < 4; ++r) {
            const int d = i * 16 + 4 * g + r;           // acc_o[i][r]: dim d, head c
            if (d < hd) my[c * hd + d] = acc_o[i][r];
        }
    if (g == 0) { my[16 * hd + c] = m; my[16 * hd + 16 + c] = lsum; }
    __syncthreads();
    for (int e = threadIdx.x; e < nheads * hd; e += 256) {
        const int h = e / hd, d = e - h * hd;
        float M = -INFINITY;
#pragma unroll
        for (int w = 0; w < 4; ++w) M = fmaxf(M, lds[w * wstride + 16 * hd + h]);
        float L = 0.f, O = 0.f;
        if (M > -INFINITY) {
#pragma unroll
            for (int w = 0; w < 4; ++w) {
                const float f = fast_exp2(lds[w * wstride + 16 * hd + h] - M);
                L += lds[w * wstride + 16 * hd + 16 + h] * f;
                O += lds[w * wstride + h * hd + d] * f;
            }
        }
        const int head = head0 + h;
        if (nsplit == 1) {
            out[((size_t)b * nq + head) * hd + d] = (bf16)(L > 0.f ? O / L : 0.f);
        } else {
            const size_t pidx = ((size_t)b * nq + head) * nsplit + split;
            part_o[pidx * hd + d] = O;
            if (d == 0) { part_ml[pidx * 2] = M; part_ml[pidx * 2 + 1] = L; }
        }
    }
}

// The same through LDS, for head sizes 64 and 128.  The workgroup brings whole pages of its
// kv head (keys 64 x hd, values hd x 64: two contiguous blocks) into a ring of S stages
// with direct global-to-LDS loads, 1 KB per wave-load, the next pages in flight while one
// is multiplied; one barrier per page.  The 4 waves share a page as (key half, dim half):
// a wave computes the scores of its 32 keys (both waves of a key half do, and get the same
// m and l) and the output of its hd / 2 dims; the two key halves of a dim half are merged
// in LDS at the end, first half first.  16-byte columns are XOR-swizzled by the row so that
// operand reads spread over the banks; the swizzle is applied by the choice of the global
// column a lane fetches.
__device__ __forceinline__ int kswz(int row, int cols) {      // the 16 key rows of a score block differ in bits 0,1,3,4
    return cols == 16 ? (((row >> 3) & 3) * 4 + (row & 3)) : (((row >> 3) & 1) * 4 + (row & 3));
}

#define DEC_MAX_RUN 1024      // pages of one workgroup's run whose numbers are kept in LDS

//
// FUSE: the step's rotation and cache write are done here instead of by rope_kv_write (one
// kernel less per layer).  `q` then points at the step's raw rows [q heads | k heads | v
// heads]; sequence b's token stands at position ctx - 1 and its angles in row b of cs / sn
// ([B, HD / 2], pairs (p, p + HD / 2); null = no rotation).  Every workgroup rotates its
// query heads in registers; the workgroup whose run holds the last page first stores the
// rotated key and the value of the new token in that page (when `write_cache`), and waits
// for the stores before the page is fetched.  For groups of up to 16 heads, so that one
// workgroup alone reads that page.
// `qruns` (FUSE only; null = none): the step's raw rows have not been put together yet; they are
// the sums of `runs` float matrices [B, (nq + 2 nkv) HD], `run_stride` elements apart, as a
// product cut along k leaves them.  Every value read from `q` is then the runs' sum in run
// order, rounded to bf16: the bits the product's own sum kernel would have stored.
template <int HD, int S, bool FUSE>
__global__ __launch_bounds__(256) void attn_decode_lds_kernel(
    const bf16* __restrict__ q, size_t q_stride, bf16* __restrict__ out, const int* __restrict__ slots,
    const int* __restrict__ ctx_lens, const int* __restrict__ block_table, int table_stride,
    bf16* __restrict__ cache, int nq, int nkv, int window, float scale, int nsplit,
    float* __restrict__ part_o, float* __restrict__ part_ml, const float* __restrict__ cs,
    const float* __restrict__ sn, int write_cache, const float* __restrict__ qruns, int runs, size_t run_stride) {
    constexpr int NB = HD / 32;                      // 32-wide k-steps of the score product
    constexpr int KROWB = HD * 2, KCOLS = KROWB / 16; // a key row in bytes, in 16-byte columns
    constexpr int KB = PAGE * KROWB, STAGE = 2 * KB;  // keys, then values [HD][128 bytes]
    constexpr int KINSTR = KB / 1024, NDMA = STAGE / 1024 / 4;   // wave-loads: of the keys; per wave and page
    constexpr int KROWS = 1024 / KROWB;              // key rows per wave-load
    constexpr int OB = HD / 2 / 16;                  // 16-dim output blocks of a wave
    constexpr int D = S - 1;
    static_assert(S >= 2 && S <= 4 && (D - 1) * NDMA <= 63, "ring");
    extern __shared__ __attribute__((aligned(1024))) unsigned char dsm[];
    int* bts = (int*)(dsm + S * STAGE);
    const int G = nq / nkv, nhb = (G + 15) / 16;
    const int split = blockIdx.x, kvh = blockIdx.y / nhb, hb = blockIdx.y % nhb, b = blockIdx.z;
    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int c = lane & 15, g = lane >> 4;
    const int kh = wave & 1, dh = wave >> 1;
    const int nheads = (G - hb * 16 < 16) ? G - hb * 16 : 16;
    const int head0 = kvh * G + hb * 16;
    const int slot = slots[b];
    const int ctx = slot < 0 ? 0 : ctx_lens[b];
    int lo = 0;
    if (window > 0 && ctx - window > 0) lo = ctx - window;
    const int pg_lo = lo / PAGE, npg = ctx > 0 ? (ctx - 1) / PAGE - pg_lo + 1 : 0;
    const int pps = (npg + nsplit - 1) / nsplit;
    const int pg_begin = pg_lo + split * pps;
    int pg_end = pg_begin + pps;
    if (pg_end > pg_lo + npg) pg_end = pg_lo + npg;
    const int n_run = pg_end > pg_begin ? pg_end - pg_begin : 0;          // at most DEC_MAX_RUN (the launcher checks)

    const int* bt = block_table + (size_t)(slot < 0 ? 0 : slot) * table_stride;
    for (int i = tid; i < n_run; i += 256) bts[i] = bt[pg_begin + i];
    const bool head_ok = c < nheads;
    const bf16* qrow = q + (size_t)b * q_stride + (size_t)(head0 + (head_ok ? c : 0)) * HD;
    bf16x8 qf[NB];
    const size_t run_ld = (size_t)(nq + 2 * nkv) * HD;
    if (FUSE && qruns) {
        // four runs' loads at a time, so that they are in flight together; a run beyond the last adds +0
        const float* pr = qruns + (size_t)b * run_ld + (size_t)(head0 + (head_ok ? c : 0)) * HD + 8 * g;
        f32x4 lo[NB], hi[NB];
#pragma unroll
        for (int s = 0; s < NB; ++s) lo[s] = hi[s] = f32x4{0.f, 0.f, 0.f, 0.f};
        for (int p0 = 0; head_ok && p0 < runs; p0 += 4) {       // lanes without a head load nothing
            f32x4 l[NB][4], h[NB][4];
#pragma unroll
            for (int s = 0; s < NB; ++s)
#pragma unroll
                for (int j = 0; j < 4; ++j) {
                    const bool on = p0 + j < runs;
                    const float* a = pr + (size_t)(on ? p0 + j : 0) * run_stride + s * 32;
                    l[s][j] = *(const f32x4*)a;
                    h[s][j] = *(const f32x4*)(a + 4);
                    if (!on) l[s][j] = h[s][j] = f32x4{0.f, 0.f, 0.f, 0.f};
                }
#pragma unroll
            for (int s = 0; s < NB; ++s)
#pragma unroll
                for (int j = 0; j < 4; ++j) { lo[s] += l[s][j]; hi[s] += h[s][j]; }
        }
#pragma unroll
        for (int s = 0; s < NB; ++s)
#pragma unroll
            for (int e = 0; e < 4; ++e) {
                qf[s][e] = head_ok ? (bf16)lo[s][e] : (bf16)0.f;
                qf[s][4 + e] = head_ok ? (bf16)hi[s][e] : (bf16)0.f;
            }
    } else {
#pragma unroll
        for (int s = 0; s < NB; ++s) qf[s] = head_ok ? *(const bf16x8*)(qrow + s * 32 + 8 * g) : zero8();
    }
    const size_t page_elems = (size_t)2 * nkv * PAGE * HD;
    const size_t k_off = (size_t)kvh * PAGE * HD, v_off = ((size_t)nkv + kvh) * PAGE * HD;
    if constexpr (FUSE) {
        constexpr int P = HD / 2;
        if (cs) {
            // this lane holds dims 32 s + 8 g + e; their partners are NB / 2 fragments on
#pragma unroll
            for (int s = 0; s < NB / 2; ++s) {
                const float* cp = cs + (size_t)b * P + s * 32 + 8 * g;
                const float* sp = sn + (size_t)b * P + s * 32 + 8 * g;
#pragma unroll
                for (int v4 = 0; v4 < 2; ++v4) {
                    const f32x4 cc = *(const f32x4*)(cp + 4 * v4), ss = *(const f32x4*)(sp + 4 * v4);
#pragma unroll
                    for (int e = 0; e < 4; ++e) {
                        const float a = (float)qf[s][4 * v4 + e], bb = (float)qf[s + NB / 2][4 * v4 + e];
                        qf[s][4 * v4 + e] = (bf16)(a * cc[e] - bb * ss[e]);
                        qf[s + NB / 2][4 * v4 + e] = (bf16)(a * ss[e] + bb * cc[e]);
                    }
                }
            }
        }
        const int last_pg = ctx > 0 ? (ctx - 1) / PAGE : -1;
        if (write_cache && hb == 0 && last_pg >= pg_begin && last_pg < pg_end) {
            const int off = (ctx - 1) % PAGE;
            bf16* pg = cache + (size_t)bt[last_pg] * page_elems;
            const size_t kcol = (size_t)(nq + kvh) * HD, vcol = kcol + (size_t)nkv * HD;
            // element `col` of sequence b's raw row, from the row or from the runs
            auto raw = [&](size_t col) -> bf16 {
                if (!qruns) return q[(size_t)b * q_stride + col];
                const float* a = qruns + (size_t)b * run_ld + col;
                float v = 0.f;
                for (int p0 = 0; p0 < runs; p0 += 4) {
                    float t[4];
#pragma unroll
                    for (int j = 0; j < 4; ++j) {
                        t[j] = a[(size_t)(p0 + j < runs ? p0 + j : 0) * run_stride];
                        if (p0 + j >= runs) t[j] = 0.f;
                    }
#pragma unroll
                    for (int j = 0; j < 4; ++j) v += t[j];
                }
                return (bf16)v;
            };
            if (tid < P) {
                const float a = (float)raw(kcol + tid), bb = (float)raw(kcol + tid + P);
                const float cc = cs ? cs[(size_t)b * P + tid] : 1.f, ss = cs ? sn[(size_t)b * P + tid] : 0.f;
                pg[k_off + (size_t)off * HD + tid] = (bf16)(a * cc - bb * ss);
                pg[k_off + (size_t)off * HD + tid + P] = (bf16)(a * ss + bb * cc);
            } else if (tid < P + HD) {
                const int d = tid - P;
                pg[v_off + (size_t)d * PAGE + off] = raw(vcol + d);
            }
        }
        // __syncthreads below waits for these stores (they have reached the L2) before any page is fetched
    }
    // the query has arrived before the loop: a wait for it inside would also wait for the pages in flight
#pragma unroll
    for (int s = 0; s < NB; ++s) asm volatile("" ::"v"(qf[s]));
    if constexpr (FUSE) asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    __syncthreads();

    const unsigned ring_lds = (unsigned)(size_t)((__attribute__((address_space(3))) unsigned char*)dsm);
#define DEC_ISSUE(I)                                                                                         \
    do {                                                                                                     \
        const bf16* pg_ = cache + (size_t)bts[I] * page_elems;                                               \
        _Pragma("unroll") for (int q_ = 0; q_ < NDMA; ++q_) {                                                \
            const int in_ = wave * NDMA + q_;                                                                \
            const bf16* gp_;                                                                                 \
            if (in_ < KINSTR) {                                                                              \
                const int row_ = in_ * KROWS + lane / KCOLS;                                                 \
                gp_ = pg_ + k_off + (size_t)row_ * HD + (((lane % KCOLS) ^ kswz(row_, KCOLS)) * 8);          \
            } else {                                                                                         \
                const int row_ = (in_ - KINSTR) * 8 + (lane >> 3);                                           \
                gp_ = pg_ + v_off + (size_t)row_ * PAGE + (((lane & 7) ^ ((row_ >> 1) & 7)) * 8);            \
            }                                                                                                \
            const unsigned lds_ = __builtin_amdgcn_readfirstlane(ring_lds + ((I) % S) * STAGE + in_ * 1024); \
            asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, off nt" ::"s"(lds_), "v"(gp_) : "m0"); \
        }                                                                                                    \
    } while (0)

    f32x4 acc_o[OB];
#pragma unroll
    for (int i = 0; i < OB; ++i)
#pragma unroll
        for (int r = 0; r < 4; ++r) acc_o[i][r] = 0.f;
    float m = -INFINITY, lsum = 0.f;
    const float scale2 = scale * LOG2E;

    for (int j = 0; j < D; ++j)
        if (j < n_run) DEC_ISSUE(j);
    for (int i = 0; i < n_run; ++i) {
        // page i has landed when at most the loads of the pages after it are in flight
        int after = n_run - 1 - i;
        if (after > D - 1) after = D - 1;
        if (after >= 2) asm volatile("s_waitcnt vmcnt(%0)" ::"n"(2 * NDMA) : "memory");
        else if (after == 1) asm volatile("s_waitcnt vmcnt(%0)" ::"n"(NDMA) : "memory");
        else asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
        __builtin_amdgcn_s_barrier();                 // every wave's part of page i is there; page i - 1 is done with
        asm volatile("" ::: "memory");
        if (i + D < n_run) DEC_ISSUE(i + D);
        const unsigned char* st = dsm + (i % S) * STAGE;
        const int kb = (pg_begin + i) * PAGE + 32 * kh;        // position of this wave's first key
        if (kb >= ctx || kb + 32 <= lo) continue;
        f32x4 s_acc[2];
#pragma unroll
        for (int j = 0; j < 2; ++j) {
#pragma unroll
            for (int r = 0; r < 4; ++r) s_acc[j][r] = 0.f;
            // row c of score block j stands for key 8 (c / 4) + 4 j + c % 4 of the 32
            const int row = 32 * kh + 8 * (c >> 2) + 4 * j + (c & 3);
#pragma unroll
            for (int s = 0; s < NB; ++s) {
                const bf16x8 kf = *(const bf16x8*)(st + row * KROWB + (((4 * s + g) ^ kswz(row, KCOLS)) * 16));
                s_acc[j] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(kf, qf[s], s_acc[j], 0, 0, 0);
            }
        }
        // s_acc[j][r]: key kb + 8 g + 4 j + r, head = this lane's column
        float sv[8];
        float mx = -INFINITY;
#pragma unroll
        for (int e = 0; e < 8; ++e) {
            const int key = kb + 8 * g + e;
            const bool ok = key >= lo && key < ctx;
            sv[e] = ok ? s_acc[e >> 2][e & 3] * scale2 : -INFINITY;
            mx = fmaxf(mx, sv[e]);
        }
        mx = fmaxf(mx, __shfl_xor(mx, 16, 64));
        mx = fmaxf(mx, __shfl_xor(mx, 32, 64));
        const float m_new = fmaxf(m, mx);             // finite: the block holds at least one visible key
        const float corr = fast_exp2(m - m_new);
        float psum = 0.f;
        bf16x8 pf;
#pragma unroll
        for (int e = 0; e < 8; ++e) {
            const float p = fast_exp2(sv[e] - m_new);
            psum += p;
            pf[e] = (bf16)p;
        }
        lsum = lsum * corr + psum;
        m = m_new;
        const bool tail = kb + 32 > ctx;              // values beyond the context are stale: read them as zero
#pragma unroll
        for (int i2 = 0; i2 < OB; ++i2) {
            const int row = dh * (HD / 2) + 16 * i2 + c;
            bf16x8 vf = *(const bf16x8*)(st + KB + row * 128 + (((4 * kh + g) ^ ((row >> 1) & 7)) * 16));
            if (tail) {
#pragma unroll
                for (int e = 0; e < 8; ++e) if (kb + 8 * g + e >= ctx) vf[e] = (bf16)0.f;
            }
#pragma unroll
            for (int r = 0; r < 4; ++r) acc_o[i2][r] *= corr;
            acc_o[i2] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(vf, pf, acc_o[i2], 0, 0, 0);
        }
    }
#undef DEC_ISSUE
    lsum += __shfl_xor(lsum, 16, 64);
    lsum += __shfl_xor(lsum, 32, 64);
    __syncthreads();                                  // the ring is free: the waves' results meet in it
    // per wave: O [16 heads][HD / 2], then m [16], l [16]
    constexpr int WST = 16 * (HD / 2) + 32;
    float* lds = (float*)dsm;
    float* my = lds + wave * WST;
#pragma unroll
    for (int i2 = 0; i2 < OB; ++i2)
#pragma unroll
        for (int r = 0; r < 4; ++r) my[c * (HD / 2) + 16 * i2 + 4 * g + r] = acc_o[i2][r];    // dim 16 i2 + 4 g + r of the half, head c
    if (g == 0) { my[16 * (HD / 2) + c] = m; my[16 * (HD / 2) + 16 + c] = lsum; }
    __syncthreads();
    for (int e = tid; e < nheads * HD; e += 256) {
        const int h = e / HD, d = e - h * HD;
        const int w0 = 2 * (d / (HD / 2)), dd = d % (HD / 2);          // the dim half's waves: key halves 0 and 1
        const float m0 = lds[w0 * WST + 16 * (HD / 2) + h], m1 = lds[(w0 + 1) * WST + 16 * (HD / 2) + h];
        const float M = fmaxf(m0, m1);
        float L = 0.f, O = 0.f;
        if (M > -INFINITY) {
            const float f0 = fast_exp2(m0 - M), f1 = fast_exp2(m1 - M);
            L = lds[w0 * WST + 16 * (HD / 2) + 16 + h] * f0 + lds[(w0 + 1) * WST + 16 * (HD / 2) + 16 + h] * f1;
            O = lds[w0 * WST + h * (HD / 2) + dd] * f0 + lds[(w0 + 1) * WST + h * (HD / 2) + dd] * f1;
        }
        const int head = head0 + h;
        if (nsplit == 1) {
            out[((size_t)b * nq + head) * HD + d] = (bf16)(L > 0.f ? O / L : 0.f);
        } else {
            const size_t pidx = ((size_t)b * nq + head) * nsplit + split;
            part_o[pidx * HD + d] = O;
            if (d == 0) { part_ml[pidx * 2] = M; part_ml[pidx * 2 + 1] = L; }
        }
    }
}

// grid = (nq, sequences), block = 256: the splits of one head are added by four waves, wave w taking
// the splits s = w, w + 4, ... in that order and the four sums being added in wave order, so the
// result depends on nsplit only.  The weights 2^(m_s - M) are computed once into LDS.
#define COMBINE_MAX_SPLIT 1024
__global__ __launch_bounds__(256) void attn_decode_combine_kernel(const float* __restrict__ part_o,
                                                                  const float* __restrict__ part_ml,
                                                                  bf16* __restrict__ out, int nq, int hd, int nsplit) {
    __shared__ float wgt[COMBINE_MAX_SPLIT];
    __shared__ float red[4];
    __shared__ float psum[4][64];
    const int head = blockIdx.x, b = blockIdx.y, tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const size_t base = ((size_t)b * nq + head) * nsplit;
    float m = -INFINITY;
    for (int s = tid; s < nsplit; s += 256) m = fmaxf(m, part_ml[(base + s) * 2]);
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) m = fmaxf(m, __shfl_xor(m, o));
    if (lane == 0) red[wave] = m;
    __syncthreads();
    const float M = fmaxf(fmaxf(red[0], red[1]), fmaxf(red[2], red[3]));
    __syncthreads();
    float l = 0.f;
    for (int s = tid; s < nsplit; s += 256) {
        const float w = M > -INFINITY ? fast_exp2(part_ml[(base + s) * 2] - M) : 0.f;
        wgt[s] = w;
        l += part_ml[(base + s) * 2 + 1] * w;
    }
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) l += __shfl_xor(l, o);
    if (lane == 0) red[wave] = l;
    __syncthreads();
    const float L = ((red[0] + red[1]) + red[2]) + red[3];
    for (int d0 = 0; d0 < hd; d0 += 64) {
        const int d = d0 + lane;
        float O = 0.f;
        if (d < hd) {
            const float* po = part_o + base * hd + d;
#pragma unroll 4
            for (int s = wave; s < nsplit; s += 4) O += po[(size_t)s * hd] * wgt[s];
        }
        psum[wave][lane] = O;
        __syncthreads();
        if (wave == 0 && d < hd) {
            const float sum = ((psum[0][lane] + psum[1][lane]) + psum[2][lane]) + psum[3][lane];
            out[((size_t)b * nq + head) * hd + d] = (bf16)(L > 0.f ? sum / L : 0.f);
        }
        __syncthreads();
    }
}

static int nb_of(int hd) { return (hd + 31) / 32; }

extern "C" int br_attn_prefill_bf16(const void* q, size_t q_stride, void* out, const int* cu_seqlens,
                                    const int* slots, const int* ctx_lens, const int* block_table,
                                    int table_stride, const void* cache, int B, int max_new, int nq, int nkv,
                                    int hd, int page, int window, float scale, int variant, hipStream_t s) {
    if (B <= 0 || max_new <= 0) return BR_OK;
    if (nq <= 0 || nkv <= 0 || nq % nkv || hd <= 0 || hd % 16 || hd > 256 || page != PAGE || window < 0 ||
        q_stride % 8 || ((uintptr_t)q % 16) || nkv > 65535 || B > 65535 || !(scale > 0.f))
        return BR_BAD_ARG;
    const int G = nq / nkv;
    // variant 0: choose; 1: fragments straight from the cache; 2: pages staged in LDS by workgroups of
    // 8 waves; 3: the same by workgroups of 4 waves; 4: pages brought into an LDS ring by direct loads
    // (head sizes 64 and 128, block tables of at most PF_MAX_RUN pages)
    const bool dma_ok = (hd == 64 || hd == 128) && table_stride <= PF_MAX_RUN && (uintptr_t)cache % 16 == 0;
    if (variant < 0 || variant > 4 || (variant == 4 && !dma_ok)) return BR_BAD_ARG;
    // (up to head size 128 two such workgroups fit a compute unit and fill each other's gaps between the
    // page barriers: 18 to 21 % faster at 8,192 tokens; beyond 128 four waves spill registers, beyond 192 eight do)
    // Short steps too: 16 to 64 new tokens over 1,024 to 8,192 earlier ones run 2.5 to 3 times faster through
    // LDS than with the fragments straight from the cache, which remains for head sizes beyond 192.
    if (variant == 0) variant = dma_ok ? 4 : hd <= 128 ? 3 : hd <= 192 ? 2 : 1;
    if (variant == 4) {
        dim3 grid4(((size_t)max_new * G + 127) / 128, nkv, B);
        const int cus = br_device_cus();
        const int pair = cus > 0 && (long long)grid4.x * nkv * B <= 2LL * cus;
#define BR_PREFILL_DMA(HD_)                                                                                \
    do {                                                                                                   \
        auto kern = attn_prefill_dma_kernel<HD_>;                                                          \
        constexpr size_t lds4 = (size_t)2 * 2 * PAGE * HD_ * 2 + PF_MAX_RUN * sizeof(int);                 \
        static bool set = false;                                                                           \
        if (!set) {                                                                                        \
            if (hipFuncSetAttribute((const void*)kern, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds4) != hipSuccess) \
                return BR_LAUNCH_FAILED;                                                                   \
            set = true;                                                                                    \
        }                                                                                                  \
        kern<<<grid4, 256, lds4, s>>>((const bf16*)q, q_stride, (bf16*)out, cu_seqlens, slots, ctx_lens,  \
                                      block_table, table_stride, (const bf16*)cache, nq, nkv, window,      \
                                      scale, pair);                                                        \
    } while (0)
        if (hd == 128) BR_PREFILL_DMA(128); else BR_PREFILL_DMA(64);
#undef BR_PREFILL_DMA
        return br_check_launch();
    }
    if (variant == 2 || variant == 3) {
        const int variant_waves = variant == 3 ? 4 : 8;
        const int nw = variant_waves;
        dim3 grid2(((size_t)max_new * G + nw * 32 - 1) / (nw * 32), nkv, B);
        const int cus = br_device_cus();
        const int pair = nw == 4 && cus > 0 && (long long)grid2.x * nkv * B <= 2LL * cus;
        const int nb = nb_of(hd) == 5 ? 6 : (nb_of(hd) == 7 ? 8 : nb_of(hd));
        const size_t lds = (size_t)2 * (PAGE * (hd + KPAD) + nb * 32 * VLD) * sizeof(bf16);
#define BR_PREFILL_LDS(N) do { if (nw == 4) BR_PREFILL_LDS2(N, 4); else BR_PREFILL_LDS2(N, 8); } while (0)
#define BR_PREFILL_LDS2(N, NW_)                                                                            \
    do {                                                                                                   \
        auto kern = attn_prefill_lds_kernel<N, NW_>;                                                       \
        static bool set = false;                                                                           \
        if (!set) {                                                                                        \
            if (hipFuncSetAttribute((const void*)kern, hipFuncAttributeMaxDynamicSharedMemorySize,         \
                                    (int)((size_t)2 * (PAGE * (N * 32 + KPAD) + N * 32 * VLD) * 2)) != hipSuccess) \
                return BR_LAUNCH_FAILED;                                                                   \
            set = true;                                                                                    \
        }                                                                                                  \
        kern<<<grid2, NW_ * 64, lds, s>>>((const bf16*)q, q_stride, (bf16*)out, cu_seqlens, slots, ctx_lens, \
                                     block_table, table_stride, (const bf16*)cache, nq, nkv, hd, window,   \
                                     scale, pair);                                                         \
    } while (0)
        switch (nb) {
            case 1: BR_PREFILL_LDS(1); break;
            case 2: BR_PREFILL_LDS(2); break;
            case 3: BR_PREFILL_LDS(3); break;
            case 4: BR_PREFILL_LDS(4); break;
            case 6: BR_PREFILL_LDS(6); break;
            default: BR_PREFILL_LDS(8); break;
        }
#undef BR_PREFILL_LDS
#undef BR_PREFILL_LDS2
        return br_check_launch();
    }
    dim3 grid(((size_t)max_new * G + 127) / 128, nkv, B);
#define BR_PREFILL(N)                                                                                      \
    attn_prefill_kernel<N><<<grid, 256, 0, s>>>((const bf16*)q, q_stride, (bf16*)out, cu_seqlens, slots,  \
                                                 ctx_lens, block_table, table_stride, (const bf16*)cache,  \
                                                 nq, nkv, hd, window, scale)
    switch (nb_of(hd)) {
        case 1: BR_PREFILL(1); break;
        case 2: BR_PREFILL(2); break;
        case 3: BR_PREFILL(3); break;
        case 4: BR_PREFILL(4); break;
        case 5: case 6: BR_PREFILL(6); break;
        default: BR_PREFILL(8); break;
    }
#undef BR_PREFILL
    return br_check_launch();
}


// part_o: float [B, nq, nsplit, hd]; part_ml: float [B, nq, nsplit, 2] (unused when nsplit == 1)
// qruns, runs: with `fuse`, the step's raw rows as the float sums of `runs` runs of the product
// that makes them ([runs][B][(nq + 2 nkv) hd], see the kernel); null = the rows stand in `q`.
static int attn_decode_launch(const void* q, size_t q_stride, void* out, const int* slots,
                              const int* ctx_lens, const int* block_table, int table_stride,
                              void* cache, int B, int nq, int nkv, int hd, int page, int window,
                              float scale, int nsplit, float* part_o, float* part_ml, int variant,
                              int fuse, const float* cs, const float* sn, int write_cache, const float* qruns,
                              int runs, hipStream_t s) {
    if (B <= 0) return BR_OK;
    if (qruns && (!fuse || runs < 1 || runs > 64 || (uintptr_t)qruns % 16)) return BR_BAD_ARG;
    const size_t run_stride = (size_t)B * (nq + 2 * nkv) * hd;
    if (nq <= 0 || nkv <= 0 || nq % nkv || hd <= 0 || hd % 16 || hd > 256 || page != PAGE || window < 0 ||
        q_stride % 8 || ((uintptr_t)q % 16) || nsplit < 1 || nsplit > 1024 || B > 65535 ||
        (nsplit > 1 && (!part_o || !part_ml)))
        return BR_BAD_ARG;
    const int G = nq / nkv, nhb = (G + 15) / 16;
    if ((long long)nkv * nhb > 65535) return BR_BAD_ARG;
    dim3 grid(nsplit, nkv * nhb, B);
    // variant 0: choose; 1: fragments straight from the cache; 2: pages through a ring in LDS
    // (head sizes 64 and 128, runs of at most DEC_MAX_RUN pages)
    const bool lds_ok = (hd == 64 || hd == 128) && (table_stride + nsplit - 1) / nsplit <= DEC_MAX_RUN &&
                        (uintptr_t)cache % 16 == 0;
    if (variant < 0 || variant > 2 || (variant == 2 && !lds_ok)) return BR_BAD_ARG;
    if (variant == 0) variant = lds_ok ? 2 : 1;
    // fuse: rotation and cache write inside the LDS kernel (see there); the caller asks only where it applies
    if (fuse && (variant != 2 || G > 16 || (cs && (!sn || ((uintptr_t)cs | (uintptr_t)sn) % 16)))) return BR_BAD_ARG;
    if (variant == 2) {
        // two stages leave room for two workgroups per CU; with at most one workgroup per CU
        // a third stage keeps two pages in flight instead (measured: 34 -> 32 us at 8 x 4096 tokens)
        const int cus = br_device_cus();
        const bool deep = cus > 0 && (long long)nsplit * nkv * nhb * B <= cus;
#define BR_DECODE_LDS(HD_, S_, FUSE_)                                                                          \
    do {                                                                                                        \
        auto kern = attn_decode_lds_kernel<HD_, S_, FUSE_>;                                                     \
        constexpr size_t lds2 = (size_t)S_ * 2 * PAGE * HD_ * 2 + DEC_MAX_RUN * sizeof(int);                    \
        static bool set = false;                                                                                \
        if (!set) {                                                                                             \
            if (hipFuncSetAttribute((const void*)kern, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds2)   \
                != hipSuccess)                                                                                  \
                return BR_LAUNCH_FAILED;                                                                        \
            set = true;                                                                                         \
        }                                                                                                       \
        kern<<<grid, 256, lds2, s>>>((const bf16*)q, q_stride, (bf16*)out, slots, ctx_lens, block_table,        \
                                     table_stride, (bf16*)cache, nq, nkv, window, scale, nsplit, part_o,        \
                                     part_ml, cs, sn, write_cache, qruns, runs, run_stride);                    \
    } while (0)
        if (fuse) {
            if (hd == 128) { if (deep) BR_DECODE_LDS(128, 3, true); else BR_DECODE_LDS(128, 2, true); }
            else { if (deep) BR_DECODE_LDS(64, 3, true); else BR_DECODE_LDS(64, 2, true); }
        } else {
            if (hd == 128) { if (deep) BR_DECODE_LDS(128, 3, false); else BR_DECODE_LDS(128, 2, false); }
            else { if (deep) BR_DECODE_LDS(64, 3, false); else BR_DECODE_LDS(64, 2, false); }
        }
#undef BR_DECODE_LDS
        int rc2 = br_check_launch();
        if (rc2 != BR_OK || nsplit == 1) return rc2;
        attn_decode_combine_kernel<<<dim3(nq, B), 256, 0, s>>>(part_o, part_ml, (bf16*)out, nq, hd, nsplit);
        return br_check_launch();
    }
    const size_t lds = (size_t)4 * (16 * hd + 32) * sizeof(float);
#define BR_DECODE(N)                                                                                        \
    do {                                                                                                    \
        auto kern = attn_decode_kernel<N>;                                                                  \
        if (lds > 48 * 1024) {                                                                              \
            static bool set = false;                                                                        \
            if (!set) {                                                                                     \
                if (hipFuncSetAttribute((const void*)kern, hipFuncAttributeMaxDynamicSharedMemorySize,      \
                                        (int)(4 * (16 * 256 + 32) * sizeof(float))) != hipSuccess)          \
                    return BR_LAUNCH_FAILED;                                                                \
                set = true;                                                                                 \
            }                                                                                               \
        }                                                                                                   \
        kern<<<grid, 256, lds, s>>>((const bf16*)q, q_stride, (bf16*)out, slots, ctx_lens, block_table,     \
                                    table_stride, (const bf16*)cache, nq, nkv, hd, window, scale, nsplit,   \
                                    part_o, part_ml);                                                       \
    } while (0)
    switch (nb_of(hd)) {
        case 1: BR_DECODE(1); break;
        case 2: BR_DECODE(2); break;
        case 3: BR_DECODE(3); break;
        case 4: BR_DECODE(4); break;
        case 5: case 6: BR_DECODE(6); break;
        default: BR_DECODE(8); break;
    }
#undef BR_DECODE
    int rc = br_check_launch();
    if (rc != BR_OK || nsplit == 1) return rc;
    attn_decode_combine_kernel<<<dim3(nq, B), 256, 0, s>>>(part_o, part_ml, (bf16*)out, nq, hd, nsplit);
    return br_check_launch();
}

extern "C" int br_attn_decode_bf16(const void* q, size_t q_stride, void* out, const int* slots,
                                   const int* ctx_lens, const int* block_table, int table_stride,
                                   void* cache, int B, int nq, int nkv, int hd, int page, int window,
                                   float scale, int nsplit, float* part_o, float* part_ml, int variant,
                                   int fuse, const float* cs, const float* sn, int write_cache, hipStream_t s) {
    return attn_decode_launch(q, q_stride, out, slots, ctx_lens, block_table, table_stride, cache, B, nq, nkv, hd,
                              page, window, scale, nsplit, part_o, part_ml, variant, fuse, cs, sn, write_cache,
                              nullptr, 0, s);
}

// br_attn_decode_bf16 with rotation and cache write inside (`fuse` as there) from raw rows that
// are still the float sums of the runs of their product.
extern "C" int br_attn_decode_bf16_runs(const float* qruns, int runs, void* out, const int* slots,
                                        const int* ctx_lens, const int* block_table, int table_stride,
                                        void* cache, int B, int nq, int nkv, int hd, int page, int window,
                                        float scale, int nsplit, float* part_o, float* part_ml,
                                        const float* cs, const float* sn, int write_cache, hipStream_t s) {
    if (!qruns) return BR_BAD_ARG;
    return attn_decode_launch(qruns, 8, out, slots, ctx_lens, block_table, table_stride, cache, B, nq, nkv, hd,
                              page, window, scale, nsplit, part_o, part_ml, 2, 1, cs, sn, write_cache, qruns, runs, s);
}


// ------------------------------------------------ an entry point that allocates nothing ----
// See no_alloc.h.  The scratch of the split runs lives in a device array of this file; host
// code never uses the array's name as an address (on the host it is a stand-in, not device
// memory): the address is asked for once per device and kept.
static __device__ __align__(256) float scratch[BR_NO_ALLOC_SCRATCH_FLOATS];
static float* scratch_of_device[64];

static float* no_alloc_scratch() {
    int dev = -1;
    if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= 64) {
        fprintf(stderr, "braidinfer_amd: br_attn_decode_bf16_no_alloc: no current device\n");
        return nullptr;
    }
    if (!scratch_of_device[dev]) {
        float* p = nullptr;
        hipError_t e = hipGetSymbolAddress((void**)&p, HIP_SYMBOL(scratch));
        if (e != hipSuccess || !p) {
            fprintf(stderr, "braidinfer_amd: br_attn_decode_bf16_no_alloc: hipGetSymbolAddress failed: %s\n",
                    hipGetErrorString(e));
            return nullptr;
        }
        scratch_of_device[dev] = p;
    }
    return scratch_of_device[dev];
}

extern "C" int br_attn_decode_bf16_no_alloc(const void* q, size_t q_stride, void* out, const int* slots,
                                            const int* ctx_lens, const int* block_table, int table_stride,
                                            void* cache, int B, int nq, int nkv, int hd, int page, int window,
                                            float scale, int nsplit, int variant, int fuse, const float* cs,
                                            const float* sn, int write_cache, hipStream_t s) {
    if (B <= 0) return BR_OK;
    if (nq <= 0 || hd <= 0 || nsplit < 1) return BR_BAD_ARG;
    float *part_o = nullptr, *part_ml = nullptr;
    if (nsplit > 1) {
        const unsigned long long rows = (unsigned long long)B * nq * nsplit;
        const unsigned long long o_floats = (rows * hd + 63) / 64 * 64, need = o_floats + rows * 2;
        if (need > BR_NO_ALLOC_SCRATCH_FLOATS) {
            fprintf(stderr, "braidinfer_amd: br_attn_decode_bf16_no_alloc: %d sequences x %d heads x %d runs x head size %d "
                            "need %llu floats of scratch, the array holds %u\n", B, nq, nsplit, hd, need,
                    (unsigned)BR_NO_ALLOC_SCRATCH_FLOATS);
            return BR_TOO_LARGE;
        }
        float* base = no_alloc_scratch();
        if (!base) return BR_LAUNCH_FAILED;
        part_o = base;
        part_ml = base + o_floats;
    }
    return br_attn_decode_bf16(q, q_stride, out, slots, ctx_lens, block_table, table_stride, cache, B, nq, nkv, hd,
                               page, window, scale, nsplit, part_o, part_ml, variant, fuse, cs, sn, write_cache, s);
}
