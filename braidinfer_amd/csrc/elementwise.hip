// Row-wise and element-wise kernels of a decoder step: embedding gather, RMSNorm,
// rotary tables, rotation + paged key/value write, SiLU*mul, residual add, row gather.
// Activations are `T` (float in the 32-bit path, bf16 in the serving path); the
// residual stream and all statistics are float in both.
#include "common.h"

// ------------------------------------------------------------------ embedding ------
// out[t, :] = float(table[token[t], :])            reference: op_embedding,
// kernels/megakernel_ops.hip:1757-1768 (one instruction per token there; one launch
// for all packed tokens here).  A token id outside the table writes zeros; the host
// rejects such ids before the launch.
template <typename W>
__global__ void embedding_kernel(const W* __restrict__ table, const int* __restrict__ tokens,
                                 float* __restrict__ out, int H, int V) {
    const int t = blockIdx.x;
    const int tok = tokens[t];
    float* o = out + (size_t)t * H;
    if (tok < 0 || tok >= V) {
        for (int i = threadIdx.x; i < H; i += blockDim.x) o[i] = 0.f;
        return;
    }
    const W* r = table + (size_t)tok * H;
    for (int i = threadIdx.x; i < H; i += blockDim.x) o[i] = to_f32<W>(r[i]);
}

extern "C" int br_embedding(const void* table, int table_is_bf16, const int* tokens, float* out,
                            int T, int H, int V, hipStream_t s) {
    if (T <= 0) return BR_OK;
    if (H <= 0 || V <= 0) return BR_BAD_ARG;
    int threads = H >= 1024 ? 256 : 64;
    if (table_is_bf16)
        embedding_kernel<bf16><<<T, threads, 0, s>>>((const bf16*)table, tokens, out, H, V);
    else
        embedding_kernel<float><<<T, threads, 0, s>>>((const float*)table, tokens, out, H, V);
    return br_check_launch();
}

// -------------------------------------------------------------------- RMSNorm ------
// y = x * rsqrt(mean(x^2) + eps) * w, statistics in float       reference:
// op_rmsnorm_wx, kernels/megakernel_ops.hip:862-904.  `rows` (optional) gathers:
// y[i] = norm(x[rows[i]]).  One block per row; the sum of squares is reduced by a
// fixed tree so a row's result does not depend on its neighbours.
template <typename T>
__global__ void rmsnorm_kernel(const float* __restrict__ x, const float* __restrict__ w,
                               T* __restrict__ y, const int* __restrict__ rows, int H, float eps) {
    __shared__ float scratch[16];
    const int r = blockIdx.x;
    const float* xr = x + (size_t)(rows ? rows[r] : r) * H;
    T* yr = y + (size_t)r * H;
    float ss = 0.f;
    for (int i = threadIdx.x; i < H; i += blockDim.x) { float v = xr[i]; ss += v * v; }
    const float tot = block_sum(ss, scratch);
    const float inv = rsqrtf(tot / (float)H + eps);
    for (int i = threadIdx.x; i < H; i += blockDim.x) yr[i] = from_f32<T>(xr[i] * inv * w[i]);
}

// The same for widths in steps of 4 up to 4 * 4 * blockDim: a row is read once, 16 bytes
// a load, and kept in registers between the sum and the scaling.
template <typename T, int VPT>
__global__ void rmsnorm_vec_kernel(const float* __restrict__ x, const float* __restrict__ w,
                                   T* __restrict__ y, const int* __restrict__ rows, int H, float eps) {
    __shared__ float scratch[16];
    const int r = blockIdx.x;
    const f32x4* xr = (const f32x4*)(x + (size_t)(rows ? rows[r] : r) * H);
    const f32x4* wr = (const f32x4*)w;
    T* yr = y + (size_t)r * H;
    const int nv = H >> 2;
    f32x4 v[VPT], wv[VPT];
    float ss = 0.f;
#pragma unroll
    for (int j = 0; j < VPT; ++j) {
        const int i = threadIdx.x + j * blockDim.x;
        if (i < nv) { v[j] = xr[i]; wv[j] = wr[i]; }
    }
#pragma unroll
    for (int j = 0; j < VPT; ++j) {
        const int i = threadIdx.x + j * blockDim.x;
        if (i < nv) ss += (v[j][0] * v[j][0] + v[j][1] * v[j][1]) + (v[j][2] * v[j][2] + v[j][3] * v[j][3]);
    }
    const float tot = block_sum(ss, scratch);
    const float inv = rsqrtf(tot / (float)H + eps);
#pragma unroll
    for (int j = 0; j < VPT; ++j) {
        const int i = threadIdx.x + j * blockDim.x;
        if (i < nv) {
#pragma unroll
            for (int e = 0; e < 4; ++e) yr[4 * i + e] = from_f32<T>(v[j][e] * inv * wv[j][e]);
        }
    }
}

extern "C" int br_rmsnorm(const float* x, const float* w, void* y, int y_is_bf16, const int* rows,
                          int R, int H, float eps, hipStream_t s) {
    if (R <= 0) return BR_OK;
    if (H <= 0) return BR_BAD_ARG;
    int threads = H >= 2048 ? 256 : (H >= 512 ? 128 : 64);
    const bool vec = (H % 4 == 0) && (H / 4 <= 4 * threads) && (((uintptr_t)x | (uintptr_t)w) % 16 == 0);
    if (vec) {
        if (y_is_bf16) rmsnorm_vec_kernel<bf16, 4><<<R, threads, 0, s>>>(x, w, (bf16*)y, rows, H, eps);
        else rmsnorm_vec_kernel<float, 4><<<R, threads, 0, s>>>(x, w, (float*)y, rows, H, eps);
    } else {
        if (y_is_bf16) rmsnorm_kernel<bf16><<<R, threads, 0, s>>>(x, w, (bf16*)y, rows, H, eps);
        else rmsnorm_kernel<float><<<R, threads, 0, s>>>(x, w, (float*)y, rows, H, eps);
    }
    return br_check_launch();
}

// --------------------------------------------------------------- rotary tables -----
// cos/sin[t, p] of theta = float(pos[t]) * inv_freq[p]         reference: op_mrope,
// kernels/megakernel_ops.hip:2019-2024 (cosf/sinf per element there; once per step
// here, shared by all layers).
__global__ void rope_table_kernel(const int* __restrict__ pos, const float* __restrict__ inv_freq,
                                  float* __restrict__ cs, float* __restrict__ sn, int T, int P) {
    const int i = blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= T * P) return;
    const int t = i / P, p = i - t * P;
    const float th = (float)pos[t] * inv_freq[p];
    cs[i] = cosf(th);
    sn[i] = sinf(th);
}

extern "C" int br_rope_table(const int* pos, const float* inv_freq, float* cs, float* sn, int T, int P,
                             hipStream_t s) {
    if (T <= 0 || P <= 0) return BR_OK;
    int n = T * P;
    rope_table_kernel<<<(n + 255) / 256, 256, 0, s>>>(pos, inv_freq, cs, sn, T, P);
    return br_check_launch();
}

// ------------------------------------------------- rotation + paged K/V write ------
// For token t with query/key/value rows in `qkv` ([T, (nq + 2 nkv) * hd], q heads
// first, then k heads, then v heads): rotate the first `rd` elements of every q and k
// head by the token's angle (reference: op_mrope, megakernel_ops.hip:2025-2030; pair
// (2p, 2p+1) when adjacent, (p, p + rd/2) when half), write q back in place, and store
// the rotated k and the untouched v in the token's cache page (reference:
// op_kv_write_paged_batch.hip:58-73 for the page/offset arithmetic; keys are stored
// after rotation, once).  Cache layout per unit: [page][K|V][kv_head], then keys as
// [token_in_page][hd] and values transposed, [hd][token_in_page], which is the operand
// layout of the matrix-core attention kernels.
// A token whose sequence has slot < 0 is padding: q is still rotated, nothing is stored.
// grid = (T, nq + 2 nkv), block = 64.
template <typename T>
__global__ void rope_kv_write_kernel(T* __restrict__ qkv, const float* __restrict__ cs,
                                     const float* __restrict__ sn, const int* __restrict__ pos,
                                     const int* __restrict__ seq_of_token, const int* __restrict__ slots,
                                     const int* __restrict__ block_table, int table_stride,
                                     T* __restrict__ cache, int nq, int nkv, int hd, int rd, int adjacent,
                                     int page, int write_cache) {
    const int t = blockIdx.x, h = blockIdx.y;
    const int width = (nq + 2 * nkv) * hd;
    T* src = qkv + (size_t)t * width + (size_t)h * hd;
    const bool is_q = h < nq, is_k = !is_q && h < nq + nkv;
    T* dst = nullptr;
    if (!is_q) {
        if (!write_cache) return;
        const int slot = slots[seq_of_token[t]];
        if (slot < 0) return;
        const int p = pos[t];
        const int pg = block_table[(size_t)slot * table_stride + p / page];
        const int kvh = is_k ? h - nq : h - nq - nkv;
        T* unit = cache + (((size_t)pg * 2 + (is_k ? 0 : 1)) * nkv + kvh) * page * hd;
        if (is_k) dst = unit + (size_t)(p % page) * hd;
        else {
            T* col = unit + (p % page);                  // values: element i of the head at [i][token]
            for (int i = threadIdx.x; i < hd; i += blockDim.x) col[(size_t)i * page] = src[i];
            return;
        }
    }
    if (is_q || is_k) {
        const int P = rd / 2;
        const float* c = cs ? cs + (size_t)t * P : nullptr;
        const float* s = sn ? sn + (size_t)t * P : nullptr;
        T* o = is_q ? src : dst;
        for (int p = threadIdx.x; p < P; p += blockDim.x) {
            const int i0 = adjacent ? 2 * p : p, i1 = adjacent ? 2 * p + 1 : p + P;
            const float a = to_f32<T>(src[i0]), b = to_f32<T>(src[i1]);
            const float co = c ? c[p] : 1.f, si = s ? s[p] : 0.f;
            o[i0] = from_f32<T>(a * co - b * si);
            o[i1] = from_f32<T>(a * si + b * co);
        }
        if (is_k) for (int i = rd + threadIdx.x; i < hd; i += blockDim.x) o[i] = src[i];
    }
}

// The same for many tokens (prompts), bf16, head sizes and rotary sizes in steps of 16:
// a workgroup takes 64 consecutive tokens of one head.  Rotation works on 16-byte vectors
// (8 low elements and their 8 partners at once); values go through an LDS tile so that a
// wave writes one element row of the transposed page for 64 tokens, contiguous wherever
// the tokens are neighbours in a page, instead of 2-byte stores 128 bytes apart.
// grid = (ceil(T / 64), nq + 2 nkv), block = 256.
#define RKV_TOK 64
__global__ __launch_bounds__(256) void rope_kv_write_tile_kernel(
    bf16* __restrict__ qkv, const float* __restrict__ cs, const float* __restrict__ sn, const int* __restrict__ pos,
    const int* __restrict__ seq_of_token, const int* __restrict__ slots, const int* __restrict__ block_table,
    int table_stride, bf16* __restrict__ cache, int T, int nq, int nkv, int hd, int rd, int adjacent,
    int write_cache) {
    extern __shared__ __attribute__((aligned(16))) unsigned char rkv_smem[];
    __shared__ int tok_page[RKV_TOK];      // page of the token's position, -1 if nothing is stored
    __shared__ int tok_off[RKV_TOK];       // its place in the page
    const int t0 = blockIdx.x * RKV_TOK, h = blockIdx.y, tid = threadIdx.x;
    const int nt = T - t0 < RKV_TOK ? T - t0 : RKV_TOK;
    const int width = (nq + 2 * nkv) * hd;
    const bool is_q = h < nq, is_k = !is_q && h < nq + nkv;
    if (!is_q && !write_cache) return;
    if (!is_q) {
        if (tid < RKV_TOK) {
            int pg = -1, off = 0;
            if (tid < nt) {
                const int slot = slots[seq_of_token[t0 + tid]];
                if (slot >= 0) {
                    const int p = pos[t0 + tid];
                    pg = block_table[(size_t)slot * table_stride + p / RKV_TOK];
                    off = p % RKV_TOK;
                }
            }
            tok_page[tid] = pg;
            tok_off[tid] = off;
        }
        __syncthreads();
    }
    const size_t unit = (size_t)RKV_TOK * hd;                  // elements of one head's keys (or values) in a page
    if (is_q || is_k) {
        const int kvh = h - nq;
        const int P = rd / 2;
        // work items of a token row: rotations of 8 pairs, then copies of 8 elements beyond rd
        const int nrot = adjacent ? rd / 8 : P / 8, ncopy = is_k ? (hd - rd) / 8 : 0, per = nrot + ncopy;
        for (int e = tid; e < nt * per; e += 256) {
            const int tl = e / per, w = e - tl * per, t = t0 + tl;
            const bf16* src = qkv + (size_t)t * width + (size_t)h * hd;
            bf16* dst;
            if (is_q) dst = qkv + (size_t)t * width + (size_t)h * hd;
            else {
                if (tok_page[tl] < 0) continue;
                dst = cache + ((size_t)tok_page[tl] * 2 * nkv + kvh) * unit + (size_t)tok_off[tl] * hd;
            }
            if (w >= nrot) {
                const int d = rd + (w - nrot) * 8;
                *(bf16x8*)(dst + d) = *(const bf16x8*)(src + d);
                continue;
            }
            if (adjacent) {
                const int d = w * 8;                            // pairs d / 2 .. d / 2 + 3
                const bf16x8 v = *(const bf16x8*)(src + d);
                const f32x4 c = cs ? *(const f32x4*)(cs + (size_t)t * P + d / 2) : f32x4{1.f, 1.f, 1.f, 1.f};
                const f32x4 sgn = sn ? *(const f32x4*)(sn + (size_t)t * P + d / 2) : f32x4{0.f, 0.f, 0.f, 0.f};
                bf16x8 o;
#pragma unroll
                for (int i = 0; i < 4; ++i) {
                    const float a = (float)v[2 * i], b = (float)v[2 * i + 1];
                    o[2 * i] = (bf16)(a * c[i] - b * sgn[i]);
                    o[2 * i + 1] = (bf16)(a * sgn[i] + b * c[i]);
                }
                *(bf16x8*)(dst + d) = o;
            } else {
                const int d = w * 8;                            // pairs d .. d + 7 with partners at d + P
                const bf16x8 lo = *(const bf16x8*)(src + d), hi = *(const bf16x8*)(src + d + P);
                bf16x8 olo, ohi;
#pragma unroll
                for (int v4 = 0; v4 < 2; ++v4) {
                    const f32x4 c = cs ? *(const f32x4*)(cs + (size_t)t * P + d + 4 * v4) : f32x4{1.f, 1.f, 1.f, 1.f};
                    const f32x4 sgn = sn ? *(const f32x4*)(sn + (size_t)t * P + d + 4 * v4) : f32x4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
                    for (int i = 0; i < 4; ++i) {
                        const float a = (float)lo[4 * v4 + i], b = (float)hi[4 * v4 + i];
                        olo[4 * v4 + i] = (bf16)(a * c[i] - b * sgn[i]);
                        ohi[4 * v4 + i] = (bf16)(a * sgn[i] + b * c[i]);
                    }
                }
                *(bf16x8*)(dst + d) = olo;
                *(bf16x8*)(dst + d + P) = ohi;
            }
        }
        return;
    }
    // values: [token][hd] rows into LDS (rows padded by one word against bank conflicts), then element rows out
    const int kvh = h - nq - nkv;
    const int ld = hd + 2;
    bf16* tile = (bf16*)rkv_smem;
    const int vec = hd / 8;
    for (int e = tid; e < nt * vec; e += 256) {
        const int tl = e / vec, c = e - tl * vec;
        const bf16x8 v = *(const bf16x8*)(qkv + (size_t)(t0 + tl) * width + (size_t)h * hd + c * 8);
#pragma unroll
        for (int i = 0; i < 8; i += 2) *(bf16x2*)(tile + tl * ld + c * 8 + i) = bf16x2{v[i], v[i + 1]};
    }
    __syncthreads();
    const int lane = tid & 63, wave = tid >> 6;
    if (lane < nt && tok_page[lane] >= 0) {
        bf16* col = cache + (((size_t)tok_page[lane] * 2 + 1) * nkv + kvh) * unit + tok_off[lane];
        for (int d = wave; d < hd; d += 4) col[(size_t)d * RKV_TOK] = tile[lane * ld + d];
    }
}

extern "C" int br_rope_kv_write(void* qkv, int is_bf16, const float* cs, const float* sn, const int* pos,
                                const int* seq_of_token, const int* slots, const int* block_table,
                                int table_stride, void* cache, int T, int nq, int nkv, int hd, int rd,
                                int adjacent, int page, int write_cache, hipStream_t s) {
    if (T <= 0) return BR_OK;
    if (nq <= 0 || nkv <= 0 || hd <= 0 || rd < 0 || rd > hd || (rd & 1) || page <= 0) return BR_BAD_ARG;
    if (nq + 2 * nkv > 65535) return BR_BAD_ARG;
    const bool vectors = is_bf16 && page == RKV_TOK && hd % 16 == 0 && rd % 16 == 0 &&
                         ((uintptr_t)qkv | (uintptr_t)cache | (uintptr_t)cs | (uintptr_t)sn) % 16 == 0;
    if (vectors && T >= 256) {             // fewer tokens: one workgroup per token and head fills the chip better
        dim3 grid((T + RKV_TOK - 1) / RKV_TOK, nq + 2 * nkv);
        const size_t lds = (size_t)RKV_TOK * (hd + 2) * sizeof(bf16);
        rope_kv_write_tile_kernel<<<grid, 256, lds, s>>>((bf16*)qkv, cs, sn, pos, seq_of_token, slots, block_table,
                                                        table_stride, (bf16*)cache, T, nq, nkv, hd, rd, adjacent,
                                                        write_cache);
        return br_check_launch();
    }
    dim3 grid(T, nq + 2 * nkv);
    if (is_bf16)
        rope_kv_write_kernel<bf16><<<grid, 64, 0, s>>>((bf16*)qkv, cs, sn, pos, seq_of_token, slots,
                                                       block_table, table_stride, (bf16*)cache, nq, nkv,
                                                       hd, rd, adjacent, page, write_cache);
    else
        rope_kv_write_kernel<float><<<grid, 64, 0, s>>>((float*)qkv, cs, sn, pos, seq_of_token, slots,
                                                        block_table, table_stride, (float*)cache, nq, nkv,
                                                        hd, rd, adjacent, page, write_cache);
    return br_check_launch();
}

// ------------------------------------------------------------------ SiLU * mul -----
// a[t, i] = silu(g[t, i]) * u[t, i], silu(x) = x / (1 + exp(-x)), from the fused
// gate/up output gu[t, 0:I] = g, gu[t, I:2I] = u       reference: op_silu_mul,
// kernels/megakernel_ops.hip:374-407.
template <typename T>
__global__ void silu_mul_kernel(const T* __restrict__ gu, T* __restrict__ a, int I, size_t n) {
    size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= n) return;
    size_t t = i / I, c = i - t * I;
    float g = to_f32<T>(gu[t * 2 * I + c]), u = to_f32<T>(gu[t * 2 * I + I + c]);
    a[i] = from_f32<T>(g / (1.f + expf(-g)) * u);
}

extern "C" int br_silu_mul(const void* gu, void* a, int is_bf16, int T, int I, hipStream_t s) {
    if (T <= 0 || I <= 0) return BR_OK;
    size_t n = (size_t)T * I;
    unsigned blocks = (unsigned)((n + 255) / 256);
    if (is_bf16) silu_mul_kernel<bf16><<<blocks, 256, 0, s>>>((const bf16*)gu, (bf16*)a, I, n);
    else silu_mul_kernel<float><<<blocks, 256, 0, s>>>((const float*)gu, (float*)a, I, n);
    return br_check_launch();
}

// ---------------------------------------------------------------- residual add -----
// x[i] += float(y[i])                 reference: op_residual_add, megakernel_ops.hip:1185-1212
template <typename T>
__global__ void residual_add_kernel(float* __restrict__ x, const T* __restrict__ y, size_t n) {
    size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i < n) x[i] += to_f32<T>(y[i]);
}

extern "C" int br_residual_add(float* x, const void* y, int y_is_bf16, size_t n, hipStream_t s) {
    if (n == 0) return BR_OK;
    unsigned blocks = (unsigned)((n + 255) / 256);
    if (y_is_bf16) residual_add_kernel<bf16><<<blocks, 256, 0, s>>>(x, (const bf16*)y, n);
    else residual_add_kernel<float><<<blocks, 256, 0, s>>>(x, (const float*)y, n);
    return br_check_launch();
}

// ------------------------------------------------------------------ row gather -----
// out[i, :] = x[rows[i], :] (float)   reference: D2dCopy of the last row,
// megakernel/megakernel_compile.rs:522-527.
__global__ void gather_rows_kernel(const float* __restrict__ x, const int* __restrict__ rows,
                                   float* __restrict__ out, int H) {
    const float* xr = x + (size_t)rows[blockIdx.x] * H;
    float* o = out + (size_t)blockIdx.x * H;
    for (int i = threadIdx.x; i < H; i += blockDim.x) o[i] = xr[i];
}

extern "C" int br_gather_rows(const float* x, const int* rows, float* out, int R, int H, hipStream_t s) {
    if (R <= 0 || H <= 0) return BR_OK;
    gather_rows_kernel<<<R, 128, 0, s>>>(x, rows, out, H);
    return br_check_launch();
}

// --------------------------------------------------------------- dtype convert -----
// float -> bf16 (round to nearest even) and bf16 -> float, for activations that meet a
// weight kept in the other precision.
__global__ void f32_to_bf16_kernel(const float* __restrict__ a, bf16* __restrict__ b, size_t n) {
    size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i < n) b[i] = (bf16)a[i];
}
__global__ void bf16_to_f32_kernel(const bf16* __restrict__ a, float* __restrict__ b, size_t n) {
    size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i < n) b[i] = (float)a[i];
}
extern "C" int br_convert(const void* a, void* b, int to_bf16, size_t n, hipStream_t s) {
    if (n == 0) return BR_OK;
    unsigned blocks = (unsigned)((n + 255) / 256);
    if (to_bf16) f32_to_bf16_kernel<<<blocks, 256, 0, s>>>((const float*)a, (bf16*)b, n);
    else bf16_to_f32_kernel<<<blocks, 256, 0, s>>>((const bf16*)a, (float*)b, n);
    return br_check_launch();
}

// Compute units of the current device (0 if the runtime does not say).
extern "C" int br_device_cu_count() { return br_device_cus(); }

// ------------------------------------------------------- memory-rate measurements -----
// Plain streaming kernels that say what this GPU's memory delivers to code like the
// kernels above: a copy (read + write) and a pure read whose result is one word per
// workgroup.  16 bytes a lane, consecutive lanes on consecutive addresses, grid-stride.
__global__ __launch_bounds__(256) void stream_copy_kernel(const f32x4* __restrict__ src, f32x4* __restrict__ dst, size_t n16) {
    const size_t stride = (size_t)gridDim.x * blockDim.x;
    for (size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x; i < n16; i += stride)
        dst[i] = __builtin_nontemporal_load(src + i);
}

__global__ __launch_bounds__(256) void stream_read_kernel(const f32x4* __restrict__ src, float* __restrict__ sums, size_t n16) {
    // Every workgroup reads a contiguous region of its own with non-temporal loads, eight in flight per lane:
    // 7.1 TB/s, where all workgroups walking one window forward together (grid stride) reach 6.0 to 6.3 and
    // either change alone nothing.
    const size_t per = n16 / gridDim.x;
    size_t i = (size_t)blockIdx.x * per + threadIdx.x;
    const size_t end = blockIdx.x + 1 == gridDim.x ? n16 : ((size_t)blockIdx.x + 1) * per;
    const size_t stride = blockDim.x;
    f32x4 a = {0.f, 0.f, 0.f, 0.f};
    for (; i + 7 * stride < end; i += 8 * stride) {
        f32x4 v[8];
#pragma unroll
        for (int u = 0; u < 8; ++u) v[u] = __builtin_nontemporal_load(src + i + u * stride);
        a += ((v[0] + v[1]) + (v[2] + v[3])) + ((v[4] + v[5]) + (v[6] + v[7]));
    }
    for (; i < end; i += stride) a += __builtin_nontemporal_load(src + i);
    const float t = wave_sum((a[0] + a[1]) + (a[2] + a[3]));
    if ((threadIdx.x & 63) == 0) sums[blockIdx.x * 4 + (threadIdx.x >> 6)] = t;
}

// bytes: a multiple of 16; sums: float [4 * blocks] for the read (blocks is returned through *blocks_out)
extern "C" int br_stream_copy(const void* src, void* dst, size_t bytes, hipStream_t s) {
    if (bytes == 0) return BR_OK;
    if (bytes % 16 || ((uintptr_t)src | (uintptr_t)dst) % 16) return BR_BAD_ARG;
    const int cus = br_device_cus();
    const unsigned blocks = (unsigned)((cus > 0 ? cus : 256) * 8);
    stream_copy_kernel<<<blocks, 256, 0, s>>>((const f32x4*)src, (f32x4*)dst, bytes / 16);
    return br_check_launch();
}

extern "C" int br_stream_read(const void* src, float* sums, int sums_len, size_t bytes, hipStream_t s) {
    if (bytes == 0) return BR_OK;
    const int cus = br_device_cus();
    const unsigned blocks = (unsigned)((cus > 0 ? cus : 256) * 8);
    if (bytes % 16 || (uintptr_t)src % 16 || !sums || sums_len < (int)(4 * blocks)) return BR_BAD_ARG;
    stream_read_kernel<<<blocks, 256, 0, s>>>((const f32x4*)src, sums, bytes / 16);
    return br_check_launch();
}
