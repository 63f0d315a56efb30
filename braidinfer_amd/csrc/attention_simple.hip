// Attention over the paged cache, one wave per (query token, query head), in float
// arithmetic for both storage types.  It serves prompts and single tokens alike: a
// query at position p of its sequence sees keys lo..p, lo = max(0, p - window + 1),
// all of which are in the cache when it runs (the step stores its own keys first).
//
// The sum runs over keys in ascending position, 64 at a time, with the online-softmax
// recurrence of the reference (m' = max(m, s), c = exp(m - m'), d = d c + w,
// acc = acc c + w v; kernels/megakernel_ops.hip:2310-2342), scores scaled by `scale`
// (rsqrt(head_dim) there, :2192-2194), kv head = q head / (nq / nkv) (:2192).  The
// chunking depends only on (p, window), never on how tokens were cut into steps or on
// what else is in the batch, so whole prompts and token-by-token runs agree bit for bit.
//
// This is the whole attention of the 32-bit path and the reference the matrix-core
// kernels are tested against.
#include "common.h"

#define MAX_DPL 8   // head_dim <= 64 * MAX_DPL

template <typename T>
__global__ __launch_bounds__(64) void attn_simple_kernel(
    const T* __restrict__ q, size_t q_stride, T* __restrict__ out, const int* __restrict__ pos,
    const int* __restrict__ seq_of_token, const int* __restrict__ slots,
    const int* __restrict__ block_table, int table_stride, const T* __restrict__ cache,
    int nq, int nkv, int hd, int page, int window, float scale) {
    extern __shared__ float lds[];
    float* qs = lds;            // [hd]
    float* ps = lds + hd;       // [64]
    const int t = blockIdx.x, h = blockIdx.y, lane = threadIdx.x;
    const int kvh = h / (nq / nkv);
    T* o = out + ((size_t)t * nq + h) * hd;
    const int slot = slots[seq_of_token[t]];
    if (slot < 0) {
        for (int d = lane; d < hd; d += 64) o[d] = from_f32<T>(0.f);
        return;
    }
    const T* qr = q + (size_t)t * q_stride + (size_t)h * hd;
    for (int d = lane; d < hd; d += 64) qs[d] = to_f32<T>(qr[d]);
    __syncthreads();
    const int p = pos[t];
    const int lo = (window > 0 && p - window + 1 > 0) ? p - window + 1 : 0;
    const int* bt = block_table + (size_t)slot * table_stride;
    // one page: [K|V][kvh], keys [tok][hd], values transposed [hd][tok]
    const size_t page_elems = (size_t)2 * nkv * page * hd;
    const size_t k_off = (size_t)kvh * page * hd, v_off = ((size_t)nkv + kvh) * page * hd;

    float m = -INFINITY, l = 0.f;
    float acc[MAX_DPL];
#pragma unroll
    for (int i = 0; i < MAX_DPL; ++i) acc[i] = 0.f;

    for (int j0 = lo; j0 <= p; j0 += 64) {
        const int j = j0 + lane;
        float s = -INFINITY;
        if (j <= p) {
            const T* kr = cache + (size_t)bt[j / page] * page_elems + k_off + (size_t)(j % page) * hd;
            float dot = 0.f;
            for (int d = 0; d < hd; ++d) dot = fmaf(qs[d], to_f32<T>(kr[d]), dot);
            s = dot * scale;
        }
        const float m_new = fmaxf(m, wave_max(s));
        const float corr = expf(m - m_new);          // exp(-inf) = 0 on the first chunk
        const float w = (j <= p) ? expf(s - m_new) : 0.f;
        l = l * corr + wave_sum(w);
        __syncthreads();
        ps[lane] = w;
        __syncthreads();
        const int nk = (p - j0 + 1) < 64 ? (p - j0 + 1) : 64;
#pragma unroll
        for (int i = 0; i < MAX_DPL; ++i) acc[i] *= corr;
        for (int jj = 0; jj < nk; ++jj) {
            const int jk = j0 + jj;
            const T* vc = cache + (size_t)bt[jk / page] * page_elems + v_off + (jk % page);
            const float pw = ps[jj];
#pragma unroll
            for (int i = 0; i < MAX_DPL; ++i) {
                const int d = lane + 64 * i;
                if (d < hd) acc[i] = fmaf(pw, to_f32<T>(vc[(size_t)d * page]), acc[i]);
            }
        }
        m = m_new;
    }
#pragma unroll
    for (int i = 0; i < MAX_DPL; ++i) {
        const int d = lane + 64 * i;
        if (d < hd) o[d] = from_f32<T>(acc[i] / l);
    }
}

extern "C" int br_attn_simple(const void* q, size_t q_stride, void* out, int is_bf16, const int* pos,
                              const int* seq_of_token, const int* slots, const int* block_table,
                              int table_stride, const void* cache, int T, int nq, int nkv, int hd,
                              int page, int window, float scale, hipStream_t s) {
    if (T <= 0) return BR_OK;
    if (nq <= 0 || nkv <= 0 || nq % nkv || hd <= 0 || hd > 64 * MAX_DPL || page <= 0 || window < 0 ||
        nq > 65535)
        return BR_BAD_ARG;
    dim3 grid(T, nq);
    size_t lds = (size_t)(hd + 64) * sizeof(float);
    if (is_bf16)
        attn_simple_kernel<bf16><<<grid, 64, lds, s>>>((const bf16*)q, q_stride, (bf16*)out, pos, seq_of_token,
                                                       slots, block_table, table_stride, (const bf16*)cache,
                                                       nq, nkv, hd, page, window, scale);
    else
        attn_simple_kernel<float><<<grid, 64, lds, s>>>((const float*)q, q_stride, (float*)out, pos,
                                                        seq_of_token, slots, block_table, table_stride,
                                                        (const float*)cache, nq, nkv, hd, page, window, scale);
    return br_check_launch();
}
