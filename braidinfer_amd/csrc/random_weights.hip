// Seeded random weights made on the device: a counter-based generator, so that a value
// depends on (key of the tensor, element index) only and is the same bits wherever it is
// computed (this kernel, the NumPy form in weights/random_weights.py).  The reference has
// no random weights; its bf16 rounding is round-to-nearest-even (quant.rs:203-207), which
// is what the conversion below does.
//
//   mix(z):  z ^= z >> 30; z *= 0xBF58476D1CE4E5B9; z ^= z >> 27; z *= 0x94D049BB133111EB; z ^= z >> 31
//   word(key, c) = mix(key + (c + 1) * 0x9E3779B97F4A7C15)                     (splitmix64 at counter c)
//   normal element i:  s = sum of the twelve 16-bit fields of word(key, 3i), word(key, 3i+1),
//                      word(key, 3i+2);  value = float(s - 393210) * scale,  scale = float(std) * 2^-16
//   (a sum of twelve uniform 16-bit integers has mean 393210 and variance 2^32 - 1: integer
//   arithmetic and one float multiplication, so no library function's rounding enters)
//   jittered one, element i:  u = float(word(key, i) >> 40) * 2^-24;  value = 1 + (2u - 1) * jitter,
//                      the product and the sum rounded separately
#include "common.h"

// every product and sum below is rounded on its own: no fused multiply-add may be formed
// (plain operators under this pragma; the __f*_rn functions of the headers are inlined with
// contraction allowed and do not prevent it)
#pragma clang fp contract(off)

#define RW_GOLDEN 0x9E3779B97F4A7C15ull

__device__ __forceinline__ uint64_t rw_mix(uint64_t z) {
    z ^= z >> 30; z *= 0xBF58476D1CE4E5B9ull;
    z ^= z >> 27; z *= 0x94D049BB133111EBull;
    return z ^ (z >> 31);
}
__device__ __forceinline__ uint64_t rw_word(uint64_t key, uint64_t c) { return rw_mix(key + (c + 1) * RW_GOLDEN); }
__device__ __forceinline__ int rw_fields(uint64_t w) {
    return (int)(w & 0xFFFF) + (int)((w >> 16) & 0xFFFF) + (int)((w >> 32) & 0xFFFF) + (int)(w >> 48);
}

template <typename T>
__global__ void random_normal_kernel(T* __restrict__ out, size_t n, size_t first, uint64_t key, float scale) {
    const size_t stride = (size_t)gridDim.x * blockDim.x;
    for (size_t j = (size_t)blockIdx.x * blockDim.x + threadIdx.x; j < n; j += stride) {
        const uint64_t i = (uint64_t)(first + j);
        const int s = rw_fields(rw_word(key, 3 * i)) + rw_fields(rw_word(key, 3 * i + 1)) + rw_fields(rw_word(key, 3 * i + 2));
        out[j] = from_f32<T>((float)(s - 393210) * scale);
    }
}

template <typename T>
__global__ void random_ones_kernel(T* __restrict__ out, size_t n, size_t first, uint64_t key, float jitter) {
    const size_t stride = (size_t)gridDim.x * blockDim.x;
    for (size_t j = (size_t)blockIdx.x * blockDim.x + threadIdx.x; j < n; j += stride) {
        const float u = (float)(rw_word(key, (uint64_t)(first + j)) >> 40) * 5.9604644775390625e-08f;   // 2^-24, exact
        const float d = ((u + u) - 1.0f) * jitter;
        out[j] = from_f32<T>(1.0f + d);
    }
}

// out[0..n) = elements first .. first + n - 1 of the tensor with this key.
extern "C" int br_random_normal(void* out, int is_bf16, size_t n, size_t first, uint64_t key, float scale, hipStream_t s) {
    if (n == 0) return BR_OK;
    if (!out) return BR_BAD_ARG;
    size_t want = (n + 255) / 256;
    unsigned blocks = (unsigned)(want < 16384 ? want : 16384);
    if (is_bf16) random_normal_kernel<bf16><<<blocks, 256, 0, s>>>((bf16*)out, n, first, key, scale);
    else random_normal_kernel<float><<<blocks, 256, 0, s>>>((float*)out, n, first, key, scale);
    return br_check_launch();
}

extern "C" int br_random_ones(void* out, int is_bf16, size_t n, size_t first, uint64_t key, float jitter, hipStream_t s) {
    if (n == 0) return BR_OK;
    if (!out) return BR_BAD_ARG;
    size_t want = (n + 255) / 256;
    unsigned blocks = (unsigned)(want < 16384 ? want : 16384);
    if (is_bf16) random_ones_kernel<bf16><<<blocks, 256, 0, s>>>((bf16*)out, n, first, key, jitter);
    else random_ones_kernel<float><<<blocks, 256, 0, s>>>((float*)out, n, first, key, jitter);
    return br_check_launch();
}
