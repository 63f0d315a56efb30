// Shared device helpers for the gfx950 kernels: storage types, wave64 reductions,
// launch checks.  Everything here is wave64-only (CDNA4 has no wave32 mode).
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>
#include <stdio.h>

typedef __bf16 bf16;
typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef __bf16 bf16x4 __attribute__((ext_vector_type(4)));
typedef __bf16 bf16x2 __attribute__((ext_vector_type(2)));
typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef float f32x16 __attribute__((ext_vector_type(16)));
typedef float f32x2 __attribute__((ext_vector_type(2)));

#define WAVE 64

// Return codes of every extern "C" launcher: 0 = launched, otherwise a code the
// Python side turns into a KernelError with the launcher's name.
#define BR_OK 0
#define BR_BAD_ARG 1
#define BR_LAUNCH_FAILED 2
#define BR_TOO_LARGE 3

static inline int br_check_launch() {
    hipError_t e = hipGetLastError();
    if (e != hipSuccess) {
        fprintf(stderr, "braidinfer_amd: kernel launch failed: %s\n", hipGetErrorString(e));
        return BR_LAUNCH_FAILED;
    }
    return BR_OK;
}

// Compute units of the current device (0 if the runtime does not say), asked once per device.
static inline int br_device_cus() {
    static int cus[64] = {0};
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= 64) return 0;
    if (!cus[dev]) {
        int n = 0;
        if (hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || n <= 0) return 0;
        cus[dev] = n;
    }
    return cus[dev];
}

template <typename T> __device__ __forceinline__ float to_f32(T v);
template <> __device__ __forceinline__ float to_f32<float>(float v) { return v; }
template <> __device__ __forceinline__ float to_f32<bf16>(bf16 v) { return (float)v; }

template <typename T> __device__ __forceinline__ T from_f32(float v);
template <> __device__ __forceinline__ float from_f32<float>(float v) { return v; }
template <> __device__ __forceinline__ bf16 from_f32<bf16>(float v) { return (bf16)v; }  // v_cvt_pk_bf16_f32: RNE

// Butterfly reductions over the 64 lanes of a wave: every lane ends with the same
// value, and the order of the additions is fixed (xor 32,16,...,1), so a result never
// depends on which other rows share the launch.
__device__ __forceinline__ float wave_sum(float v) {
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) v += __shfl_xor(v, o, WAVE);
    return v;
}
__device__ __forceinline__ float wave_max(float v) {
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) v = fmaxf(v, __shfl_xor(v, o, WAVE));
    return v;
}

// Block-wide sum for blocks of up to 16 waves; `scratch` holds 16 floats of LDS.
// Partial sums of the waves are added in wave order by every thread.
__device__ __forceinline__ float block_sum(float v, float* scratch) {
    const int lane = threadIdx.x & 63, w = threadIdx.x >> 6, nw = (blockDim.x + 63) >> 6;
    v = wave_sum(v);
    __syncthreads();
    if (lane == 0) scratch[w] = v;
    __syncthreads();
    float t = 0.f;
    for (int i = 0; i < nw; ++i) t += scratch[i];
    return t;
}
