// Helpers shared by the kernels of hybrid decoders (fp32 residual stream, zero-centred or grouped
// norms, attention with a sink or a window, gated outer-product recurrences, expert routing).
// Activations are bfloat16 or float (template parameter), everything a norm, a softmax or a
// recurrence touches is fp32.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

namespace hyb {

constexpr int kWave = 64;

struct bf16_t { uint16_t v; };

template <typename T> __device__ __forceinline__ float ld(const T* p);
template <> __device__ __forceinline__ float ld<float>(const float* p) { return *p; }
template <> __device__ __forceinline__ float ld<bf16_t>(const bf16_t* p) {
    return __uint_as_float(((uint32_t)p->v) << 16);
}
template <typename T> __device__ __forceinline__ void st(T* p, float f);
template <> __device__ __forceinline__ void st<float>(float* p, float f) { *p = f; }
template <> __device__ __forceinline__ void st<bf16_t>(bf16_t* p, float f) {
    __bf16 b = (__bf16)f;                          // round to nearest even
    p->v = __builtin_bit_cast(uint16_t, b);
}

__device__ __forceinline__ float wave_sum(float v) {
#pragma unroll
    for (int o = kWave / 2; o > 0; o >>= 1) v += __shfl_xor(v, o, kWave);
    return v;
}
__device__ __forceinline__ float wave_max(float v) {
#pragma unroll
    for (int o = kWave / 2; o > 0; o >>= 1) v = fmaxf(v, __shfl_xor(v, o, kWave));
    return v;
}

// sum over a workgroup of up to 1024 threads; `red` holds 16 floats of LDS; every thread gets it
__device__ __forceinline__ float block_sum(float v, float* red) {
    v = wave_sum(v);
    const int w = threadIdx.x / kWave, nw = (blockDim.x + kWave - 1) / kWave;
    __syncthreads();
    if ((threadIdx.x & (kWave - 1)) == 0) red[w] = v;
    __syncthreads();
    float s = 0.f;
    for (int i = 0; i < nw; ++i) s += red[i];
    return s;
}
__device__ __forceinline__ float block_max(float v, float* red) {
    v = wave_max(v);
    const int w = threadIdx.x / kWave, nw = (blockDim.x + kWave - 1) / kWave;
    __syncthreads();
    if ((threadIdx.x & (kWave - 1)) == 0) red[w] = v;
    __syncthreads();
    float s = red[0];
    for (int i = 1; i < nw; ++i) s = fmaxf(s, red[i]);
    return s;
}

__device__ __forceinline__ float sigmoidf_(float z) { return 1.f / (1.f + expf(-z)); }
__device__ __forceinline__ float siluf_(float z) { return z / (1.f + expf(-z)); }
__device__ __forceinline__ float softplusf_(float z) { return z > 20.f ? z : log1pf(expf(z)); }
__device__ __forceinline__ float gelu_erf(float z) { return 0.5f * z * (1.f + erff(z * 0.70710678118654752f)); }

// four (Vec4) or N (load_run, N % 4 == 0) consecutive elements widened to fp32; the address must
// be aligned to the run of four (8 bytes for bfloat16, 16 for float)
template <typename T> struct Vec4;
template <> struct Vec4<float> {
    static __device__ __forceinline__ void load(const float* p, float* o) {
        const float4 v = *reinterpret_cast<const float4*>(p);
        o[0] = v.x; o[1] = v.y; o[2] = v.z; o[3] = v.w;
    }
};
template <> struct Vec4<bf16_t> {
    static __device__ __forceinline__ void load(const bf16_t* p, float* o) {
        const uint2 v = *reinterpret_cast<const uint2*>(p);
        o[0] = __uint_as_float(v.x << 16); o[1] = __uint_as_float(v.x & 0xffff0000u);
        o[2] = __uint_as_float(v.y << 16); o[3] = __uint_as_float(v.y & 0xffff0000u);
    }
};
template <typename T, int N> __device__ __forceinline__ void load_run(const T* p, float* o) {
#pragma unroll
    for (int i = 0; i < N; i += 4) Vec4<T>::load(p + i, o + i);
}

// eight consecutive elements narrowed from fp32 and stored as one run (16 bytes of bfloat16, two
// 16-byte stores of float); the address must be aligned to the run
template <typename T> __device__ __forceinline__ void store_run8(T* p, const float* v);
template <> __device__ __forceinline__ void store_run8<float>(float* p, const float* v) {
    *reinterpret_cast<float4*>(p) = make_float4(v[0], v[1], v[2], v[3]);
    *reinterpret_cast<float4*>(p + 4) = make_float4(v[4], v[5], v[6], v[7]);
}
template <> __device__ __forceinline__ void store_run8<bf16_t>(bf16_t* p, const float* v) {
    uint32_t w[4];
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        const __bf16 lo = (__bf16)v[2 * i], hi = (__bf16)v[2 * i + 1];
        w[i] = (uint32_t)__builtin_bit_cast(uint16_t, lo) | ((uint32_t)__builtin_bit_cast(uint16_t, hi) << 16);
    }
    *reinterpret_cast<uint4*>(p) = make_uint4(w[0], w[1], w[2], w[3]);
}

#define HYB_DISPATCH(dt, ...)                                         \
    do {                                                              \
        if ((dt) == 0) { using T = hyb::bf16_t; __VA_ARGS__; }        \
        else if ((dt) == 2) { using T = float; __VA_ARGS__; }         \
        else return 1;                                                \
    } while (0)

#define HYB_LAUNCH_OK() (hipGetLastError() == hipSuccess ? 0 : 2)

}  // namespace hyb
