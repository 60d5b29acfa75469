// Row-wise I/O helpers shared by the HBM-bound kernels (norms, cross entropy): 8 consecutive
// elements per lane as one 16-byte (bf16) or two 16-byte (fp32) accesses, converted to and from fp32.
#pragma once
#include <hip/hip_runtime.h>

#include <cstdint>

namespace ma {

typedef __bf16 bf16x8_v __attribute__((ext_vector_type(8)));

template <typename T>
__device__ __forceinline__ void ld8(const T* p, float* v);
template <>
__device__ __forceinline__ void ld8<float>(const float* p, float* v) {
    const float4 a = *(const float4*)p, b = *(const float4*)(p + 4);
    v[0] = a.x; v[1] = a.y; v[2] = a.z; v[3] = a.w; v[4] = b.x; v[5] = b.y; v[6] = b.z; v[7] = b.w;
}
template <>
__device__ __forceinline__ void ld8<uint16_t>(const uint16_t* p, float* v) {
    const uint4 a = *(const uint4*)p;
    const uint32_t w[4] = {a.x, a.y, a.z, a.w};
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        v[2 * i] = __uint_as_float(w[i] << 16);
        v[2 * i + 1] = __uint_as_float(w[i] & 0xffff0000u);
    }
}
template <typename T>
__device__ __forceinline__ void st8(T* p, const float* v);
template <>
__device__ __forceinline__ void st8<float>(float* p, const float* v) {
    *(float4*)p = make_float4(v[0], v[1], v[2], v[3]);
    *(float4*)(p + 4) = make_float4(v[4], v[5], v[6], v[7]);
}
template <>
__device__ __forceinline__ void st8<uint16_t>(uint16_t* p, const float* v) {
    bf16x8_v o;
#pragma unroll
    for (int i = 0; i < 8; ++i) o[i] = (__bf16)v[i];  // round to nearest even, like torch's cast
    *(bf16x8_v*)p = o;
}
// what a value becomes when it is stored in T and read back
template <typename T>
__device__ __forceinline__ float through(float v);
template <>
__device__ __forceinline__ float through<float>(float v) { return v; }
template <>
__device__ __forceinline__ float through<uint16_t>(float v) { return (float)(__bf16)v; }

__device__ __forceinline__ float wave_sum(float x) {
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) x += __shfl_xor(x, off, 64);
    return x;
}

}  // namespace ma
