// Storage <-> register conversions with the rounding rules of zyx's C backend
// (zyx/src/codegen/c.rs:456-497): bf16 and f16 widen exactly on load; on store bf16
// keeps the top 16 bits (truncation) and f16 truncates the mantissa, saturates to inf
// and flushes results below the normal range to signed zero.
#pragma once
#include <hip/hip_runtime.h>
#include <hip/hip_fp16.h>
#include <stdint.h>

namespace zk {

// dtype codes of include/zyx_hip.h (zyx/src/dtype.rs:20-47)
enum : int { DT_BF16 = 0, DT_F16 = 1, DT_F32 = 2, DT_F64 = 3, DT_U8 = 4, DT_U16 = 5, DT_U32 = 6, DT_U64 = 7,
             DT_I8 = 8, DT_I16 = 9, DT_I32 = 10, DT_I64 = 11, DT_BOOL = 12 };

__device__ __forceinline__ float bf16_to_f32(uint16_t h) { return __uint_as_float((uint32_t)h << 16); }
__device__ __forceinline__ uint16_t f32_to_bf16_trunc(float v) { return (uint16_t)(__float_as_uint(v) >> 16); }
__device__ __forceinline__ float f16_to_f32(uint16_t h) {
    return __half2float(__ushort_as_half(h)); // exact, subnormals included
}
__device__ __forceinline__ uint16_t f32_to_f16_trunc(float v) {
    uint32_t f = __float_as_uint(v);
    uint32_t sign = (f >> 16) & 0x8000u, ex = (f >> 23) & 0xffu, man = f & 0x7fffffu;
    if (ex == 0) return (uint16_t)sign;
    if (ex == 255) return (uint16_t)(sign | 0x7c00u | (man >> 13));
    int ne = (int)ex - 127 + 15;
    if (ne >= 31) return (uint16_t)(sign | 0x7c00u);
    if (ne <= 0) return (uint16_t)sign;
    return (uint16_t)(sign | ((uint32_t)ne << 10) | (man >> 13));
}

__host__ __device__ inline int dtype_size(int dt) {
    switch (dt) {
    case DT_BF16: case DT_F16: case DT_U16: case DT_I16: return 2;
    case DT_F32: case DT_U32: case DT_I32: return 4;
    case DT_F64: case DT_U64: case DT_I64: return 8;
    default: return 1;
    }
}

} // namespace zk
