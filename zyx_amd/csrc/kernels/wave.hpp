// Wave-64 building blocks shared by the memory-bound kernels (gfx950 only).
#pragma once
#include <hip/hip_runtime.h>
#include <float.h>
#include <stdint.h>

namespace zk {

constexpr int kWave = 64;

typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef int i32x4 __attribute__((ext_vector_type(4)));

// Streaming (read-once / write-once) 128-bit accesses: marked non-temporal so the
// lines do not displace data that is reused.
__device__ __forceinline__ f32x4 load_stream(const f32x4 *p) { return __builtin_nontemporal_load(p); }
__device__ __forceinline__ void store_stream(f32x4 v, f32x4 *p) { __builtin_nontemporal_store(v, p); }

// DPP controls (CDNA ISA: quad_perm 0x00-0xff, row_mirror 0x140, row_half_mirror 0x141)
constexpr int kDppQuadXor1 = 0xB1;       // quad_perm [1,0,3,2]
constexpr int kDppQuadXor2 = 0x4E;       // quad_perm [2,3,0,1]
constexpr int kDppRowHalfMirror = 0x141; // lane i <-> 7-i inside each 8
constexpr int kDppRowMirror = 0x140;     // lane i <-> 15-i inside each 16

template <int CTRL> __device__ __forceinline__ float dpp_f32(float v) {
    return __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), CTRL, 0xf, 0xf, true));
}
template <int CTRL> __device__ __forceinline__ int dpp_i32(int v) {
    return __builtin_amdgcn_update_dpp(0, v, CTRL, 0xf, 0xf, true);
}
__device__ __forceinline__ float readlane_f32(float v, int lane) {
    return __int_as_float(__builtin_amdgcn_readlane(__float_as_int(v), lane));
}

struct OpAdd { template <class T> __device__ __forceinline__ T operator()(T a, T b) const { return a + b; } };
struct OpMaxF { __device__ __forceinline__ float operator()(float a, float b) const { return fmaxf(a, b); } };
struct OpMaxI { __device__ __forceinline__ int operator()(int a, int b) const { return a > b ? a : b; } };

// All-reduce over the 64 lanes of a wave. Four DPP steps leave every 16-lane row
// uniform (each step pairs lanes that already agree inside the smaller group), then
// the four row values are fetched with v_readlane and folded, so no LDS is touched.
template <class Op> __device__ __forceinline__ float wave_allreduce_f32(float v, Op op) {
    v = op(v, dpp_f32<kDppQuadXor1>(v));
    v = op(v, dpp_f32<kDppQuadXor2>(v));
    v = op(v, dpp_f32<kDppRowHalfMirror>(v));
    v = op(v, dpp_f32<kDppRowMirror>(v));
    float a = readlane_f32(v, 0), b = readlane_f32(v, 16), c = readlane_f32(v, 32), d = readlane_f32(v, 48);
    return op(op(a, b), op(c, d));
}
template <class Op> __device__ __forceinline__ int wave_allreduce_i32(int v, Op op) {
    v = op(v, dpp_i32<kDppQuadXor1>(v));
    v = op(v, dpp_i32<kDppQuadXor2>(v));
    v = op(v, dpp_i32<kDppRowHalfMirror>(v));
    v = op(v, dpp_i32<kDppRowMirror>(v));
    int a = __builtin_amdgcn_readlane(v, 0), b = __builtin_amdgcn_readlane(v, 16);
    int c = __builtin_amdgcn_readlane(v, 32), d = __builtin_amdgcn_readlane(v, 48);
    return op(op(a, b), op(c, d));
}

// exp(d) for d <= 0 through the hardware exp2 (v_exp_f32). The product d*log2(e) is
// split so its rounding error does not grow with |d|: hi = fl(d*L), lo = the exact
// remainder of that product plus d times the tail of L; exp2(hi) is then corrected
// by (1 + lo*ln2). Relative error stays ~2 ulp for the whole range. Where exp2 underflows to 0 the
// result must be 0 whatever the correction term holds: for d = -inf (a masked score) and for products that
// overflow, `lo` is inf - inf or inf. The correction is therefore formed with v_mul_legacy_f32, whose
// product is 0 whenever a factor is 0 (0 * NaN = 0 * inf = 0); a NaN d still gives NaN (r is NaN).
__device__ __forceinline__ float exp_neg(float d) {
    const float L_hi = 1.44269502162933349609375f; // fl(log2 e)
    const float L_lo = 1.925963033500011e-08f;     // log2 e - L_hi
    float hi = d * L_hi;
    float lo = __builtin_fmaf(d, L_hi, -hi) + d * L_lo;
    float r = __builtin_amdgcn_exp2f(hi);
    float corr;
    asm("v_mul_legacy_f32 %0, %1, %2" : "=v"(corr) : "v"(r), "v"(lo * 0.693147182464599609375f));
    return r + corr;
}

} // namespace zk
