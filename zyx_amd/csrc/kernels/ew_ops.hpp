// Scalar semantics of the elementwise chain ops (zhip_ew_op in include/zyx_hip.h), shared by the interpreting
// kernel and by the chain kernels generated and compiled at run time (this file's text is the prelude of
// their source, so it includes nothing and names only compiler builtins and HIP device functions).
// Op meaning: zyx/src/kernel/ops.rs:187-261, C meaning zyx/src/codegen/c.rs:290-304,593-611, composites
// zyx/src/tensor/elementwise.rs:168-170,289-293,305-307,457-460,585-588.
#pragma once

namespace zkew {

// storage <-> register conversions (zyx/src/codegen/c.rs:456-497): bf16 widens exactly and truncates on store;
// f16 widens exactly, the store truncates the mantissa, saturates to inf and flushes subnormal results
__device__ __forceinline__ float bf16_bits_to_f32(unsigned int h) { return __uint_as_float(h << 16); }
__device__ __forceinline__ unsigned int f32_to_bf16_bits(float v) { return __float_as_uint(v) >> 16; }
__device__ __forceinline__ float f16_bits_to_f32(unsigned int h) {
    const unsigned short s = (unsigned short)h;
    return (float)__builtin_bit_cast(_Float16, s);
}
__device__ __forceinline__ unsigned int f32_to_f16_bits(float v) {
    const unsigned int f = __float_as_uint(v);
    const unsigned int sign = (f >> 16) & 0x8000u, ex = (f >> 23) & 0xffu, man = f & 0x7fffffu;
    if (ex == 0) return sign;
    if (ex == 255) return sign | 0x7c00u | (man >> 13);
    const int ne = (int)ex - 127 + 15;
    if (ne >= 31) return sign | 0x7c00u;
    if (ne <= 0) return sign;
    return sign | ((unsigned int)ne << 10) | (man >> 13);
}

// tanh as the reference writes it, (e^{2z}-1)/(e^{2z}+1) (elementwise.rs:585-588), made
// saturating where e^{2z} overflows and the reference's own value is inf/inf.
__device__ __forceinline__ float ref_tanh(float z) {
    float e = expf(z + z);
    float r = (e - 1.0f) / (e + 1.0f);
    return (z + z) > 88.0f ? 1.0f : r;
}
__device__ __forceinline__ float ref_gelu(float x) {
    float inner = (x + ((x * x) * x) * 0.044715f) * 0.79788456080286535588f;
    return (x * 0.5f) * (ref_tanh(inner) + 1.0f);
}

__device__ __forceinline__ float ref_gelu_grad(float x) {
    const float k = 0.79788456080286535588f, x2 = x * x;
    const float t = ref_tanh((x + x2 * x * 0.044715f) * k);
    return 0.5f * (1.0f + t) + (0.5f * x) * ((1.0f - t * t) * (k * (1.0f + 0.134145f * x2)));
}

// The sigmoid family on v_exp_f32 / v_rcp_f32 (about 1 ulp of f32 each), for results that are stored in 16 bits:
// 0.5 (1 + tanh(u)) = sigmoid(2u) = 1 / (1 + 2^(-2u log2 e)), so gelu(x) = x * sigmoid(2u) and
// gelu'(x) = s + x * 2 s (1 - s) * k (1 + 3 * 0.044715 x^2) with s = sigmoid(2u). All of them saturate where e^{2u}
// overflows, like ref_tanh.
__device__ __forceinline__ float quick_sigmoid(float z) { // 1 / (1 + e^-z)
    return __builtin_amdgcn_rcpf(1.0f + __builtin_amdgcn_exp2f(z * -1.44269504088896340736f));
}
__device__ __forceinline__ float op_f_quick(int op, float x, float a, float b) {
    (void)a;
    (void)b;
    const float k = 0.79788456080286535588f;
    switch (op) {
    case 39: return 1.0f - 2.0f * __builtin_amdgcn_rcpf(__builtin_amdgcn_exp2f(x * 2.88539008177792681472f) + 1.0f);
    case 40: return x * quick_sigmoid((x + ((x * x) * x) * 0.044715f) * (2.0f * k));
    case 41: return quick_sigmoid(x);
    default: { // 44
        const float x2 = x * x, s = quick_sigmoid((x + (x2 * x) * 0.044715f) * (2.0f * k));
        return s + (x * s) * ((2.0f - 2.0f * s) * (k * (1.0f + 0.134145f * x2)));
    }
    }
}

__device__ __forceinline__ float op_f(int op, float x, float a, float b) {
    switch (op) {
    case 0: return a;                                  // LOAD
    case 2: return -x;                                 // NEG
    case 4: return expf(x);
    case 5: return exp2f(x);
    case 6: return logf(x);
    case 7: return log2f(x);
    case 8: return 1.0f / x;
    case 9: return sqrtf(x);
    case 10: return sinf(x);
    case 11: return cosf(x);
    case 12: return floorf(x);
    case 13: return truncf(x);
    case 14: return fabsf(x);
    case 15: return x + a;
    case 16: return x - a;
    case 17: return x * a;
    case 18: return x / a;
    case 19: return exp2f(log2f(x) * a);               // Pow is unfolded to exp2(log2(x)*y)
    case 20: return (float)((int)x % ((int)a == 0 ? 1 : (int)a)); // (int)x % (int)y
    case 21: return x < a ? 1.0f : 0.0f;
    case 22: return x > a ? 1.0f : 0.0f;
    case 23: return x >= a ? 1.0f : 0.0f;
    case 24: return fmaxf(x, a);
    case 25: return (x != 0.0f || a != 0.0f) ? 1.0f : 0.0f;
    case 26: return (x != 0.0f && a != 0.0f) ? 1.0f : 0.0f;
    case 32: return x != a ? 1.0f : 0.0f;
    case 33: return x == a ? 1.0f : 0.0f;
    case 34: return a - x;                             // RSUB
    case 35: return a / x;                             // RDIV
    case 36: return x != 0.0f ? a : b;                 // WHERE
    case 37: return x * a + b;                         // MAD
    case 38: return (x > 0.0f ? 1.0f : 0.0f) * x;      // RELU = (x > 0) * x
    case 39: return ref_tanh(x);
    case 40: return ref_gelu(x);
    case 41: { float e = expf(x); return e / (e + 1.0f); }
    case 42: return sqrtf(1.0f / x);                   // rsqrt = reciprocal().sqrt()
    case 43: return truncf(x);                         // CAST_INT inside a float chain
    case 44: return ref_gelu_grad(x);
    default: return x;
    }
}
__device__ __forceinline__ int op_i(int op, int x, int a, int b) {
    switch (op) {
    case 0: return a;
    case 2: return (int)(0u - (unsigned int)x);
    case 3: return ~x;
    case 14: return x < 0 ? (int)(0u - (unsigned int)x) : x;
    case 15: return (int)((unsigned int)x + (unsigned int)a);
    case 16: return (int)((unsigned int)x - (unsigned int)a);
    case 17: return (int)((unsigned int)x * (unsigned int)a);
    case 18: return a == 0 ? 0 : (a == -1 ? (int)(0u - (unsigned int)x) : x / a);
    case 20: return (a == 0 || a == -1) ? 0 : x % a;
    case 21: return x < a;
    case 22: return x > a;
    case 23: return x >= a;
    case 24: return x > a ? x : a;
    case 25: return (x != 0) || (a != 0);
    case 26: return (x != 0) && (a != 0);
    case 27: return x ^ a;
    case 28: return x | a;
    case 29: return x & a;
    case 30: return (int)((unsigned int)x << (a & 31));
    case 31: return x >> (a & 31);
    case 32: return x != a;
    case 33: return x == a;
    case 34: return (int)((unsigned int)a - (unsigned int)x);
    case 35: return x == 0 ? 0 : (x == -1 ? (int)(0u - (unsigned int)a) : a / x);
    case 36: return x != 0 ? a : b;
    case 37: return (int)((unsigned int)x * (unsigned int)a + (unsigned int)b);
    case 38: return x > 0 ? x : 0;
    default: return x;
    }
}

} // namespace zkew
