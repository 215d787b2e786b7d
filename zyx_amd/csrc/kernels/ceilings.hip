// Measured ceilings of the device this context runs on: what a streaming kernel and a register-only stream of
// matrix instructions reach here, today, on this clock and power state. The reference describes a device to its
// optimiser by nominal figures (DeviceInfo.compute, zyx/src/backend/mod.rs:506-531) and finds everything else by
// launch-and-time (zyx/src/kernel/autotune.rs:775-798); these probes are the same idea applied to the two
// rooflines the hand-written kernels are priced against.
#include "kernels.hpp"
#include "wave.hpp"

namespace zk {

namespace {

typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef float f32x16 __attribute__((ext_vector_type(16)));

// dst[i] = src[i]: every wave moves one contiguous 4 KiB piece, its 4 loads of 16 bytes per lane all in flight before
// the first store (the access pattern of the row kernels: four waves per 16 KiB row), streaming accesses. n16 is a
// multiple of 4096. (With 16 KiB per wave the same copy reaches 5.8-5.9 TB/s instead of 6.1-6.2.)
__global__ __launch_bounds__(256) void probe_copy_k(const f32x4 *__restrict__ src, f32x4 *__restrict__ dst, int64_t n16) {
    const int64_t base = ((int64_t)blockIdx.x * 4 + (threadIdx.x >> 6)) * 256 + (threadIdx.x & 63);
    if (base >= n16) return;
    f32x4 v[4];
#pragma unroll
    for (int k = 0; k < 4; k++) v[k] = load_stream(src + base + k * 64);
#pragma unroll
    for (int k = 0; k < 4; k++) store_stream(v[k], dst + base + k * 64);
}
// out[wave] = sum of the wave's 2 KiB: the read-only ceiling. Every wave reads 2 KiB of consecutive bytes once and ends
// (the pattern that measured fastest: 7.0 TB/s against 6.7 for 4-16 KiB per wave and 5.6-6.1 for a grid-stride loop).
__global__ __launch_bounds__(256) void probe_read_k(const f32x4 *__restrict__ src, float *__restrict__ out, int64_t n16) {
    const int lane = threadIdx.x & 63;
    const int64_t wave = (int64_t)blockIdx.x * 4 + (threadIdx.x >> 6), base = wave * 128;
    f32x4 s0 = {0, 0, 0, 0}, s1 = s0;
    if (base + lane < n16) s0 = load_stream(src + base + lane);
    if (base + 64 + lane < n16) s1 = load_stream(src + base + 64 + lane);
    s0 += s1;
    float v = wave_allreduce_f32(s0[0] + s0[1] + s0[2] + s0[3], OpAdd());
    if (lane == 0) out[wave] = v;
}

// One wave per SIMD issues 16 * iters v_mfma_f32_32x32x16_bf16 back to back on 16 independent accumulator tiles,
// operands in registers only. RANDOM: four operand pairs of uniform(-1, 1) values take turns (the switching activity
// of real data); else one pair of small constants. clk[0..1]: shader-clock and 100 MHz wall-clock ticks of wave 0.
template <int RANDOM>
__global__ __launch_bounds__(256, 1) void probe_mfma_k(float *__restrict__ out, int iters, long long *__restrict__ clk) {
    f32x16 acc[16];
#pragma unroll
    for (int i = 0; i < 16; i++)
#pragma unroll
        for (int r = 0; r < 16; r++) acc[i][r] = 0.0f;
    bf16x8 a[4], b[4];
    unsigned seed = threadIdx.x * 2654435761u + blockIdx.x * 40503u + 12345u;
#pragma unroll
    for (int q = 0; q < 4; q++)
#pragma unroll
        for (int k = 0; k < 8; k++) {
            seed = seed * 1664525u + 1013904223u;
            a[q][k] = RANDOM ? (__bf16)(((int)(seed >> 8) % 2001 - 1000) / 1000.0f) : (__bf16)(0.5f);
            seed = seed * 1664525u + 1013904223u;
            b[q][k] = RANDOM ? (__bf16)(((int)(seed >> 8) % 2001 - 1000) / 1000.0f) : (__bf16)(0.25f);
        }
    const long long c0 = clock64(), w0 = wall_clock64();
    for (int it = 0; it < iters; it++) {
#pragma unroll
        for (int i = 0; i < 16; i++) acc[i] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a[i & 3], b[(i >> 2) & 3], acc[i], 0, 0, 0);
    }
    const long long c1 = clock64(), w1 = wall_clock64();
    float s = 0.0f;
#pragma unroll
    for (int i = 0; i < 16; i++)
#pragma unroll
        for (int r = 0; r < 16; r++) s += acc[i][r];
    out[blockIdx.x * 256 + threadIdx.x] = s;
    if (blockIdx.x == 0 && threadIdx.x == 0) {
        clk[0] = c1 - c0;
        clk[1] = w1 - w0;
    }
}

} // namespace

hipError_t measure_ceilings(uint64_t bytes, int compute_units, Ceilings *out, hipStream_t st) {
    *out = Ceilings{};
    bytes = bytes / 65536 * 65536; // whole 16 KiB pieces for every wave of a copy workgroup
    if (bytes < (1u << 20) || compute_units <= 0) return hipErrorInvalidValue;
    char *a = nullptr, *b = nullptr;
    long long *clk = nullptr;
    hipEvent_t e0 = nullptr, e1 = nullptr;
    hipError_t e = hipMalloc(&a, bytes);
    if (e == hipSuccess) e = hipMalloc(&b, bytes);
    if (e == hipSuccess) e = hipMalloc(&clk, 16);
    if (e == hipSuccess) e = hipEventCreate(&e0);
    if (e == hipSuccess) e = hipEventCreate(&e1);
    if (e == hipSuccess) e = hipMemsetAsync(a, 1, bytes, st);
    if (e == hipSuccess) e = hipMemsetAsync(b, 2, bytes, st);
    auto timed = [&](auto &&body, int reps, float *us) {
        if (e != hipSuccess) return;
        (void)body(); // warm
        e = hipEventRecord(e0, st);
        for (int i = 0; i < reps && e == hipSuccess; i++) e = body();
        if (e == hipSuccess) e = hipEventRecord(e1, st);
        if (e == hipSuccess) e = hipEventSynchronize(e1);
        float ms = 0.0f;
        if (e == hipSuccess) e = hipEventElapsedTime(&ms, e0, e1);
        *us = ms * 1000.0f / (float)reps;
    };
    const int64_t n16 = (int64_t)(bytes / 16);
    float us = 0.0f;
    // buffers alternate direction so a launch never finds its source in the cache the launch before left behind
    int flip = 0;
    timed([&] { flip ^= 1; return hipMemcpyAsync(flip ? b : a, flip ? a : b, bytes, hipMemcpyDeviceToDevice, st); }, 10, &us);
    if (e == hipSuccess) out->memcpy_d2d_GBps = 2.0f * (float)bytes / us / 1e3f;
    timed([&] {
        flip ^= 1;
        hipLaunchKernelGGL(probe_copy_k, dim3((unsigned)(n16 / 1024)), dim3(256), 0, st, (const f32x4 *)(flip ? a : b), (f32x4 *)(flip ? b : a), n16);
        return hipGetLastError();
    }, 10, &us);
    if (e == hipSuccess) out->copy_kernel_GBps = 2.0f * (float)bytes / us / 1e3f;
    timed([&] {
        flip ^= 1;
        // a partial sum per 2 KiB read lands at the start of the other buffer (1/512 of the bytes read)
        hipLaunchKernelGGL(probe_read_k, dim3((unsigned)((n16 + 511) / 512)), dim3(256), 0, st, (const f32x4 *)(flip ? a : b), (float *)(flip ? b : a), n16);
        return hipGetLastError();
    }, 10, &us);
    if (e == hipSuccess) out->read_kernel_GBps = (float)bytes / us / 1e3f;
    // one 256-thread workgroup per CU, 4096 matrix instructions per wave and launch (the count of a 4096^3 product's tile)
    const int iters = 256;
    const double flop = (double)compute_units * 4.0 * iters * 16.0 * 2.0 * 32 * 32 * 16;
    for (int random = 0; random < 2; random++) {
        long long h[2] = {0, 1};
        // settle the clock on this kind of work first
        timed([&] {
            if (random) hipLaunchKernelGGL(probe_mfma_k<1>, dim3(compute_units), dim3(256), 0, st, (float *)a, iters, clk);
            else hipLaunchKernelGGL(probe_mfma_k<0>, dim3(compute_units), dim3(256), 0, st, (float *)a, iters, clk);
            return hipGetLastError();
        }, 200, &us);
        timed([&] {
            if (random) hipLaunchKernelGGL(probe_mfma_k<1>, dim3(compute_units), dim3(256), 0, st, (float *)a, iters, clk);
            else hipLaunchKernelGGL(probe_mfma_k<0>, dim3(compute_units), dim3(256), 0, st, (float *)a, iters, clk);
            return hipGetLastError();
        }, 100, &us);
        if (e == hipSuccess) e = hipMemcpy(h, clk, 16, hipMemcpyDeviceToHost);
        if (e != hipSuccess) break;
        const float mhz = h[1] > 0 ? (float)((double)h[0] / (double)h[1] * 100.0) : 0.0f;
        // in-kernel duration of one wave's 4096 instructions (100 MHz ticks): launch gaps excluded
        const float tf = h[1] > 0 ? (float)(flop / ((double)h[1] / 100.0) / 1e6) : 0.0f;
        if (random) { out->mfma_bf16_random_TFLOPs = tf; out->mfma_bf16_random_MHz = mhz; out->mfma_bf16_random_launch_us = us; }
        else { out->mfma_bf16_const_TFLOPs = tf; out->mfma_bf16_const_MHz = mhz; out->mfma_bf16_const_launch_us = us; }
    }
    (void)hipStreamSynchronize(st);
    if (e0) (void)hipEventDestroy(e0);
    if (e1) (void)hipEventDestroy(e1);
    if (a) (void)hipFree(a);
    if (b) (void)hipFree(b);
    if (clk) (void)hipFree(clk);
    return e;
}

} // namespace zk
