// f16 instances of the LDS-tiled MFMA GEMM (gemm_tiled.inc): v_mfma_f32_32x32x16_f16, f16 bias / residual / result
// conversions with the C backend's rounding (zyx/src/codegen/c.rs:456-497: mantissa truncation, overflow to inf,
// subnormal results flushed). Shapes, tile choice, split-K and column blocks are the bf16 kernel's.
#define ZK_GEMM_F16 true
#include "gemm_tiled.inc"

namespace zk {

hipError_t gemm_f16_init() { return tiled_init(); }
hipError_t gemm_f16(const GemmBf16 &p, hipStream_t st) { return tiled_gemm(p, st); }

} // namespace zk
