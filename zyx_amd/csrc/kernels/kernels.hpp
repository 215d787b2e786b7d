// Launchers of the hand-written gfx950 kernels. Each takes device pointers that the
// runtime has already bounds-checked against the registered shape, enqueues on the
// given stream and returns the HIP status of the launch.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

namespace zk {

struct SoftmaxRows {
    int64_t rows, cols;
    const float *x;
    float *y;       // may be null
    float *rowsum;  // may be null
    int32_t *arg;   // may be null
};
hipError_t softmax_rows(const SoftmaxRows &p, hipStream_t stream);

} // namespace zk
