// Generic kernels: a linearized zyx kernel (image layout: include/zyx_hip.h, "linearized kernel IR") is turned
// into HIP source, compiled for gfx950 with hiprtc and launched on the grid its Index ops name.
#pragma once

#include <hip/hip_runtime.h>

#include <cstdint>
#include <string>
#include <vector>

namespace zk {

struct IrParam {
    int kind;       // zhip_ir_param_kind
    int dtype;      // zhip_dtype
    uint64_t elems; // elements the kernel may touch, 0 = unknown
};

struct IrDim { // one grid axis: a constant, or the value of the Variable parameter `ordinal` at launch
    bool from_param = false;
    uint64_t value = 1;
    int ordinal = -1;
};

struct IrProgram {
    hipModule_t mod = nullptr;
    hipFunction_t fn = nullptr;
    std::vector<IrParam> params;
    IrDim grid[3];
    unsigned block[3] = {1, 1, 1};
    std::string source;
};

// Parses and checks the image and writes the kernel's source; no device is touched. False with the reason in err.
bool ir_generate(const void *image, uint64_t bytes, IrProgram &out, std::string &err);
// ir_generate + hiprtc + module load on the current device. Null with the reason in err.
IrProgram *ir_compile(const void *image, uint64_t bytes, std::string &err);
// slots[i]: for a buffer parameter the address of a variable holding the device pointer, for a Variable
// parameter the address of its value's bytes. Grid axes that come from a parameter are read from those bytes.
hipError_t ir_launch(const IrProgram *p, void *const *slots, hipStream_t stream, std::string *why);
void ir_destroy(IrProgram *p);

} // namespace zk
