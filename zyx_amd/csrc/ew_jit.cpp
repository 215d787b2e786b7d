// Run-time specialisation of elementwise chains: the accumulator program of a ZHIP_K_ELEMENTWISE kernel is
// turned into straight-line HIP source (ops, dtypes, broadcasts, constants and the shape are literals), compiled
// for gfx950 with hiprtc and loaded as a module. This is what zyx does for every fused kernel: generate source
// per kernel and hand it to the vendor's run-time compiler (zyx/src/codegen/c.rs:16-527 for the C backend; the
// HIP slot was to load hiprtc for it, zyx/src/backend/hip.rs:122-188, 604-651). The op semantics are the text of
// kernels/ew_ops.hpp, the same functions the interpreting kernel calls, so both paths compute the same bits.
//
// Generated kernel: V elements per vector (8 when the result is 16-bit and every full-tensor operand is, else
// 4), U vectors per thread and trip; the loads of all U vectors are the first statements of a trip, so a thread
// keeps U x (full-tensor operands) 128-bit loads in flight; streaming accesses are non-temporal.
#include "kernels/kernels.hpp"

#include "rtc_cache.hpp"

#include <cstdarg>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <string>
#include <vector>

namespace zk {

namespace {

const char kPrelude[] =
#include "ew_ops_src.inc"
    ;

enum : int { DT_BF16 = 0, DT_F16 = 1, DT_F32 = 2, DT_U8 = 4, DT_I32 = 10, DT_BOOL = 12 };
int esize(int dt) { return dt == DT_F32 || dt == DT_I32 ? 4 : (dt == DT_BF16 || dt == DT_F16 ? 2 : 1); }

struct Gen {
    std::string s;
    void f(const char *fmt, ...) __attribute__((format(printf, 2, 3))) {
        char buf[1024];
        va_list ap;
        va_start(ap, fmt);
        vsnprintf(buf, sizeof buf, fmt, ap);
        va_end(ap);
        s += buf;
    }
};

// element k of a vector loaded as 32-bit words w{0..}: expression of register type R
std::string elem_expr(const std::string &w, int dt, int k, bool ireg) {
    char b[256];
    const char *R = ireg ? "int" : "float";
    switch (dt) {
    case DT_F32: snprintf(b, sizeof b, "(%s)__uint_as_float(%s%d)", R, w.c_str(), k); break;
    case DT_I32: snprintf(b, sizeof b, "(%s)(int)%s%d", R, w.c_str(), k); break;
    case DT_BF16:
        if (k & 1) snprintf(b, sizeof b, "(%s)__uint_as_float(%s%d & 0xffff0000u)", R, w.c_str(), k / 2);
        else snprintf(b, sizeof b, "(%s)__uint_as_float(%s%d << 16)", R, w.c_str(), k / 2);
        break;
    case DT_F16: snprintf(b, sizeof b, "(%s)zkew::f16_bits_to_f32((%s%d >> %d) & 0xffffu)", R, w.c_str(), k / 2, 16 * (k & 1)); break;
    default: snprintf(b, sizeof b, "(%s)((%s%d >> %d) & 0xffu)", R, w.c_str(), k / 4, 8 * (k & 3)); break;
    }
    return b;
}

// statements loading `bytes` (4, 8, 16 or 32) from `ptr + off` into words name0..: non-temporal when streaming
void emit_load(Gen &g, const std::string &name, const std::string &ptr, const std::string &off, int bytes, bool stream) {
    const char *ld = stream ? "__builtin_nontemporal_load" : "*";
    if (bytes == 4) {
        g.f("        const unsigned int %s0 = %s((const unsigned int *)(%s + %s));\n", name.c_str(), stream ? ld : "*", ptr.c_str(), off.c_str());
        return;
    }
    const int nvec = bytes == 32 ? 2 : 1, per = bytes == 8 ? 2 : 4;
    for (int q = 0; q < nvec; q++) {
        g.f("        const u32x%d %sv%d = %s((const u32x%d *)(%s + %s + %d));\n", per, name.c_str(), q, ld, per, ptr.c_str(), off.c_str(), q * 16);
        for (int k = 0; k < per; k++) g.f("        const unsigned int %s%d = %sv%d[%d];\n", name.c_str(), q * 4 + k, name.c_str(), q, k);
    }
}

} // namespace

struct EwJit {
    hipModule_t mod = nullptr;
    hipFunction_t fn = nullptr;
    int V = 4, U = 2;
    int64_t nvec = 0;
};

bool ew_jit_eligible(const Elementwise &p, int *Vout) {
    const int64_t n = p.rows * p.cols;
    if (n <= 0 || n % 4) return false;
    bool v8 = n % 8 == 0 && esize(p.out_dtype) == 2;
    for (int k = 0; k < p.n_in; k++) {
        if (p.in_bcast[k] == 0 && esize(p.in_dtype[k]) != 2) v8 = false;
        if ((p.in_bcast[k] == 1 || p.in_bcast[k] == 2) && p.cols % 8) v8 = false;
    }
    const int V = v8 ? 8 : 4;
    for (int k = 0; k < p.n_in; k++)
        if ((p.in_bcast[k] == 1 || p.in_bcast[k] == 2) && p.cols % V) return false;
    *Vout = V;
    return true;
}

std::string ew_jit_source(const Elementwise &p, int V, int U) {
    const bool ireg = p.reg_class == DT_I32;
    const char *R = ireg ? "int" : "float";
    const int64_t n = p.rows * p.cols, nvec = n / V;
    // A result stored in 16 bits keeps 8 or 11 significant bits: the sigmoid family then runs on the hardware's
    // exp2 and reciprocal approximations (1 ulp of f32 each) instead of the library routines.
    const bool fast16 = esize(p.out_dtype) == 2;
    Gen g;
    g.s = kPrelude;
    g.f("\ntypedef unsigned int u32x4 __attribute__((ext_vector_type(4)));\ntypedef unsigned int u32x2 __attribute__((ext_vector_type(2)));\n");
    g.f("extern \"C\" __global__ __launch_bounds__(256) void zk_ew(const char *__restrict__ in0, const char *__restrict__ in1,\n"
        "        const char *__restrict__ in2, const char *__restrict__ in3, char *__restrict__ out) {\n");
    g.f("    const long NVEC = %lldL;\n", (long long)nvec);
    for (int c = 0; c < 8; c++) {
        uint32_t bits;
        memcpy(&bits, &p.consts[c], 4);
        g.f("    const %s c%d = (%s)__uint_as_float(0x%08xu);\n", R, c, R, bits);
    }
    // every wave owns U consecutive pieces of 64 vectors: its requests cover one contiguous stretch of every operand
    g.f("    const long v = ((long)blockIdx.x * 4L + (threadIdx.x >> 6)) * %dL + (threadIdx.x & 63);\n", 64 * U);

    // which inputs does the program read?
    bool used[4] = {false, false, false, false};
    for (int j = 0; j < p.n_instr; j++) {
        const int op = p.code[j] & 0xff, sa = (p.code[j] >> 8) & 0xff, sb = (p.code[j] >> 16) & 0xff;
        const bool unary = (op >= 2 && op <= 14) || op >= 38 || op == 1;
        if (!unary && sa < 4) used[sa] = true;
        if ((op == 36 || op == 37) && sb < 4) used[sb] = true;
    }
    auto loads = [&](int u) { // requests for the full-tensor operands of vector u
        for (int k = 0; k < p.n_in; k++) {
            if (!used[k] || p.in_bcast[k] != 0) continue;
            char name[32], off[64], ptr[16];
            snprintf(name, sizeof name, "r%d_%d_", u, k);
            snprintf(off, sizeof off, "(v + %d) * %d", u * 64, V * esize(p.in_dtype[k]));
            snprintf(ptr, sizeof ptr, "in%d", k);
            emit_load(g, name, ptr, off, V * esize(p.in_dtype[k]), true);
        }
    };
    auto body = [&](int u) {
        g.f("        {\n        const long i0 = (v + %d) * %d;\n", u * 64, V);
        if (p.need_rowcol) {
            if (n < (1ll << 31)) g.f("        const unsigned int row = (unsigned int)i0 / %uu, col = (unsigned int)i0 - row * %uu;\n", (unsigned)p.cols, (unsigned)p.cols);
            else g.f("        const long row = i0 / %lldL, col = i0 - row * %lldL;\n", (long long)p.cols, (long long)p.cols);
        }
        for (int k = 0; k < p.n_in; k++) {
            if (!used[k]) continue;
            const int dt = p.in_dtype[k], es = esize(dt);
            char name[32];
            snprintf(name, sizeof name, "r%d_%d_", u, k);
            if (p.in_bcast[k] == 1) { // row vector [cols]: V consecutive elements at `col`
                char ptr[16], off[64];
                snprintf(ptr, sizeof ptr, "in%d", k);
                snprintf(off, sizeof off, "(long)col * %d", es);
                emit_load(g, name, ptr, off, V * es, false);
            }
            if (p.in_bcast[k] == 0 || p.in_bcast[k] == 1) {
                for (int e = 0; e < V; e++) g.f("        const %s x%d_%d = %s;\n", R, k, e, elem_expr(name, dt, e, ireg).c_str());
            } else { // column vector [rows] or scalar: one element
                const char *idx = p.in_bcast[k] == 2 ? "(long)row" : "0L";
                const char *raw = es == 4 ? "*(const unsigned int *)(in%d + %s * 4)" : (es == 2 ? "(unsigned int)*(const unsigned short *)(in%d + %s * 2)" : "(unsigned int)*(const unsigned char *)(in%d + %s)");
                g.f("        const unsigned int %s0 = ", name);
                g.f(raw, k, idx);
                g.f(";\n        const %s x%d = %s;\n", R, k, elem_expr(name, dt, 0, ireg).c_str());
            }
        }
        auto operand = [&](int src, int e) -> std::string {
            char b[32];
            if (src < 4) {
                if (p.in_bcast[src] == 0 || p.in_bcast[src] == 1) snprintf(b, sizeof b, "x%d_%d", src, e);
                else snprintf(b, sizeof b, "x%d", src);
            } else if (src == 0x10) snprintf(b, sizeof b, "t%d", e);
            else snprintf(b, sizeof b, "c%d", (src - 0x20) & 7);
            return b;
        };
        for (int e = 0; e < V; e++) g.f("        %s a%d = (%s)0, t%d = (%s)0;\n", R, e, R, e, R);
        for (int j = 0; j < p.n_instr; j++) {
            const int op = p.code[j] & 0xff, sa = (p.code[j] >> 8) & 0xff, sb = (p.code[j] >> 16) & 0xff;
            if (op == 1) {
                for (int e = 0; e < V; e++) g.f("        t%d = a%d;\n", e, e);
                continue;
            }
            const bool unary = (op >= 2 && op <= 14) || op >= 38;
            const bool three = op == 36 || op == 37;
            for (int e = 0; e < V; e++) {
                const std::string A = unary ? std::string("(") + R + ")0" : operand(sa, e);
                const std::string B = three ? operand(sb, e) : std::string("(") + R + ")0";
                const bool quick = !ireg && fast16 && (op == 39 || op == 40 || op == 41 || op == 44);
                g.f("        a%d = zkew::%s(%d, a%d, %s, %s);\n", e, ireg ? "op_i" : quick ? "op_f_quick" : "op_f", op, e, A.c_str(), B.c_str());
            }
        }
        // store
        const int odt = p.out_dtype, oes = esize(odt);
        const int words = V * oes / 4;
        for (int w = 0; w < words; w++) {
            if (oes == 4) g.f("        const unsigned int o%d = %s;\n", w, odt == DT_F32 ? (std::string("__float_as_uint((float)a") + std::to_string(w) + ")").c_str() : (std::string("(unsigned int)(int)a") + std::to_string(w)).c_str());
            else if (oes == 2) {
                const char *cv = odt == DT_BF16 ? "zkew::f32_to_bf16_bits" : "zkew::f32_to_f16_bits";
                g.f("        const unsigned int o%d = (%s((float)a%d) & 0xffffu) | (%s((float)a%d) << 16);\n", w, cv, 2 * w, cv, 2 * w + 1);
            } else
                g.f("        const unsigned int o%d = (unsigned int)(unsigned char)(int)a%d | ((unsigned int)(unsigned char)(int)a%d << 8) | "
                    "((unsigned int)(unsigned char)(int)a%d << 16) | ((unsigned int)(unsigned char)(int)a%d << 24);\n", w, 4 * w, 4 * w + 1, 4 * w + 2, 4 * w + 3);
        }
        if (words == 1) g.f("        *(unsigned int *)(out + i0 * %d) = o0;\n", oes);
        else if (words == 2) g.f("        __builtin_nontemporal_store(u32x2{o0, o1}, (u32x2 *)(out + i0 * %d));\n", oes);
        else
            for (int q = 0; q < words / 4; q++)
                g.f("        __builtin_nontemporal_store(u32x4{o%d, o%d, o%d, o%d}, (u32x4 *)(out + i0 * %d + %d));\n", 4 * q, 4 * q + 1, 4 * q + 2, 4 * q + 3, oes, 16 * q);
        g.f("        }\n");
    };
    g.f("    if (v + %d < NVEC) {\n", (U - 1) * 64); // all requests of the thread in flight before the first use
    for (int u = 0; u < U; u++) loads(u);
    for (int u = 0; u < U; u++) body(u);
    g.f("    } else {\n");
    for (int u = 0; u < U; u++) {
        g.f("    if (v + %d < NVEC) {\n", u * 64);
        loads(u);
        body(u);
        g.f("    }\n");
    }
    g.f("    }\n}\n");
    return g.s;
}

EwJit *ew_jit_compile(const Elementwise &p, std::string &err) {
    int V;
    if (!ew_jit_eligible(p, &V)) {
        err = "shape not eligible";
        return nullptr;
    }
    // two pieces of 64 vectors per wave (2 KiB of f32 per operand): with 8 and 4 pieces for one- and two-operand chains
    // the same kernels ran 1-9 % slower (gelu f32 46.4 -> 42.5 us, copy f32 43.8 -> 42.9 at 8192 x 4096), with one piece 1-4 %
    const int U = 2;
    const std::string src = ew_jit_source(p, V, U);
    // same code generation switches as the ahead-of-time kernels: gfx950, packed-FP32 instructions off
    // -ffp-contract=on: a*b+c fuses only inside one source expression, as in the interpreting kernel's build,
    // never across two ops of the chain
    const std::vector<const char *> opts = {"--offload-arch=gfx950", "-O3", "-std=c++17", "-ffp-contract=on",
                                            "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops"};
    const auto code = rtc_compile(src, opts, "zk_ew.hip", err);
    if (!code) return nullptr;
    EwJit *j = new EwJit();
    j->V = V;
    j->U = U;
    j->nvec = p.rows * p.cols / V;
    hipError_t e = hipModuleLoadData(&j->mod, code->data());
    if (e == hipSuccess) e = hipModuleGetFunction(&j->fn, j->mod, "zk_ew");
    if (e != hipSuccess) {
        err = std::string("module load: ") + hipGetErrorString(e);
        if (j->mod) (void)hipModuleUnload(j->mod);
        delete j;
        return nullptr;
    }
    return j;
}

void ew_jit_destroy(EwJit *j) {
    if (!j) return;
    if (j->mod) (void)hipModuleUnload(j->mod);
    delete j;
}

// The generated code assumes 16-byte aligned tensors (the pool's blocks are 256-byte aligned).
bool ew_jit_can_launch(const EwJit *j, const Elementwise &p) {
    if (!j) return false;
    if (reinterpret_cast<uintptr_t>(p.out) % 16) return false;
    for (int k = 0; k < p.n_in; k++)
        if ((p.in_bcast[k] == 0 || p.in_bcast[k] == 1) && reinterpret_cast<uintptr_t>(p.in[k]) % 16) return false;
    return true;
}

hipError_t ew_jit_launch(const EwJit *j, const Elementwise &p, hipStream_t st) {
    const int64_t blocks = (j->nvec + 256 * j->U - 1) / (256 * j->U); // one pass: a thread's U vectors are all it does
    if (blocks < 1 || blocks >= (1ll << 31)) return hipErrorInvalidValue;
    const void *in[4] = {p.in[0], p.in[1], p.in[2], p.in[3]};
    void *out = p.out;
    void *args[5] = {&in[0], &in[1], &in[2], &in[3], &out};
    return hipModuleLaunchKernel(j->fn, (unsigned)blocks, 1, 1, 256, 1, 1, 0, st, args, nullptr);
}

} // namespace zk
