// Device::compile for the HIP slot: source generation for a linearized kernel, the job generate_cuda does for
// CUDA (zyx/src/codegen/cuda.rs:18-396) with the C backend's meaning of every op (zyx/src/codegen/c.rs:74-395,
// 583-612): one SSA value per op, declared at the top of the function like the reference's register file;
// bf16 / f16 values are f32 in registers and in register / local storage, widen on a load from global memory and
// truncate on a store to it; comparisons give 0 / 1 in an unsigned char; indices are 64-bit. Where C leaves the
// result open this code picks one: integer division or remainder by zero gives 0, shift counts are taken modulo
// the width, signed arithmetic wraps (-fwrapv). a * b is never fused with a following add unless the kernel says
// Mad (-ffp-contract=off), so kernels without Mad round exactly like the scalar C loop.
#include "ir_compile.hpp"

#include "rtc_cache.hpp"

#include <cmath>
#include <cstdarg>
#include <cstdio>
#include <cstring>
#include <map>
#include <set>

#include "../../include/zyx_hip.h"

namespace zk {
namespace {

// storage <-> register conversions of the 16-bit floats, shared with the elementwise chains
const char kConv[] =
#include "ew_ops_src.inc"
    ;

const char kHelpers[] = R"ZIR(
template <class T> __device__ __forceinline__ T zir_div(T x, T y) {
    if (y == (T)0) return (T)0;
    if ((T)-1 < (T)0 && y == (T)-1) return (T)((T)0 - x);
    return (T)(x / y);
}
__device__ __forceinline__ int zir_mod(int x, int y) { return (y == 0 || y == -1) ? 0 : x % y; }
)ZIR";

bool is_f16ish(int dt) { return dt == ZHIP_BF16 || dt == ZHIP_F16; }
bool is_f32reg(int dt) { return dt == ZHIP_BF16 || dt == ZHIP_F16 || dt == ZHIP_F32; }
bool is_float(int dt) { return is_f32reg(dt) || dt == ZHIP_F64; }
bool is_signed_int(int dt) { return dt == ZHIP_I8 || dt == ZHIP_I16 || dt == ZHIP_I32 || dt == ZHIP_I64; }

// register type of a dtype (c.rs:614-629)
const char *reg_type(int dt) {
    switch (dt) {
    case ZHIP_BF16: case ZHIP_F16: case ZHIP_F32: return "float";
    case ZHIP_F64: return "double";
    case ZHIP_U8: case ZHIP_BOOL: return "unsigned char";
    case ZHIP_U16: return "unsigned short";
    case ZHIP_U32: return "unsigned int";
    case ZHIP_U64: return "unsigned long long";
    case ZHIP_I8: return "signed char";
    case ZHIP_I16: return "short";
    case ZHIP_I32: return "int";
    case ZHIP_I64: return "long long";
    default: return nullptr;
    }
}
// element type in global memory
const char *mem_type(int dt) { return is_f16ish(dt) ? "unsigned short" : reg_type(dt); }
int mem_bytes(int dt) {
    switch (dt) {
    case ZHIP_BF16: case ZHIP_F16: case ZHIP_U16: case ZHIP_I16: return 2;
    case ZHIP_F32: case ZHIP_U32: case ZHIP_I32: return 4;
    case ZHIP_F64: case ZHIP_U64: case ZHIP_I64: return 8;
    case ZHIP_U8: case ZHIP_I8: case ZHIP_BOOL: return 1;
    default: return 0;
    }
}
int bits_of(int dt) { return mem_bytes(dt) * 8; }

std::string fmt(const char *f, ...) __attribute__((format(printf, 1, 2)));
std::string fmt(const char *f, ...) {
    char buf[512];
    va_list ap;
    va_start(ap, f);
    vsnprintf(buf, sizeof buf, f, ap);
    va_end(ap);
    return buf;
}

float f16_to_f32_host(uint16_t h) {
    const uint32_t sign = (uint32_t)(h & 0x8000u) << 16, ex = (h >> 10) & 31u, man = h & 0x3ffu;
    uint32_t f;
    if (ex == 0) {
        if (man == 0) f = sign;
        else {
            int e = -1;
            uint32_t m = man;
            while (!(m & 0x400u)) { m <<= 1; e--; }
            f = sign | (uint32_t)(127 - 15 + 1 + e) << 23 | (m & 0x3ffu) << 13;
        }
    } else if (ex == 31) f = sign | 0x7f800000u | man << 13;
    else f = sign | (ex + 112) << 23 | man << 13;
    float r;
    memcpy(&r, &f, 4);
    return r;
}

std::string float_literal(double v, bool f32) {
    if (std::isnan(v)) return f32 ? "__builtin_nanf(\"\")" : "__builtin_nan(\"\")";
    if (std::isinf(v)) return fmt("(%s__builtin_huge_val%s())", v < 0 ? "-" : "", f32 ? "f" : "");
    return fmt("(%a%s)", v, f32 ? "f" : ""); // hexadecimal floating literal: exact
}

// Constant::c_code (c.rs:632-652), as an exact literal of the register type
std::string const_literal(int dt, uint64_t imm) {
    switch (dt) {
    case ZHIP_BF16: {
        const uint32_t b = (uint32_t)(imm & 0xffffu) << 16;
        float f;
        memcpy(&f, &b, 4);
        return float_literal(f, true);
    }
    case ZHIP_F16: return float_literal(f16_to_f32_host((uint16_t)imm), true);
    case ZHIP_F32: {
        const uint32_t b = (uint32_t)imm;
        float f;
        memcpy(&f, &b, 4);
        return float_literal(f, true);
    }
    case ZHIP_F64: {
        double d;
        memcpy(&d, &imm, 8);
        return float_literal(d, false);
    }
    case ZHIP_BOOL: return imm & 0xff ? "((unsigned char)1)" : "((unsigned char)0)";
    default: {
        const int bits = bits_of(dt);
        const uint64_t mask = bits == 64 ? ~0ull : ((1ull << bits) - 1);
        return fmt("((%s)0x%llxULL)", reg_type(dt), (unsigned long long)(imm & mask));
    }
    }
}

struct Val {
    enum Cls { Value, Const, Param, Storage, LoopVar, None } cls = Value; // None: the op yields nothing an operand can name
    int dtype = 0;
    int vlen = 0;     // 0 scalar, else lanes
    int kind = 0;     // Param: zhip_ir_param_kind, Storage: zhip_ir_scope
    int ordinal = -1; // Param: position among the parameters
    uint64_t imm = 0;
    std::string name; // expression naming the value (literal for a constant)
    int depth = 0;    // loop nesting depth at the definition (a loop variable dies with its loop)
    bool open = true; // LoopVar: its loop is still open
};

struct Gen {
    std::map<uint32_t, Val> vals;
    std::set<std::string> vec_types;
    std::string decls, body, typedefs, args;
    std::string indent = "  ";
    std::string &err; // the caller's reason string
    explicit Gen(std::string &e) : err(e) {}

    bool fail(size_t i, const std::string &m) {
        err = fmt("op %zu: ", i) + m;
        return false;
    }
    std::string vec_type(const char *base, int n, bool memory) {
        std::string b = base;
        for (char &ch : b)
            if (ch == ' ') ch = '_';
        std::string name = fmt("zir_%s_x%d%s", b.c_str(), n, memory ? "_m" : "");
        if (vec_types.insert(name).second) {
            // memory flavour: element alignment only, so any index a scalar load could use is legal
            if (memory) typedefs += fmt("typedef %s %s __attribute__((ext_vector_type(%d), aligned(__alignof__(%s))));\n", base, name.c_str(), n, base);
            else typedefs += fmt("typedef %s %s __attribute__((ext_vector_type(%d)));\n", base, name.c_str(), n);
        }
        return name;
    }
    std::string reg_decl_type(int dt, int vlen) { return vlen ? vec_type(reg_type(dt), vlen, false) : std::string(reg_type(dt)); }
    static std::string lane(const Val &v, int i) { return (v.vlen && v.cls != Val::Const) ? fmt("%s[%d]", v.name.c_str(), i) : v.name; }
    void line(const std::string &s) { body += indent + s + "\n"; }
};

bool valid_vlen(uint32_t n) { return n == 0 || n == 2 || n == 4 || n == 8 || n == 16; }

// expression of one lane of a unary op (c.rs:286-304); empty = no meaning for this dtype
std::string unary_expr(int uop, int dt, const std::string &x) {
    const char *T = reg_type(dt);
    if (is_float(dt)) {
        const bool d = dt == ZHIP_F64;
        const char *s = d ? "" : "f";
        switch (uop) {
        case ZHIP_IR_NEG: return "-" + x;
        case ZHIP_IR_EXP: return fmt("exp%s(%s)", s, x.c_str());
        case ZHIP_IR_EXP2: return fmt("exp2%s(%s)", s, x.c_str());
        case ZHIP_IR_LN: return fmt("log%s(%s)", s, x.c_str());
        case ZHIP_IR_LOG2: return fmt("log2%s(%s)", s, x.c_str());
        case ZHIP_IR_RECIPROCAL: return fmt("%s / %s", d ? "1.0" : "1.0f", x.c_str());
        case ZHIP_IR_SQRT: return fmt("sqrt%s(%s)", s, x.c_str());
        case ZHIP_IR_SIN: return fmt("sin%s(%s)", s, x.c_str());
        case ZHIP_IR_COS: return fmt("cos%s(%s)", s, x.c_str());
        case ZHIP_IR_FLOOR: return fmt("floor%s(%s)", s, x.c_str());
        case ZHIP_IR_TRUNC: return fmt("trunc%s(%s)", s, x.c_str());
        case ZHIP_IR_ABS: return fmt("fabs%s(%s)", s, x.c_str());
        default: return "";
        }
    }
    switch (uop) { // integers and Bool: the C expression on the integer, math functions through double
    case ZHIP_IR_NEG: return fmt("(%s)(-%s)", T, x.c_str());
    case ZHIP_IR_BITNOT: return fmt("(%s)(~%s)", T, x.c_str());
    case ZHIP_IR_ABS: return is_signed_int(dt) ? fmt("(%s)(%s < 0 ? -%s : %s)", T, x.c_str(), x.c_str(), x.c_str()) : x;
    case ZHIP_IR_RECIPROCAL: return fmt("zir_div<%s>((%s)1, %s)", T, T, x.c_str());
    case ZHIP_IR_FLOOR: case ZHIP_IR_TRUNC: return x;
    case ZHIP_IR_EXP: return fmt("(%s)exp((double)%s)", T, x.c_str());
    case ZHIP_IR_EXP2: return fmt("(%s)exp2((double)%s)", T, x.c_str());
    case ZHIP_IR_LN: return fmt("(%s)log((double)%s)", T, x.c_str());
    case ZHIP_IR_LOG2: return fmt("(%s)log2((double)%s)", T, x.c_str());
    case ZHIP_IR_SQRT: return fmt("(%s)sqrt((double)%s)", T, x.c_str());
    case ZHIP_IR_SIN: return fmt("(%s)sin((double)%s)", T, x.c_str());
    case ZHIP_IR_COS: return fmt("(%s)cos((double)%s)", T, x.c_str());
    default: return "";
    }
}

// expression of one lane of a binary op (c.rs:583-612); dt = dtype of x, the result's unless it is a Bool
std::string binary_expr(int bop, int dt, const std::string &x, const std::string &y) {
    const char *T = reg_type(dt);
    const char *a = x.c_str(), *b = y.c_str();
    switch (bop) {
    case ZHIP_IR_CMPLT: return fmt("(unsigned char)(%s < %s)", a, b);
    case ZHIP_IR_CMPGT: return fmt("(unsigned char)(%s > %s)", a, b);
    case ZHIP_IR_CMPGE: return fmt("(unsigned char)(%s >= %s)", a, b);
    case ZHIP_IR_NOTEQ: return fmt("(unsigned char)(%s != %s)", a, b);
    case ZHIP_IR_EQ: return fmt("(unsigned char)(%s == %s)", a, b);
    case ZHIP_IR_OR: return fmt("(unsigned char)(%s || %s)", a, b);
    case ZHIP_IR_AND: return fmt("(unsigned char)(%s && %s)", a, b);
    default: break;
    }
    if (is_float(dt)) {
        const bool d = dt == ZHIP_F64;
        switch (bop) {
        case ZHIP_IR_ADD: return fmt("%s + %s", a, b);
        case ZHIP_IR_SUB: return fmt("%s - %s", a, b);
        case ZHIP_IR_MUL: return fmt("%s * %s", a, b);
        case ZHIP_IR_DIV: return fmt("%s / %s", a, b);
        case ZHIP_IR_POW: return fmt("%s(%s, %s)", d ? "pow" : "powf", a, b);
        case ZHIP_IR_MOD: return fmt("(%s)zir_mod((int)%s, (int)%s)", T, a, b);
        case ZHIP_IR_MAX: return fmt("%s(%s, %s)", d ? "fmax" : "fmaxf", a, b);
        default: return ""; // bit operations have no meaning on floats
        }
    }
    const int mask = bits_of(dt) - 1;
    switch (bop) {
    case ZHIP_IR_ADD: return fmt("(%s)(%s + %s)", T, a, b);
    case ZHIP_IR_SUB: return fmt("(%s)(%s - %s)", T, a, b);
    case ZHIP_IR_MUL: return fmt("(%s)(%s * %s)", T, a, b);
    case ZHIP_IR_DIV: return fmt("zir_div<%s>(%s, (%s)%s)", T, a, T, b);
    case ZHIP_IR_POW: return fmt("(%s)pow((double)%s, (double)%s)", T, a, b);
    case ZHIP_IR_MOD: return fmt("(%s)zir_mod((int)%s, (int)%s)", T, a, b);
    case ZHIP_IR_MAX: return fmt("(%s)(%s > (%s)%s ? %s : (%s)%s)", T, a, T, b, a, T, b);
    case ZHIP_IR_BITXOR: return fmt("(%s)(%s ^ %s)", T, a, b);
    case ZHIP_IR_BITOR: return fmt("(%s)(%s | %s)", T, a, b);
    case ZHIP_IR_BITAND: return fmt("(%s)(%s & %s)", T, a, b);
    case ZHIP_IR_SHL: return fmt("(%s)(%s << ((int)%s & %d))", T, a, b, mask);
    case ZHIP_IR_SHR: return fmt("(%s)(%s >> ((int)%s & %d))", T, a, b, mask);
    default: return "";
    }
}

bool returns_bool(int bop) { // BOp::returns_bool (ops.rs:279-282)
    return bop == ZHIP_IR_CMPLT || bop == ZHIP_IR_CMPGT || bop == ZHIP_IR_CMPGE || bop == ZHIP_IR_NOTEQ || bop == ZHIP_IR_EQ ||
           bop == ZHIP_IR_OR || bop == ZHIP_IR_AND;
}

} // namespace

bool ir_generate(const void *image, uint64_t bytes, IrProgram &out, std::string &err) {
    Gen g(err);
    if (!image || bytes < sizeof(zhip_ir_header)) {
        err = "kernel image shorter than its header";
        return false;
    }
    zhip_ir_header h;
    memcpy(&h, image, sizeof h);
    if (h.magic != ZHIP_IR_MAGIC) {
        err = "kernel image: bad magic";
        return false;
    }
    if (h.n_ops == 0 || h.n_ops > (1u << 20) || h.n_extra > (1u << 24) ||
        bytes != sizeof h + (uint64_t)h.n_ops * sizeof(zhip_ir_op) + (uint64_t)h.n_extra * 4) {
        err = "kernel image: size does not match its header";
        return false;
    }
    std::vector<zhip_ir_op> ops(h.n_ops);
    memcpy(ops.data(), (const uint8_t *)image + sizeof h, (size_t)h.n_ops * sizeof(zhip_ir_op));
    std::vector<uint32_t> extra(h.n_extra);
    if (h.n_extra) memcpy(extra.data(), (const uint8_t *)image + sizeof h + (size_t)h.n_ops * sizeof(zhip_ir_op), (size_t)h.n_extra * 4);

    bool have_group[3] = {false, false, false}, have_local[3] = {false, false, false};
    std::vector<char> blocks; // 'L' loop, 'I' if
    std::vector<uint32_t> open_loops;
    int depth = 0;

    // an operand must name an earlier op that yields a value
    auto value_of = [&](size_t i, uint32_t id, const Val **v) -> bool {
        auto it = g.vals.find(id);
        if (it == g.vals.end()) return g.fail(i, fmt("operand %u is not defined before its use", id));
        const Val &x = it->second;
        if (x.cls == Val::None) return g.fail(i, fmt("operand %u yields no value", id));
        if (x.cls == Val::Storage || (x.cls == Val::Param && x.kind != ZHIP_IR_VARIABLE))
            return g.fail(i, fmt("operand %u is memory, a value is needed", id));
        if (x.cls == Val::LoopVar && !x.open) return g.fail(i, fmt("operand %u is the variable of a loop that has ended", id));
        *v = &x;
        return true;
    };

    for (size_t i = 0; i < ops.size(); i++) {
        const zhip_ir_op &o = ops[i];
        if (o.id == ZHIP_IR_NULL || g.vals.count(o.id)) return g.fail(i, fmt("op id %u is null or defined twice", o.id));
        Val v;
        v.depth = depth;
        const std::string vn = fmt("v%u", o.id);
        bool declares = false; // a value variable declared at the top
        switch (o.opcode) {
        case ZHIP_IR_CONST: {
            if (!reg_type(o.dtype)) return g.fail(i, "constant of unknown dtype");
            v.cls = Val::Const;
            v.dtype = o.dtype;
            v.imm = o.imm;
            v.name = const_literal(o.dtype, o.imm);
            break;
        }
        case ZHIP_IR_PARAM: {
            if (!reg_type(o.dtype)) return g.fail(i, "parameter of unknown dtype");
            if (o.aux > ZHIP_IR_GLOBAL_MUT) return g.fail(i, "parameter of unknown kind");
            if (out.params.size() >= ZHIP_IR_MAX_PARAMS) return g.fail(i, fmt("more than %d parameters", ZHIP_IR_MAX_PARAMS));
            v.cls = Val::Param;
            v.dtype = o.dtype;
            v.kind = (int)o.aux;
            v.ordinal = (int)out.params.size();
            v.name = fmt("p%u", o.id);
            if (!g.args.empty()) g.args += ",\n";
            if (o.aux == ZHIP_IR_VARIABLE) {
                if (is_f16ish(o.dtype)) { // passed as its 16 bits, widened once (c.rs:48-56, 126-130)
                    g.args += fmt("    const unsigned short q%u", o.id);
                    g.decls += fmt("  const float p%u = zkew::%s(q%u);\n", o.id, o.dtype == ZHIP_BF16 ? "bf16_bits_to_f32" : "f16_bits_to_f32", o.id);
                } else g.args += fmt("    const %s p%u", reg_type(o.dtype), o.id);
            } else g.args += fmt("    %s%s *p%u", o.aux == ZHIP_IR_GLOBAL ? "const " : "", mem_type(o.dtype), o.id);
            out.params.push_back(IrParam{(int)o.aux, (int)o.dtype, o.imm});
            break;
        }
        case ZHIP_IR_STORAGE: {
            if (!reg_type(o.dtype)) return g.fail(i, "storage of unknown dtype");
            if (o.aux != ZHIP_IR_SCOPE_LOCAL && o.aux != ZHIP_IR_SCOPE_REGISTER)
                return g.fail(i, "storage must be local or register scoped");
            // local memory: what one workgroup can have on this part (160 KiB); register arrays: a bound that keeps
            // a corrupt length from asking the compiler for gigabytes of scratch
            if (o.imm == 0 || (o.aux == ZHIP_IR_SCOPE_LOCAL ? o.imm * (uint64_t)(is_f16ish(o.dtype) ? 4 : mem_bytes(o.dtype)) > 160u * 1024 : o.imm > 16384))
                return g.fail(i, "storage length out of range");
            if (o.aux == ZHIP_IR_SCOPE_LOCAL && depth) return g.fail(i, "local storage must be declared outside loops and branches");
            v.cls = Val::Storage;
            v.dtype = o.dtype;
            v.kind = (int)o.aux;
            v.imm = o.imm;
            v.name = fmt("s%u", o.id);
            g.line(fmt("%s%s s%u[%llu];", o.aux == ZHIP_IR_SCOPE_LOCAL ? "__shared__ " : "", reg_type(o.dtype), o.id, (unsigned long long)o.imm));
            break;
        }
        case ZHIP_IR_LOAD: {
            auto it = g.vals.find(o.a);
            if (it == g.vals.end()) return g.fail(i, fmt("load source %u is not defined", o.a));
            const Val &src = it->second;
            if (src.cls != Val::Param && src.cls != Val::Storage) return g.fail(i, "load source must be a parameter or storage");
            if (!valid_vlen(o.aux)) return g.fail(i, "unsupported vector length");
            v.dtype = src.dtype;
            v.vlen = (int)o.aux;
            v.name = vn;
            declares = true;
            if (src.cls == Val::Param && src.kind == ZHIP_IR_VARIABLE) {
                if (v.vlen) return g.fail(i, "vector load of a scalar parameter");
                g.line(fmt("%s = %s;", vn.c_str(), src.name.c_str()));
                break;
            }
            const Val *idx;
            if (!value_of(i, o.b, &idx)) return false;
            if (idx->vlen) return g.fail(i, "index must be a scalar");
            const bool widen = src.cls == Val::Param && is_f16ish(src.dtype);
            const char *conv = src.dtype == ZHIP_BF16 ? "zkew::bf16_bits_to_f32" : "zkew::f16_bits_to_f32";
            if (!v.vlen) {
                if (widen) g.line(fmt("%s = %s(%s[%s]);", vn.c_str(), conv, src.name.c_str(), idx->name.c_str()));
                else g.line(fmt("%s = %s[%s];", vn.c_str(), src.name.c_str(), idx->name.c_str()));
            } else {
                const char *mt = src.cls == Val::Param ? mem_type(src.dtype) : reg_type(src.dtype);
                const std::string vt = g.vec_type(mt, v.vlen, true);
                if (widen) {
                    g.line(fmt("{ const %s t = *(const %s *)(%s + %s);", vt.c_str(), vt.c_str(), src.name.c_str(), idx->name.c_str()));
                    for (int l = 0; l < v.vlen; l++) g.line(fmt("  %s[%d] = %s(t[%d]);", vn.c_str(), l, conv, l));
                    g.line("}");
                } else g.line(fmt("%s = *(const %s *)(%s + %s);", vn.c_str(), vt.c_str(), src.name.c_str(), idx->name.c_str()));
            }
            break;
        }
        case ZHIP_IR_STORE: {
            auto it = g.vals.find(o.a);
            if (it == g.vals.end()) return g.fail(i, fmt("store destination %u is not defined", o.a));
            const Val &dst = it->second;
            if (!(dst.cls == Val::Storage || (dst.cls == Val::Param && dst.kind == ZHIP_IR_GLOBAL_MUT)))
                return g.fail(i, "store destination must be a writable global parameter or storage");
            if (!valid_vlen(o.aux)) return g.fail(i, "unsupported vector length");
            const Val *src, *idx;
            if (!value_of(i, o.b, &src) || !value_of(i, o.c, &idx)) return false;
            if (idx->vlen) return g.fail(i, "index must be a scalar");
            const int vlen = (int)o.aux;
            if (src->cls != Val::Const && src->vlen != vlen) return g.fail(i, "stored value and store layout differ in vector length");
            const bool narrow = dst.cls == Val::Param && is_f16ish(dst.dtype);
            const char *conv = dst.dtype == ZHIP_BF16 ? "zkew::f32_to_bf16_bits" : "zkew::f32_to_f16_bits";
            const char *et = dst.cls == Val::Param ? mem_type(dst.dtype) : reg_type(dst.dtype);
            if (!vlen) {
                if (narrow) g.line(fmt("%s[%s] = (unsigned short)%s((float)%s);", dst.name.c_str(), idx->name.c_str(), conv, src->name.c_str()));
                else g.line(fmt("%s[%s] = (%s)%s;", dst.name.c_str(), idx->name.c_str(), et, src->name.c_str()));
            } else {
                const std::string vt = g.vec_type(et, vlen, true);
                g.line(fmt("{ %s t;", vt.c_str()));
                for (int l = 0; l < vlen; l++) {
                    if (narrow) g.line(fmt("  t[%d] = (unsigned short)%s((float)%s);", l, conv, Gen::lane(*src, l).c_str()));
                    else g.line(fmt("  t[%d] = (%s)%s;", l, et, Gen::lane(*src, l).c_str()));
                }
                g.line(fmt("  *(%s *)(%s + %s) = t; }", vt.c_str(), dst.name.c_str(), idx->name.c_str()));
            }
            v.cls = Val::None;
            break;
        }
        case ZHIP_IR_CAST: {
            const Val *x;
            if (!value_of(i, o.a, &x)) return false;
            if (!reg_type(o.dtype)) return g.fail(i, "cast to unknown dtype");
            v.dtype = o.dtype;
            v.vlen = x->vlen;
            v.name = vn;
            declares = true;
            for (int l = 0; l < (v.vlen ? v.vlen : 1); l++) // (T)x; to bf16 / f16 it is (float)x, no rounding (c.rs:243-261)
                g.line(fmt("%s = (%s)%s;", v.vlen ? fmt("%s[%d]", vn.c_str(), l).c_str() : vn.c_str(), reg_type(o.dtype), Gen::lane(*x, l).c_str()));
            break;
        }
        case ZHIP_IR_UNARY: {
            const Val *x;
            if (!value_of(i, o.a, &x)) return false;
            v.dtype = x->dtype;
            v.vlen = x->vlen;
            v.name = vn;
            declares = true;
            for (int l = 0; l < (v.vlen ? v.vlen : 1); l++) {
                const std::string e = unary_expr((int)o.aux, x->dtype, Gen::lane(*x, l));
                if (e.empty()) return g.fail(i, fmt("unary op %u has no meaning for dtype %d", o.aux, x->dtype));
                g.line(fmt("%s = %s;", v.vlen ? fmt("%s[%d]", vn.c_str(), l).c_str() : vn.c_str(), e.c_str()));
            }
            break;
        }
        case ZHIP_IR_BINARY: {
            const Val *x, *y;
            if (!value_of(i, o.a, &x) || !value_of(i, o.b, &y)) return false;
            if (x->vlen && y->vlen && x->vlen != y->vlen) return g.fail(i, "operands differ in vector length");
            v.dtype = returns_bool((int)o.aux) ? (int)ZHIP_BOOL : x->dtype;
            v.vlen = x->vlen ? x->vlen : y->vlen;
            v.name = vn;
            declares = true;
            for (int l = 0; l < (v.vlen ? v.vlen : 1); l++) {
                const std::string e = binary_expr((int)o.aux, x->dtype, Gen::lane(*x, l), Gen::lane(*y, l));
                if (e.empty()) return g.fail(i, fmt("binary op %u has no meaning for dtype %d", o.aux, x->dtype));
                g.line(fmt("%s = %s;", v.vlen ? fmt("%s[%d]", vn.c_str(), l).c_str() : vn.c_str(), e.c_str()));
            }
            break;
        }
        case ZHIP_IR_MAD: {
            const Val *x, *y, *z;
            if (!value_of(i, o.a, &x) || !value_of(i, o.b, &y) || !value_of(i, o.c, &z)) return false;
            v.dtype = x->dtype;
            v.vlen = x->vlen ? x->vlen : (y->vlen ? y->vlen : z->vlen);
            v.name = vn;
            declares = true;
            for (int l = 0; l < (v.vlen ? v.vlen : 1); l++) {
                const std::string a = Gen::lane(*x, l), b = Gen::lane(*y, l), c = Gen::lane(*z, l);
                std::string e;
                if (is_f32reg(x->dtype)) e = fmt("fmaf(%s, %s, %s)", a.c_str(), b.c_str(), c.c_str());
                else if (x->dtype == ZHIP_F64) e = fmt("fma(%s, %s, %s)", a.c_str(), b.c_str(), c.c_str());
                else e = fmt("(%s)(%s * %s + %s)", reg_type(x->dtype), a.c_str(), b.c_str(), c.c_str());
                g.line(fmt("%s = %s;", v.vlen ? fmt("%s[%d]", vn.c_str(), l).c_str() : vn.c_str(), e.c_str()));
            }
            break;
        }
        case ZHIP_IR_STACK: {
            if (!valid_vlen(o.b) || o.b == 0 || (uint64_t)o.a + o.b > extra.size()) return g.fail(i, "stack operand list out of range");
            v.vlen = (int)o.b;
            v.name = vn;
            declares = true;
            for (uint32_t l = 0; l < o.b; l++) {
                const Val *x;
                if (!value_of(i, extra[o.a + l], &x)) return false;
                if (x->vlen) return g.fail(i, "stack of vectors");
                if (l == 0) v.dtype = x->dtype;
                g.line(fmt("%s[%u] = (%s)%s;", vn.c_str(), l, reg_type(v.dtype), x->name.c_str()));
            }
            break;
        }
        case ZHIP_IR_DEVECTORIZE: {
            const Val *x;
            if (!value_of(i, o.a, &x)) return false;
            if (!x->vlen || (int)o.aux >= x->vlen) return g.fail(i, "lane out of range");
            v.dtype = x->dtype;
            v.name = vn;
            declares = true;
            g.line(fmt("%s = %s;", vn.c_str(), Gen::lane(*x, (int)o.aux).c_str()));
            break;
        }
        case ZHIP_IR_INDEX: {
            const uint32_t axis = o.aux & 0xff, kind = o.aux >> 8;
            if (axis > 2) return g.fail(i, "index axis above 2");
            static const char *xyz[3] = {"x", "y", "z"};
            v.dtype = ZHIP_I64; // IDX_T (kernel/mod.rs:131)
            v.name = vn;
            declares = true;
            if (kind == ZHIP_IR_IDX_GROUP) {
                if (have_group[axis]) return g.fail(i, "two group indices on one axis");
                have_group[axis] = true;
                auto it = g.vals.find(o.a);
                if (it == g.vals.end()) return g.fail(i, "group length is not defined");
                const Val &len = it->second;
                if (len.cls == Val::Const) {
                    if (is_float(len.dtype)) return g.fail(i, "group length must be an integer");
                    const int bits = bits_of(len.dtype);
                    out.grid[axis].value = bits == 64 ? len.imm : (len.imm & ((1ull << bits) - 1));
                } else if (len.cls == Val::Param && len.kind == ZHIP_IR_VARIABLE && !is_float(len.dtype)) {
                    out.grid[axis].from_param = true;
                    out.grid[axis].ordinal = len.ordinal;
                } else return g.fail(i, "group length must be a constant or an integer Variable parameter"); // backend/mod.rs:84-88
                g.line(fmt("%s = (long long)blockIdx.%s;", vn.c_str(), xyz[axis]));
            } else if (kind == ZHIP_IR_IDX_LOCAL) {
                if (have_local[axis]) return g.fail(i, "two local indices on one axis");
                have_local[axis] = true;
                if (o.imm == 0 || o.imm > 1024) return g.fail(i, "local length out of range");
                out.block[axis] = (unsigned)o.imm;
                g.line(fmt("%s = (long long)threadIdx.%s;", vn.c_str(), xyz[axis]));
            } else return g.fail(i, "warp indices have no code"); // cuda.rs:304,310
            if (depth) return g.fail(i, "index inside a loop or branch");
            break;
        }
        case ZHIP_IR_LOOP: {
            const Val *len;
            if (!value_of(i, o.a, &len)) return false;
            if (len->vlen || is_float(len->dtype)) return g.fail(i, "loop length must be an integer scalar");
            v.cls = Val::LoopVar;
            v.dtype = ZHIP_I64;
            v.name = vn;
            g.line(fmt("for (long long %s = 0; %s < (long long)%s; ++%s) {", vn.c_str(), vn.c_str(), len->name.c_str(), vn.c_str()));
            g.indent += "  ";
            blocks.push_back('L');
            open_loops.push_back(o.id);
            depth++;
            break;
        }
        case ZHIP_IR_ENDLOOP: {
            if (blocks.empty() || blocks.back() != 'L') return g.fail(i, "EndLoop without an open loop");
            blocks.pop_back();
            g.vals[open_loops.back()].open = false;
            open_loops.pop_back();
            depth--;
            g.indent.resize(g.indent.size() - 2);
            g.line("}");
            break;
        }
        case ZHIP_IR_IF: {
            const Val *cnd;
            if (!value_of(i, o.a, &cnd)) return false;
            if (cnd->vlen) return g.fail(i, "branch condition must be a scalar");
            g.line(fmt("if (%s) {", cnd->name.c_str()));
            g.indent += "  ";
            blocks.push_back('I');
            depth++;
            break;
        }
        case ZHIP_IR_ENDIF: {
            if (blocks.empty() || blocks.back() != 'I') return g.fail(i, "EndIf without an open branch");
            blocks.pop_back();
            depth--;
            g.indent.resize(g.indent.size() - 2);
            g.line("}");
            break;
        }
        case ZHIP_IR_BARRIER: g.line("__syncthreads();"); break;
        case ZHIP_IR_WMMA: case ZHIP_IR_REDUCE_TILE: case ZHIP_IR_MATMUL_TILE: case ZHIP_IR_TRANSPOSE_TILE: case ZHIP_IR_ASM:
            return g.fail(i, "tile, tensor-core and assembly ops have no code in this backend");
        case ZHIP_IR_MOVE: case ZHIP_IR_REDUCE: return g.fail(i, "unexpected kernel op (should be unfolded)"); // cuda.rs:56-65
        default: return g.fail(i, fmt("unknown opcode %u", o.opcode));
        }
        if (declares) g.decls += fmt("  %s %s;\n", g.reg_decl_type(v.dtype, v.vlen).c_str(), vn.c_str());
        if (o.opcode == ZHIP_IR_ENDLOOP || o.opcode == ZHIP_IR_IF || o.opcode == ZHIP_IR_ENDIF || o.opcode == ZHIP_IR_BARRIER) v.cls = Val::None;
        g.vals[o.id] = v;
    }
    if (!blocks.empty()) {
        err = "kernel ends inside an open loop or branch";
        return false;
    }
    const uint64_t threads = (uint64_t)out.block[0] * out.block[1] * out.block[2];
    if (threads > 1024) {
        err = fmt("%llu threads per group, the device runs at most 1024", (unsigned long long)threads);
        return false;
    }
    out.source = "// generated from a linearized zyx kernel\n";
    out.source += kConv;
    out.source += kHelpers;
    out.source += g.typedefs;
    out.source += fmt("extern \"C\" __global__ void __launch_bounds__(%llu) zir_kernel(\n", (unsigned long long)threads);
    out.source += g.args;
    out.source += ") {\n";
    out.source += g.decls;
    out.source += g.body;
    out.source += "}\n";
    return true;
}

IrProgram *ir_compile(const void *image, uint64_t bytes, std::string &err) {
    IrProgram *p = new IrProgram();
    if (!ir_generate(image, bytes, *p, err)) {
        delete p;
        return nullptr;
    }
    // gfx950 only, packed-FP32 instructions off like every kernel of this library; no contraction, wrapping ints
    const std::vector<const char *> opts = {"--offload-arch=gfx950", "-O3", "-std=c++17", "-ffp-contract=off", "-fwrapv",
                                            "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops"};
    const auto code = rtc_compile(p->source, opts, "zir_kernel.hip", err);
    if (!code) {
        delete p;
        return nullptr;
    }
    hipError_t e = hipModuleLoadData(&p->mod, code->data());
    if (e == hipSuccess) e = hipModuleGetFunction(&p->fn, p->mod, "zir_kernel");
    if (e != hipSuccess) {
        err = std::string("loading the compiled kernel failed: ") + hipGetErrorString(e);
        if (p->mod) (void)hipModuleUnload(p->mod);
        delete p;
        return nullptr;
    }
    return p;
}

hipError_t ir_launch(const IrProgram *p, void *const *slots, hipStream_t stream, std::string *why) {
    uint64_t grid[3];
    static const uint64_t limit[3] = {2147483647ull, 65535ull, 65535ull};
    for (int a = 0; a < 3; a++) {
        grid[a] = p->grid[a].value;
        if (p->grid[a].from_param) { // GwsDim::Param: the Variable's value, as Constant::as_dim reads it (cuda.rs:730-736)
            const IrParam &q = p->params[p->grid[a].ordinal];
            uint64_t raw = 0;
            memcpy(&raw, slots[p->grid[a].ordinal], mem_bytes(q.dtype));
            if (is_signed_int(q.dtype)) {
                const int bits = bits_of(q.dtype);
                const int64_t s = bits == 64 ? (int64_t)raw : (int64_t)(raw << (64 - bits)) >> (64 - bits);
                if (s < 0) {
                    if (why) *why = "negative group count";
                    return hipErrorInvalidValue;
                }
            }
            grid[a] = raw;
        }
        if (grid[a] == 0) return hipSuccess; // an empty grid runs nothing
        if (grid[a] > limit[a]) {
            if (why) *why = fmt("group count %llu on axis %d is above the device's limit %llu", (unsigned long long)grid[a], a, (unsigned long long)limit[a]);
            return hipErrorInvalidValue;
        }
    }
    void *args[ZHIP_IR_MAX_PARAMS];
    for (size_t i = 0; i < p->params.size(); i++) args[i] = slots[i];
    return hipModuleLaunchKernel(p->fn, (unsigned)grid[0], (unsigned)grid[1], (unsigned)grid[2], p->block[0], p->block[1], p->block[2], 0,
                                 stream, args, nullptr);
}

void ir_destroy(IrProgram *p) {
    if (!p) return;
    if (p->mod) (void)hipModuleUnload(p->mod);
    delete p;
}

} // namespace zk
