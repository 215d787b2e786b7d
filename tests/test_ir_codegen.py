"""Source generation for linearized kernels, without a GPU: every test kernel's HIP source cross-compiles for gfx950
with the flags the run-time compiler gets, malformed or unsupported images are refused with KernelCompilation and a
reason, and the image layout matches the C header."""
import ctypes
import os
import shutil
import subprocess
import tempfile

import pytest

import ir_kernels as K
from zyx_amd import BackendError, DType, ErrorStatus
from zyx_amd import ir
from zyx_amd.backend import generate_source
from zyx_amd.ir import BOp, MemScope, Opcode, ParamKind, UOp

HIPCC = shutil.which("hipcc") or "/opt/rocm/bin/hipcc"


def kernels():
    return {
        "elementwise_bf16": K.elementwise(16, 256, (UOp.Exp2, UOp.Sin, UOp.Reciprocal), DType.BF16, DType.F16),
        "matmul_f32": K.matmul(64, 16, 97, local=(8, 4), first_id=7, id_step=3),
        "matmul_i64_mad": K.matmul(8, 8, 8, DType.I64, DType.I64, use_mad=True),
        "softmax": K.softmax_rows(64, 333),
        "row_sum_local": K.row_sum_local(6, 1024, 256),
        "padded_copy": K.padded_copy(37, 5, 9),
        "vector_axpy8_bf16": K.vector_axpy(3, 64, 8, DType.BF16),
        "vector_scale4": K.vector_scale(3, 64, 4),
        "dynamic_rows": K.dynamic_rows(64),
        "ragged_loop": K.ragged_loop(64),
        "u8_div": K.binary_table(256, DType.U8, BOp.Div),
        "i8_shift": K.binary_table(256, DType.I8, BOp.BitShiftRight),
        "f64_pow": K.binary_table(256, DType.F64, BOp.Pow),
        "i32_abs": K.unary_table(256, DType.I32, UOp.Abs),
        "cast_bool": K.cast_table(256, DType.F32, DType.Bool),
    }


def test_image_layout_matches_the_header():
    assert ctypes.sizeof(ir.IrHeader) == 16 and ctypes.sizeof(ir.IrOp) == 32
    assert ir.IrOp.imm.offset == 24 and ir.IrOp.aux.offset == 20 and ir.IrOp.opcode.offset == 4 and ir.IrOp.dtype.offset == 6
    k = K.vector_axpy(1, 64, 4)
    img = k.to_bytes()
    assert len(img) == 16 + 32 * len(k.ops) + 4 * len(k.extra) and img[:4] == b"ZIR1"
    hdr = open(os.path.join(os.path.dirname(__file__), "..", "include", "zyx_hip.h")).read()
    for name, members in (("zhip_ir_opcode", Opcode), ("zhip_ir_uop", UOp), ("zhip_ir_bop", BOp)):
        body = hdr[hdr.index("enum " + name):]
        body = body[body.index("{") + 1:body.index("}")]
        body = "\n".join(line.split("/*")[0] for line in body.splitlines())
        names = [t.split("=")[0].strip() for t in body.replace("\n", " ").split(",") if t.strip()]
        assert len(names) == len(members), name                    # same count, same order as the Python enums
    assert [m.name.upper() for m in UOp] == [n.replace("ZHIP_IR_", "") for n in
                                             "ZHIP_IR_NEG ZHIP_IR_BITNOT ZHIP_IR_EXP ZHIP_IR_EXP2 ZHIP_IR_LN ZHIP_IR_LOG2 ZHIP_IR_RECIPROCAL "
                                             "ZHIP_IR_SQRT ZHIP_IR_SIN ZHIP_IR_COS ZHIP_IR_FLOOR ZHIP_IR_TRUNC ZHIP_IR_ABS".split()]


def test_generated_source_shape():
    src = generate_source(K.matmul(64, 16, 97, local=(8, 4)).to_bytes())
    body = src[src.index('extern "C"'):]
    assert "__launch_bounds__(32)" in body and "blockIdx.y" in body and "threadIdx.y" in body
    assert body.count("for (long long") == 1 and "fmaf" not in body      # a product and a sum stay two roundings
    assert "fmaf" in generate_source(K.matmul(8, 8, 8, use_mad=True).to_bytes())
    src = generate_source(K.row_sum_local(6, 1024, 256).to_bytes())
    assert "__shared__ float" in src and src.count("__syncthreads();") == 9
    src = generate_source(K.elementwise(4, 64, (), DType.BF16, DType.F16).to_bytes())
    assert "const unsigned short *p" in src and "bf16_bits_to_f32" in src and "f32_to_f16_bits" in src
    src = generate_source(K.dynamic_rows(64).to_bytes())
    assert "const long long p0" in src


@pytest.mark.parametrize("name", sorted(kernels()))
def test_generated_source_compiles_for_gfx950(name):
    """hiprtc includes the HIP runtime header by itself; the offline compiler gets it with -include."""
    if not os.path.exists(HIPCC):
        pytest.skip("no hipcc")
    src = generate_source(kernels()[name].to_bytes())
    with tempfile.TemporaryDirectory() as d:
        path = os.path.join(d, "k.hip")
        open(path, "w").write(src)
        r = subprocess.run([HIPCC, "--offload-arch=gfx950", "-O3", "-std=c++17", "-ffp-contract=off", "-fwrapv", "-Xclang",
                            "-target-feature", "-Xclang", "-packed-fp32-ops", "--cuda-device-only", "-Werror=return-type",
                            "-include", "hip/hip_runtime.h", "-c", path, "-o", os.path.join(d, "k.o")],
                           capture_output=True, text=True, timeout=120)
        assert r.returncode == 0, r.stderr[-2000:]


def refused(kernel_or_bytes, needle):
    img = kernel_or_bytes if isinstance(kernel_or_bytes, bytes) else kernel_or_bytes.to_bytes()
    with pytest.raises(BackendError) as e:
        generate_source(img)
    assert e.value.status == ErrorStatus.KernelCompilation and needle in str(e.value), str(e.value)


def test_refusals():
    refused(b"", "header")
    refused(b"\0" * 16, "magic")
    good = K.elementwise(4, 64).to_bytes()
    refused(good[:-8], "size")
    k = ir.Kernel()
    k.raw(Opcode.WMMA)
    refused(k, "tensor-core")
    k = ir.Kernel()
    k.raw(Opcode.REDUCE)
    refused(k, "unfolded")
    k = ir.Kernel()
    k.raw(99)
    refused(k, "unknown opcode")
    k = ir.Kernel()                                   # operand used before its definition
    y = k.param(DType.F32, ParamKind.GlobalMut, 4)
    k.store(y, 1234, k.const_idx(0))
    refused(k, "not defined")
    k = ir.Kernel()                                   # store into a read-only parameter
    x = k.param(DType.F32, ParamKind.Global, 4)
    k.store(x, k.const(1.0, DType.F32), k.const_idx(0))
    refused(k, "writable")
    k = ir.Kernel()                                   # loop left open
    k.loop(k.const_idx(4))
    refused(k, "open loop")
    k = ir.Kernel()
    k.end_loop()
    refused(k, "EndLoop")
    k = ir.Kernel()                                   # loop variable used after its loop
    y = k.param(DType.I64, ParamKind.GlobalMut, 4)
    r = k.loop(k.const_idx(4))
    k.end_loop()
    k.store(y, r, k.const_idx(0))
    refused(k, "ended")
    k = ir.Kernel()                                   # 2048 threads per group
    k.local_index(0, 1024)
    k.local_index(1, 2)
    refused(k, "1024")
    k = ir.Kernel()                                   # group length computed inside the kernel
    a = k.const_idx(4)
    k.group_index(0, k.add(a, a))
    refused(k, "constant or an integer Variable")
    k = ir.Kernel()
    x = k.param(DType.F32, ParamKind.Global, 4)
    k.unary(k.load(x, k.const_idx(0)), UOp.BitNot)
    refused(k, "no meaning")
    k = ir.Kernel()
    k.storage(DType.F32, MemScope.Global, 4)
    refused(k, "local or register")
    k = ir.Kernel()
    x = k.param(DType.F32, ParamKind.Global, 4)
    k.load(x, k.const_idx(0), vlen=3)
    refused(k, "vector length")
    k = ir.Kernel()
    for _ in range(33):
        k.param(DType.F32, ParamKind.Global, 4)
    refused(k, "parameters")
    k = ir.Kernel()                                   # the same id twice
    k.const_idx(1)
    k._next = 0
    k.const_idx(2)
    refused(k, "defined twice")


def test_mutated_images_are_refused_or_compiled_never_crash():
    """The image comes from outside the library: random corruptions of valid images (opcodes, operand ids, dtypes,
    lengths, the header) must each end in source text or a KernelCompilation reason."""
    import random
    rnd = random.Random(1234)
    bases = [k.to_bytes() for k in kernels().values()]
    outcomes = {"ok": 0, "refused": 0}
    for trial in range(3000):
        img = bytearray(rnd.choice(bases))
        for _ in range(rnd.randint(1, 4)):
            kind = rnd.random()
            if len(img) < 48:
                break
            if kind < 0.6:      # one field of one op
                n_ops = (len(img) - 16) // 32
                op = rnd.randrange(max(n_ops, 1))
                off = 16 + 32 * op + rnd.choice([0, 4, 6, 8, 12, 16, 20, 24])
                val = rnd.choice([0, 1, 2, 3, 7, 16, 0xFFFF, 0xFFFFFFFF, rnd.getrandbits(32)])
                img[off:off + 2] = (val & 0xFFFF).to_bytes(2, "little")
            elif kind < 0.8:    # any byte
                img[rnd.randrange(len(img))] = rnd.getrandbits(8)
            elif kind < 0.9:    # truncation
                del img[rnd.randrange(len(img)):]
            else:               # header counts
                img[4:12] = rnd.getrandbits(64).to_bytes(8, "little")
        try:
            src = generate_source(bytes(img))
            assert "zir_kernel" in src
            outcomes["ok"] += 1
        except BackendError as e:
            assert e.status == ErrorStatus.KernelCompilation and str(e)
            outcomes["refused"] += 1
    assert outcomes["ok"] > 50 and outcomes["refused"] > 500, outcomes
