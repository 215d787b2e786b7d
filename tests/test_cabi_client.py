"""include/zyx_hip.h used from plain C (tests/cabi/client.c, built with gcc -std=c99): the header is valid C, the
struct layouts a foreign binding would mirror equal the ones the Python mirror uses, and a kernel launch driven
from C alone gives the right answer."""
import ctypes
import os
import subprocess

import pytest

from zyx_amd import backend

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


@pytest.fixture(scope="module")
def client(tmp_path_factory):
    exe = str(tmp_path_factory.mktemp("cabi") / "client")
    lib_dir = os.path.join(ROOT, "zyx_amd")
    cmd = ["gcc", "-std=c99", "-Wall", "-Wextra", "-Werror", "-I", os.path.join(ROOT, "include"), "-o", exe,
           os.path.join(ROOT, "tests", "cabi", "client.c"), "-L", lib_dir, "-lzyx_hip", "-lm", f"-Wl,-rpath,{lib_dir}"]
    subprocess.run(cmd, check=True, capture_output=True, text=True)
    return exe


def test_header_is_c_and_layouts_match_the_python_mirror(client):
    out = subprocess.run([client, "layout"], check=True, capture_output=True, text=True).stdout.split("\n")
    kd = out[0].split()
    assert kd[0] == "zhip_kernel_desc" and int(kd[1]) == ctypes.sizeof(backend.KernelDesc)
    offsets = {kd[i]: int(kd[i + 1]) for i in range(2, len(kd), 2)}
    assert offsets == {f[0]: getattr(backend.KernelDesc, f[0]).offset for f in backend.KernelDesc._fields_}
    cfg = out[1].split()
    assert int(cfg[1]) == ctypes.sizeof(backend._Config)
    assert {cfg[i]: int(cfg[i + 1]) for i in range(2, len(cfg), 2)} == {f[0]: getattr(backend._Config, f[0]).offset for f in backend._Config._fields_}
    assert int(out[2].split()[1]) == ctypes.sizeof(backend._DeviceInfo)
    from zyx_amd import kernels as K
    assert [int(v) for v in out[3].split()[1:]] == [K.K_SOFTMAX_ROWS, K.K_ELEMENTWISE, K.K_REDUCE, K.K_GEMM, K.K_NORM_ROWS, K.K_CROSS_ENTROPY,
                                                    K.K_CONV2D, K.K_MAX_POOL2D, K.K_INDEX, K.K_ATTENTION, K.K_ATTENTION_BWD, K.K_NORM_ROWS_BWD]
    from zyx_amd import ir
    op = out[4].split()
    assert op[0] == "zhip_ir_op" and int(op[1]) == ctypes.sizeof(ir.IrOp) == 32
    assert {op[i]: int(op[i + 1]) for i in range(2, len(op), 2)} == {f[0]: getattr(ir.IrOp, f[0]).offset for f in ir.IrOp._fields_}
    assert [int(v) for v in out[5].split()[1:]] == [ctypes.sizeof(ir.IrHeader), ir.MAGIC, ir.Opcode.BARRIER, ir.Opcode.REDUCE, ir.UOp.Abs,
                                                    ir.BOp.Eq, ir.ParamKind.GlobalMut, ir.MemScope.Register]
    ce = out[6].split()
    assert ce[0] == "zhip_ceilings" and int(ce[1]) == ctypes.sizeof(backend._Ceilings) == 36
    assert {ce[i]: int(ce[i + 1]) for i in range(2, len(ce), 2)} == {n: getattr(backend._Ceilings, n).offset for n in ce[2::2]}
    rg = out[7].split()
    assert rg[:2] == ["zhip_rng", "32"] and [int(v) for v in rg[3:7]] == [0, 1, 2, 3]
    assert int(rg[8]) == K.K_ARGMAX and int(rg[10]) == K.CE_DENSE
    from zyx_amd.rng import Rng
    assert int(out[8].split()[1]) == Rng(42069).next_u64()   # the generator driven from C and through the Python mirror
    assert out[9].split()[0] == "cache" and len(out[9].split()) == 4


@pytest.mark.gpu
def test_softmax_launch_driven_from_c(client):
    r = subprocess.run([client, "softmax"], capture_output=True, text=True, timeout=120)
    assert r.returncode == 0 and "ok" in r.stdout, r.stdout + r.stderr
