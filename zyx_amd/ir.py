"""Builder for the image of a linearized zyx kernel, the argument of `HIPDevice.compile`.

A zyx `Kernel` after linearization is a linear list of ops in SSA form (zyx/src/kernel/ops.rs:22-147); the Rust
side of the backend slot would write this image by walking `kernel.head -> next_op` (zyx/src/codegen/cuda.rs:24-37).
This module builds the same image from Python with the reference's op names, for the tests and benchmarks.
Layout (`zhip_ir_header`, `zhip_ir_op`, little endian): see include/zyx_hip.h.
"""
from __future__ import annotations

import ctypes as C
import enum

import numpy as np

from .backend import DType

NULL = 0xFFFFFFFF
MAGIC = 0x3152495A


class Opcode(enum.IntEnum):
    CONST = 0; PARAM = 1; STORAGE = 2; LOAD = 3; STORE = 4; CAST = 5; UNARY = 6; BINARY = 7; MAD = 8; STACK = 9
    DEVECTORIZE = 10; INDEX = 11; LOOP = 12; ENDLOOP = 13; IF = 14; ENDIF = 15; BARRIER = 16
    WMMA = 17; REDUCE_TILE = 18; MATMUL_TILE = 19; TRANSPOSE_TILE = 20; ASM = 21; MOVE = 22; REDUCE = 23


class ParamKind(enum.IntEnum):  # ops.rs:11-19
    Variable = 0; Global = 1; GlobalMut = 2


class MemScope(enum.IntEnum):  # kernel/mod.rs:203-212
    Global = 0; Local = 1; Register = 2; Circular = 3


class UOp(enum.IntEnum):  # ops.rs:187-213
    Neg = 0; BitNot = 1; Exp = 2; Exp2 = 3; Ln = 4; Log2 = 5; Reciprocal = 6; Sqrt = 7; Sin = 8; Cos = 9; Floor = 10
    Trunc = 11; Abs = 12


class BOp(enum.IntEnum):  # ops.rs:221-260
    Add = 0; Sub = 1; Mul = 2; Div = 3; Pow = 4; Mod = 5; Cmplt = 6; Cmpgt = 7; Cmpge = 8; Max = 9; Or = 10; And = 11
    BitXor = 12; BitOr = 13; BitAnd = 14; BitShiftLeft = 15; BitShiftRight = 16; NotEq = 17; Eq = 18


class IrHeader(C.Structure):
    """zhip_ir_header"""
    _fields_ = [("magic", C.c_uint32), ("n_ops", C.c_uint32), ("n_extra", C.c_uint32), ("reserved", C.c_uint32)]


class IrOp(C.Structure):
    """zhip_ir_op"""
    _fields_ = [("id", C.c_uint32), ("opcode", C.c_uint16), ("dtype", C.c_uint16), ("a", C.c_uint32), ("b", C.c_uint32),
                ("c", C.c_uint32), ("aux", C.c_uint32), ("imm", C.c_uint64)]


_NP = {DType.BF16: np.uint16, DType.F16: np.float16, DType.F32: np.float32, DType.F64: np.float64, DType.U8: np.uint8,
       DType.U16: np.uint16, DType.U32: np.uint32, DType.U64: np.uint64, DType.I8: np.int8, DType.I16: np.int16,
       DType.I32: np.int32, DType.I64: np.int64, DType.Bool: np.uint8}


def constant_bits(value, dtype: DType) -> int:
    """Little-endian bytes of a `Constant` (zyx/src/dtype.rs) as an integer; a bf16 constant truncates its f32 value."""
    dtype = DType(dtype)
    if dtype == DType.BF16:
        return int(np.array([value], np.float32).view(np.uint32)[0]) >> 16
    raw = np.array([value], _NP[dtype]).tobytes()
    return int.from_bytes(raw, "little")


class Kernel:
    """Ops are appended in execution order; every method returns the new op's id. `first_id` and `id_step` let a
    test use the sparse, unordered ids a real kernel has after its rewrite passes."""

    def __init__(self, first_id: int = 0, id_step: int = 1):
        self.ops: list[IrOp] = []
        self.extra: list[int] = []
        self._next, self._step = first_id, id_step

    def _push(self, opcode, dtype=0, a=NULL, b=NULL, c=NULL, aux=0, imm=0) -> int:
        op = IrOp(self._next, int(opcode), int(dtype), a, b, c, int(aux), int(imm) & 0xFFFFFFFFFFFFFFFF)
        self.ops.append(op)
        self._next += self._step
        return op.id

    # leaves
    def const(self, value, dtype: DType) -> int:
        return self._push(Opcode.CONST, dtype, imm=constant_bits(value, dtype))

    def const_idx(self, value: int) -> int:
        """Index constants are I64 (IDX_T, kernel/mod.rs:131)."""
        return self.const(value, DType.I64)

    def param(self, dtype: DType, kind: ParamKind, elems: int = 0) -> int:
        return self._push(Opcode.PARAM, dtype, aux=kind, imm=elems)

    def storage(self, dtype: DType, scope: MemScope, length: int) -> int:
        return self._push(Opcode.STORAGE, dtype, aux=scope, imm=length)

    # memory
    def load(self, src: int, index: int, vlen: int = 0) -> int:
        return self._push(Opcode.LOAD, a=src, b=index, aux=vlen)

    def store(self, dst: int, src: int, index: int, vlen: int = 0) -> int:
        return self._push(Opcode.STORE, a=dst, b=src, c=index, aux=vlen)

    # values
    def cast(self, x: int, dtype: DType) -> int:
        return self._push(Opcode.CAST, dtype, a=x)

    def unary(self, x: int, uop: UOp) -> int:
        return self._push(Opcode.UNARY, a=x, aux=uop)

    def binary(self, x: int, y: int, bop: BOp) -> int:
        return self._push(Opcode.BINARY, a=x, b=y, aux=bop)

    def mad(self, x: int, y: int, z: int) -> int:
        return self._push(Opcode.MAD, a=x, b=y, c=z)

    def stack(self, ops) -> int:
        first = len(self.extra)
        self.extra.extend(int(o) for o in ops)
        return self._push(Opcode.STACK, a=first, b=len(ops))

    def devectorize(self, vec: int, lane: int) -> int:
        return self._push(Opcode.DEVECTORIZE, a=vec, aux=lane)

    # shorthands used by the linearizer's own helpers (kernel/linearize.rs: self.mul, self.mad, self.cmplt, ...)
    def add(self, x, y): return self.binary(x, y, BOp.Add)
    def sub(self, x, y): return self.binary(x, y, BOp.Sub)
    def mul(self, x, y): return self.binary(x, y, BOp.Mul)
    def div(self, x, y): return self.binary(x, y, BOp.Div)
    def max(self, x, y): return self.binary(x, y, BOp.Max)
    def cmplt(self, x, y): return self.binary(x, y, BOp.Cmplt)
    def cmpge(self, x, y): return self.binary(x, y, BOp.Cmpge)
    def and_(self, x, y): return self.binary(x, y, BOp.And)

    # indices and control flow
    def group_index(self, axis: int, len_op: int) -> int:
        """Op::Index { axis, kind: IdxKind::Group(len_op) }: len_op is a Const or a Variable Param."""
        return self._push(Opcode.INDEX, a=len_op, aux=axis)

    def local_index(self, axis: int, length: int) -> int:
        """Op::Index { axis, kind: IdxKind::Local(length) }"""
        return self._push(Opcode.INDEX, aux=axis | (1 << 8), imm=length)

    def loop(self, len_op: int) -> int:
        return self._push(Opcode.LOOP, a=len_op)

    def end_loop(self) -> int:
        return self._push(Opcode.ENDLOOP)

    def if_(self, condition: int) -> int:
        return self._push(Opcode.IF, a=condition)

    def end_if(self) -> int:
        return self._push(Opcode.ENDIF)

    def barrier(self) -> int:
        return self._push(Opcode.BARRIER)

    def raw(self, opcode: int, **fields) -> int:
        """Any op, including the ones the backend refuses (tests of the refusal)."""
        return self._push(opcode, **fields)

    def to_bytes(self) -> bytes:
        head = IrHeader(MAGIC, len(self.ops), len(self.extra), 0)
        ops = (IrOp * len(self.ops))(*self.ops)
        return bytes(head) + bytes(ops) + np.asarray(self.extra, np.uint32).tobytes()
