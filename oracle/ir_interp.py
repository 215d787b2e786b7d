"""TEST INFRASTRUCTURE, not product code: a CPU interpreter for the image of a linearized zyx kernel (layout in
include/zyx_hip.h), the checker for kernels the HIP backend generates from such an image.

It restates the meaning the reference's C backend gives every op (zyx/src/codegen/c.rs:74-395 statement by
statement, 583-612 binary ops, 614-629 register types, 456-497 the 16-bit float conversions): f32 registers for
f32 / f16 / bf16, widening loads and truncating stores for the 16-bit floats, math functions evaluated through
`double` and narrowed on assignment, `(int)x % (int)y`, comparisons giving 0 / 1. The C backend runs a kernel as
nested loops over the group indices (c.rs:74-95); local indices and local storage exist only on the GPU backends
(cuda.rs:66-70, 286-311), where each group runs its threads side by side. Here every thread of the whole grid
advances one op at a time (numpy arrays over threads), which serialises nothing the C loop nest would order and
makes a barrier a no-op; stores and register updates of threads switched off by a loop bound or an `If` are masked.
Where C leaves a result open (integer division or remainder by zero, shift counts beyond the width, signed
overflow) it yields 0 / the count modulo the width / the wrapped value, the choices the generated HIP code makes.

Checked in tests/test_ir_oracle.py against: the reference's golden matmul and softmax values computed through
kernels in this format, the C oracle's serial-order matmul, softmax and elementwise chains (bit for bit), exhaustive
8-bit tables of the integer ops computed with Python integers, and closed forms.
"""
from __future__ import annotations

import struct

import numpy as np

BF16, F16, F32, F64, U8, U16, U32, U64, I8, I16, I32, I64, BOOL = range(13)
_REG = {BF16: np.float32, F16: np.float32, F32: np.float32, F64: np.float64, U8: np.uint8, U16: np.uint16, U32: np.uint32,
        U64: np.uint64, I8: np.int8, I16: np.int16, I32: np.int32, I64: np.int64, BOOL: np.uint8}
_BITS = {BF16: 16, F16: 16, F32: 32, F64: 64, U8: 8, U16: 16, U32: 32, U64: 64, I8: 8, I16: 16, I32: 32, I64: 64, BOOL: 8}
_FLOATS = (BF16, F16, F32, F64)

(CONST, PARAM, STORAGE, LOAD, STORE, CAST, UNARY, BINARY, MAD, STACK, DEVECTORIZE, INDEX, LOOP, ENDLOOP, IF, ENDIF,
 BARRIER) = range(17)
VARIABLE, GLOBAL, GLOBAL_MUT = range(3)
LOCAL, REGISTER = 1, 2
MAGIC = 0x3152495A


class IrError(ValueError):
    pass


def parse(image: bytes):
    if len(image) < 16:
        raise IrError("image shorter than its header")
    magic, n_ops, n_extra, _ = struct.unpack_from("<4I", image, 0)
    if magic != MAGIC or len(image) != 16 + 32 * n_ops + 4 * n_extra:
        raise IrError("bad magic or size")
    ops = [struct.unpack_from("<IHH4IQ", image, 16 + 32 * i) for i in range(n_ops)]  # id opcode dtype a b c aux imm
    extra = list(struct.unpack_from(f"<{n_extra}I", image, 16 + 32 * n_ops))
    return ops, extra


# ---- 16-bit float storage (c.rs:456-497) ----------------------------------------------------------------------

def bf16_bits_to_f32(h):
    return (np.asarray(h, np.uint16).astype(np.uint32) << 16).view(np.float32)


def f32_to_bf16_bits(v):
    return (np.ascontiguousarray(v, np.float32).view(np.uint32) >> 16).astype(np.uint16)


def f16_bits_to_f32(h):
    return np.asarray(h, np.uint16).view(np.float16).astype(np.float32)


def f32_to_f16_bits(v):
    f = np.ascontiguousarray(v, np.float32).view(np.uint32).astype(np.int64)
    sign, ex, man = (f >> 16) & 0x8000, (f >> 23) & 0xFF, f & 0x7FFFFF
    ne = ex - 127 + 15
    out = np.where(ex == 0, sign,
          np.where(ex == 255, sign | 0x7C00 | (man >> 13),
          np.where(ne >= 31, sign | 0x7C00,
          np.where(ne <= 0, sign, sign | (np.maximum(ne, 0) << 10) | (man >> 13)))))
    return out.astype(np.uint16)


# ---- op semantics ------------------------------------------------------------------------------------------------

def _through_double(fn, x, dt):
    with np.errstate(all="ignore"):
        return fn(x.astype(np.float64)).astype(_REG[dt])


def _c_cast(x, dt):
    """`(T)x` of C: float -> integer truncates toward zero, integer -> narrower integer wraps."""
    tgt = _REG[dt]
    if x.dtype.kind == "f" and np.dtype(tgt).kind in "iu":
        with np.errstate(all="ignore"):
            t = np.trunc(x)
            wide = np.where(np.isfinite(t), t, 0).astype(np.int64 if np.dtype(tgt).kind == "i" or dt != U64 else np.uint64)
        return wide.astype(tgt)
    with np.errstate(all="ignore"):
        return x.astype(tgt)


def unary(uop, x, dt):
    reg = _REG[dt]
    with np.errstate(all="ignore"):
        if dt in _FLOATS:
            one = reg(1.0)
            table = {0: lambda: -x, 2: lambda: _through_double(np.exp, x, dt), 3: lambda: _through_double(np.exp2, x, dt),
                     4: lambda: _through_double(np.log, x, dt), 5: lambda: _through_double(np.log2, x, dt),
                     6: lambda: (one / x).astype(reg), 7: lambda: _through_double(np.sqrt, x, dt),
                     8: lambda: _through_double(np.sin, x, dt), 9: lambda: _through_double(np.cos, x, dt),
                     10: lambda: np.floor(x), 11: lambda: np.trunc(x), 12: lambda: np.abs(x)}
        else:
            table = {0: lambda: (0 - x).astype(reg), 1: lambda: (~x).astype(reg), 12: lambda: np.abs(x).astype(reg) if np.dtype(reg).kind == "i" else x,
                     6: lambda: _int_div(np.ones_like(x), x), 10: lambda: x, 11: lambda: x,
                     2: lambda: _c_cast(np.exp(x.astype(np.float64)), dt), 3: lambda: _c_cast(np.exp2(x.astype(np.float64)), dt),
                     4: lambda: _c_cast(np.log(x.astype(np.float64)), dt), 5: lambda: _c_cast(np.log2(x.astype(np.float64)), dt),
                     7: lambda: _c_cast(np.sqrt(x.astype(np.float64)), dt), 8: lambda: _c_cast(np.sin(x.astype(np.float64)), dt),
                     9: lambda: _c_cast(np.cos(x.astype(np.float64)), dt)}
        if uop not in table:
            raise IrError(f"unary op {uop} has no meaning for dtype {dt}")
        return np.asarray(table[uop]()).astype(reg)


def _int_div(x, y):
    """C's truncating division; 0 for a zero divisor, the wrapped negation for -1."""
    with np.errstate(all="ignore"):
        safe = np.where(y == 0, 1, y)
        if x.dtype.kind == "i":
            safe = np.where(safe == -1, 1, safe)
            q = (np.abs(x.astype(np.int64)).astype(np.uint64) // np.abs(safe.astype(np.int64)).astype(np.uint64)).astype(np.int64)
            q = np.where((x < 0) != (safe < 0), -q, q)
            q = np.where(y == -1, (0 - x.astype(np.int64)), q)
        else:
            q = x // safe
        return np.where(y == 0, 0, q).astype(x.dtype)


def _c_mod(x, y):
    """`(int)x % (int)y` (c.rs:598): 32-bit operands, remainder with the dividend's sign; 0 for divisors 0 and -1."""
    xi, yi = _c_cast(x, I32).astype(np.int64), _c_cast(y, I32).astype(np.int64)
    safe = np.where((yi == 0) | (yi == -1), 1, yi)
    r = np.fmod(xi, safe)
    return np.where((yi == 0) | (yi == -1), 0, r)


def binary(bop, x, y, dt):
    """dt is x's dtype; the result takes it unless the op yields a Bool (kernel/mod.rs:308-316)."""
    reg = _REG[dt]
    with np.errstate(all="ignore"):
        if bop in (6, 7, 8, 17, 18):
            return {6: x < y, 7: x > y, 8: x >= y, 17: x != y, 18: x == y}[bop].astype(np.uint8)
        if bop == 10:
            return ((x != 0) | (y != 0)).astype(np.uint8)
        if bop == 11:
            return ((x != 0) & (y != 0)).astype(np.uint8)
        if bop == 5:
            return _c_mod(x, y).astype(reg)
        if dt in _FLOATS:
            if bop == 0: r = x + y
            elif bop == 1: r = x - y
            elif bop == 2: r = x * y
            elif bop == 3: r = x / y
            elif bop == 4: r = np.power(x.astype(np.float64), np.asarray(y).astype(np.float64))
            elif bop == 9: r = np.fmax(x, y)
            else: raise IrError(f"binary op {bop} has no meaning for dtype {dt}")
            return np.asarray(r).astype(reg)
        y = np.asarray(y)
        if y.dtype.kind in "iub" and y.dtype != x.dtype:
            y = y.astype(x.dtype)
        mask = _BITS[dt] - 1
        if bop == 0: r = x + y
        elif bop == 1: r = x - y
        elif bop == 2: r = x * y
        elif bop == 3: r = _int_div(x, y.astype(x.dtype))
        elif bop == 4: r = _c_cast(np.power(x.astype(np.float64), y.astype(np.float64)), dt)
        elif bop == 9: r = np.maximum(x, y)
        elif bop == 12: r = x ^ y
        elif bop == 13: r = x | y
        elif bop == 14: r = x & y
        elif bop == 15: r = x << (y.astype(np.int64) & mask).astype(x.dtype)
        elif bop == 16: r = x >> (y.astype(np.int64) & mask).astype(x.dtype)
        else: raise IrError(f"unknown binary op {bop}")
        return np.asarray(r).astype(reg)


def mad(x, y, z, dt):
    """x * y + z with one rounding for f32 (the product of two f32 is exact in double), plain for the rest."""
    reg = _REG[dt]
    with np.errstate(all="ignore"):
        if reg == np.float32:
            return (x.astype(np.float64) * np.asarray(y).astype(np.float64) + np.asarray(z).astype(np.float64)).astype(np.float32)
        return np.asarray(x * y + z).astype(reg)


# ---- execution ---------------------------------------------------------------------------------------------------

def run(image: bytes, args) -> None:
    """Runs the kernel. `args`: one entry per PARAM op in order -- a Python / numpy scalar for a Variable, a numpy
    array in storage format for a buffer (uint16 bit patterns for bf16 and f16). GlobalMut arrays are written in place."""
    ops, extra = parse(image)
    params = [o for o in ops if o[1] == PARAM]
    if len(params) != len(args):
        raise IrError(f"kernel takes {len(params)} arguments, got {len(args)}")
    arg_of = {o[0]: a for o, a in zip(params, args)}
    kind_of = {o[0]: o[6] for o in params}

    # grid and block (backend/mod.rs:74-98)
    consts = {o[0]: o for o in ops if o[1] == CONST}
    grid, block = [1, 1, 1], [1, 1, 1]
    for o in ops:
        if o[1] == INDEX:
            axis, kind = o[6] & 0xFF, o[6] >> 8
            if kind == 0:
                ln = o[3]
                if ln in consts:
                    grid[axis] = _const_value(consts[ln]).item()
                else:
                    grid[axis] = int(arg_of[ln])
            elif kind == 1:
                block[axis] = int(o[7])
            else:
                raise IrError("warp index")
    n_groups, n_local = int(np.prod(grid)), int(np.prod(block))
    T = n_groups * n_local
    if T == 0:
        return
    t = np.arange(T, dtype=np.int64)
    grp, loc = t // n_local, t % n_local
    gidx = [grp % grid[0], (grp // grid[0]) % grid[1], grp // (grid[0] * grid[1])]
    lidx = [loc % block[0], (loc // block[0]) % block[1], loc // (block[0] * block[1])]

    # matching EndLoop / EndIf of every Loop / If
    match, stack = {}, []
    for pc, o in enumerate(ops):
        if o[1] in (LOOP, IF):
            stack.append(pc)
        elif o[1] in (ENDLOOP, ENDIF):
            match[stack.pop()] = pc
    vals: dict[int, np.ndarray] = {}
    dtypes: dict[int, int] = {}
    storage: dict[int, tuple] = {}
    mask = np.ones(T, bool)
    frames = []  # ("L", pc, len array, iteration, parent mask) | ("I", parent mask)

    def assign(op_id, new, dt):
        new = np.asarray(new)
        if new.shape[0] != T:
            new = np.broadcast_to(new, (T,) + new.shape[1:]).copy()
        old = vals.get(op_id)
        if old is not None and old.shape == new.shape and not mask.all():
            m = mask if new.ndim == 1 else mask[:, None]
            new = np.where(m, new, old)
        vals[op_id], dtypes[op_id] = new, dt

    def lanes(v, n):  # scalar operand of a vector op is broadcast
        return v if (v.ndim == 2 or n == 0) else np.repeat(v[:, None], n, axis=1)

    pc = 0
    while pc < len(ops):
        op_id, opc, dt, a, b, c, aux, imm = ops[pc]
        if opc == CONST:
            assign(op_id, np.full(T, _const_value(ops[pc])), dt)
        elif opc == PARAM:
            dtypes[op_id] = dt
            if aux == VARIABLE:  # passed by value; a bf16 / f16 scalar travels as its 16 bits
                raw = arg_of[op_id]
                if dt == BF16: raw = bf16_bits_to_f32(f32_to_bf16_bits(np.float32(raw)))
                elif dt == F16: raw = f16_bits_to_f32(f32_to_f16_bits(np.float32(raw)))
                vals[op_id] = np.full(T, raw, _REG[dt])
        elif opc == STORAGE:
            dtypes[op_id] = dt
            storage[op_id] = (aux, np.zeros((n_groups if aux == LOCAL else T, imm), _REG[dt]))
        elif opc == LOAD:
            sdt = dtypes[a]
            if kind_of.get(a) == VARIABLE:
                assign(op_id, vals[a], sdt)  # Variable parameter: its value, the index is not used (c.rs:125-131)
            else:
                idx = np.where(mask, vals[b], 0)
                n = aux if aux else 1
                off = idx[:, None] + np.arange(n, dtype=np.int64)[None, :]
                if (off < 0).any():
                    raise IndexError(f"op {pc}: negative load index")
                if a in storage:
                    scope, mem = storage[a]
                    row = grp if scope == LOCAL else t
                    got = mem[row[:, None], off]
                else:
                    flat = arg_of[a].reshape(-1)
                    got = flat[off]
                    if sdt == BF16: got = bf16_bits_to_f32(got)
                    elif sdt == F16: got = f16_bits_to_f32(got.view(np.uint16) if got.dtype == np.float16 else got)
                    else: got = got.astype(_REG[sdt])
                assign(op_id, got if aux else got[:, 0], sdt)
        elif opc == STORE:
            ddt = dtypes[a]
            n = aux if aux else 1
            src = lanes(vals[b], n).reshape(T, n)
            off = vals[c][:, None] + np.arange(n, dtype=np.int64)[None, :]
            m = mask
            if (off[m] < 0).any():
                raise IndexError(f"op {pc}: negative store index")
            if a in storage:
                scope, mem = storage[a]
                row = (grp if scope == LOCAL else t)[:, None] + np.zeros_like(off)
                mem[row[m], off[m]] = _c_cast(src[m], ddt) if src.dtype != mem.dtype else src[m]
            else:
                flat = arg_of[a].reshape(-1)
                if ddt == BF16: out = f32_to_bf16_bits(src[m].astype(np.float32))
                elif ddt == F16:
                    out = f32_to_f16_bits(src[m].astype(np.float32))
                    if flat.dtype == np.float16: out = out.view(np.float16)
                else: out = _c_cast(src[m], ddt)
                flat[off[m]] = out
        elif opc == CAST:
            x = vals[a]
            assign(op_id, x.astype(np.float32) if dt in (BF16, F16) else _c_cast(x, dt), dt)
        elif opc == UNARY:
            assign(op_id, unary(aux, vals[a], dtypes[a]), dtypes[a])
        elif opc == BINARY:
            x, y = vals[a], vals[b]
            n = max(x.shape[1] if x.ndim == 2 else 0, y.shape[1] if y.ndim == 2 else 0)
            r = binary(aux, lanes(x, n), lanes(y, n), dtypes[a])
            assign(op_id, r, BOOL if aux in (6, 7, 8, 10, 11, 17, 18) else dtypes[a])
        elif opc == MAD:
            x, y, z = vals[a], vals[b], vals[c]
            n = max(v.shape[1] if v.ndim == 2 else 0 for v in (x, y, z))
            assign(op_id, mad(lanes(x, n), lanes(y, n), lanes(z, n), dtypes[a]), dtypes[a])
        elif opc == STACK:
            members = extra[a:a + b]
            d0 = dtypes[members[0]]
            assign(op_id, np.stack([vals[m].astype(_REG[d0]) for m in members], axis=1), d0)
        elif opc == DEVECTORIZE:
            assign(op_id, vals[a][:, aux], dtypes[a])
        elif opc == INDEX:
            axis, kind = aux & 0xFF, aux >> 8
            assign(op_id, (gidx if kind == 0 else lidx)[axis].astype(np.int64), I64)
        elif opc == LOOP:
            ln = vals[a].astype(np.int64)
            parent = mask
            mask = parent & (0 < ln)
            if not mask.any():
                mask = parent
                pc = match[pc]
            else:
                frames.append(["L", pc, ln, 0, parent])
                vals[op_id], dtypes[op_id] = np.zeros(T, np.int64), I64
        elif opc == ENDLOOP:
            fr = frames[-1]
            fr[3] += 1
            nxt = fr[4] & (fr[3] < fr[2])
            if nxt.any():
                mask = nxt
                loop_id = ops[fr[1]][0]
                vals[loop_id] = np.full(T, fr[3], np.int64)
                pc = fr[1]
            else:
                mask = fr[4]
                frames.pop()
        elif opc == IF:
            frames.append(["I", mask])
            mask = mask & (vals[a] != 0)
        elif opc == ENDIF:
            mask = frames.pop()[1]
        elif opc == BARRIER:
            pass
        else:
            raise IrError(f"op {pc}: opcode {opc} has no meaning here")
        pc += 1


def _const_value(o):
    dt, imm = o[2], o[7]
    raw = struct.pack("<Q", imm)
    if dt == BF16:
        return bf16_bits_to_f32(np.uint16(imm & 0xFFFF))
    if dt == F16:
        return f16_bits_to_f32(np.uint16(imm & 0xFFFF))
    return np.frombuffer(raw[:_BITS[dt] // 8], _REG[dt] if dt != BOOL else np.uint8)[0]
