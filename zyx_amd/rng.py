"""zyx's host-side random tensors (zyx/src/rng.rs, zyx/src/tensor/mod.rs:516-660) through the backend library's
`zhip_rng_*` calls: the same seeded values the reference draws, as numpy arrays. Needs no GPU."""
from __future__ import annotations

import ctypes as C

import numpy as np

from .backend import BackendError, DType, ErrorStatus, load_library

_RAND, _UNIFORM, _RANDN, _RANDINT = 0, 1, 2, 3
_NP = {DType.F32: np.float32, DType.U8: np.uint8, DType.I8: np.int8, DType.U16: np.uint16, DType.I16: np.int16,
       DType.U32: np.uint32, DType.I32: np.int32, DType.U64: np.uint64, DType.I64: np.int64}


class Rng:
    """`Rng::seed_from_u64` (rng.rs:15-57); the runtime's default seed is 42069 (zyx/src/runtime.rs:178) and
    `Tensor::manual_seed` re-seeds it."""

    def __init__(self, seed: int = 42069):
        self._lib = load_library()
        self._lib.zhip_rng_next_u64.restype = C.c_uint64
        self._s = (C.c_uint64 * 4)()
        self._lib.zhip_rng_seed(self._s, C.c_uint64(seed))

    def next_u64(self) -> int:
        return int(self._lib.zhip_rng_next_u64(self._s))

    def _fill(self, kind: int, dtype: DType, shape, lo: float = 0.0, hi: float = 0.0) -> np.ndarray:
        out = np.empty(shape, _NP[DType(dtype)])
        rc = self._lib.zhip_rng_fill(self._s, C.c_int32(kind), C.c_int32(int(dtype)), C.c_void_p(out.ctypes.data),
                                     C.c_uint64(out.size), C.c_double(lo), C.c_double(hi))
        if rc != 0:
            raise BackendError(ErrorStatus(rc), f"zhip_rng_fill: kind {kind} does not produce dtype {DType(dtype).name}")
        return out

    def rand(self, shape, dtype: DType = DType.F32) -> np.ndarray:
        """Tensor::rand: floats in [0, 1], integers over their whole range."""
        return self._fill(_RAND, dtype, shape)

    def uniform(self, shape, lo: float, hi: float) -> np.ndarray:
        """Tensor::uniform(shape, lo..hi) as f32."""
        return self._fill(_UNIFORM, DType.F32, shape, lo, hi)

    def randn(self, shape, scale: float = 1.0) -> np.ndarray:
        """Tensor::randn(shape, F32) * scale."""
        return self._fill(_RANDN, DType.F32, shape, 0.0, scale)

    def randint(self, shape, lo: int, hi: int, dtype: DType = DType.I32) -> np.ndarray:
        """Tensor::randint(shape, lo..hi)."""
        return self._fill(_RANDINT, dtype, shape, lo, hi)
