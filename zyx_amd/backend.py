"""ctypes binding of ``libzyx_hip.so`` shaped like the reference's HIP backend slot.

Names, argument meaning and error behaviour follow `HIPMemoryPool` / `HIPDevice`
(zyx/src/backend/hip.rs:340-459, 487-728) and the dispatching enums in
zyx/src/backend/mod.rs:556-1028. A Rust shim would bind the same C symbols through
`libloading` exactly as this file does through ctypes.
"""
from __future__ import annotations

import ctypes as C
import enum
import os
from dataclasses import dataclass, field
from typing import Optional, Sequence

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB_NAME = "libzyx_hip.so"


def library_path() -> str:
    return os.path.join(_HERE, _LIB_NAME)


class ErrorStatus(enum.IntEnum):
    """zyx/src/error.rs:125-153"""
    DyLibNotFound = 1
    Initialization = 2
    Deinitialization = 3
    DeviceEnumeration = 4
    DeviceQuery = 5
    MemoryAllocation = 6
    MemoryDeallocation = 7
    MemoryCopyH2P = 8
    MemoryCopyP2H = 9
    IncorrectKernelArg = 10
    KernelCompilation = 11
    KernelLaunch = 12
    KernelSync = 13


class BackendError(Exception):
    """zyx/src/error.rs:107-123: `{status:?}: {context}`"""

    def __init__(self, status: ErrorStatus, context: str):
        super().__init__(f"{status.name}: {context}")
        self.status = status
        self.context = context


class DType(enum.IntEnum):
    """zyx/src/dtype.rs:20-47"""
    BF16 = 0
    F16 = 1
    F32 = 2
    F64 = 3
    U8 = 4
    U16 = 5
    U32 = 6
    U64 = 7
    I8 = 8
    I16 = 9
    I32 = 10
    I64 = 11
    Bool = 12

    def byte_size(self) -> int:
        return {0: 2, 1: 2, 2: 4, 3: 8, 4: 1, 5: 2, 6: 4, 7: 8, 8: 1, 9: 2, 10: 4, 11: 8, 12: 1}[int(self)]


class _Config(C.Structure):
    _fields_ = [("device_id", C.c_int32), ("debug", C.c_uint32), ("cache_bytes", C.c_uint64)]


class _DeviceInfo(C.Structure):
    _fields_ = [("compute", C.c_uint64), ("max_global_work_dims", C.c_uint64 * 3), ("max_local_threads", C.c_uint32),
                ("max_local_work_dims", C.c_uint32 * 3), ("preferred_vector_size", C.c_uint32),
                ("local_mem_size", C.c_uint64), ("max_register_bytes", C.c_uint64), ("tensor_cores", C.c_uint32),
                ("warp_size", C.c_uint32), ("dtype_capability", C.c_uint32 * 13), ("has_native_exp2", C.c_uint32),
                ("n_supported_vec_lens", C.c_uint32), ("supported_vec_lens", C.c_uint32 * 4),
                ("total_bytes", C.c_uint64), ("compute_units", C.c_uint32), ("clock_khz", C.c_uint32),
                ("name", C.c_char * 64), ("arch", C.c_char * 32)]


class KernelDesc(C.Structure):
    """zhip_kernel_desc"""
    _fields_ = [("kind", C.c_int32), ("dtype", C.c_int32), ("out_dtype", C.c_int32), ("flags", C.c_int32),
                ("dims", C.c_int64 * 8), ("fparams", C.c_float * 8), ("iparams", C.c_int32 * 24)]


class _Ceilings(C.Structure):
    _fields_ = [(n, C.c_float) for n in ("memcpy_d2d_GBps", "copy_kernel_GBps", "read_kernel_GBps",
                                         "mfma_bf16_const_TFLOPs", "mfma_bf16_const_MHz", "mfma_bf16_const_launch_us",
                                         "mfma_bf16_random_TFLOPs", "mfma_bf16_random_MHz", "mfma_bf16_random_launch_us")]


@dataclass
class DeviceInfo:
    """zyx/src/backend/mod.rs:506-531"""
    compute: int
    max_global_work_dims: list
    max_local_threads: int
    max_local_work_dims: list
    preferred_vector_size: int
    local_mem_size: int
    max_register_bytes: int
    tensor_cores: bool
    warp_size: int
    dtype_capability: list
    has_native_exp2: bool
    supported_vec_lens: list
    total_bytes: int = 0
    compute_units: int = 0
    clock_khz: int = 0
    name: str = ""
    arch: str = ""


@dataclass
class HIPConfig:
    """zyx/src/backend/hip.rs:27-32: `device_ids: None` = all devices, `Some([])` = backend disabled."""
    device_ids: Optional[list] = None
    cache_bytes: int = 0


@dataclass(frozen=True)
class Event:
    """Event::HIP (zyx/src/backend/mod.rs:1030-1040). Owned by the caller, consumed once."""
    handle: int = 0


_lib = None

_EXPORTS = ["zhip_device_count", "zhip_init", "zhip_deinit", "zhip_last_error", "zhip_get_device_info",
            "zhip_free_bytes", "zhip_free_compute", "zhip_alloc", "zhip_free", "zhip_store_variable",
            "zhip_get_variable", "zhip_h2d", "zhip_d2h", "zhip_d2d", "zhip_sync_events", "zhip_release_events",
            "zhip_buffer_ptr", "zhip_register_kernel", "zhip_compile_ir", "zhip_compile_cache_stats", "zhip_ir_generate", "zhip_program_source", "zhip_launch",
            "zhip_release_program",
            "zhip_rng_seed", "zhip_rng_next_u64", "zhip_rng_fill", "zhip_reduce_static", "zhip_measure_ceilings", "zhip_time_kernel", "zhip_profile_kernel", "zhip_plan_create", "zhip_plan_launch", "zhip_plan_destroy"]


def load_library() -> C.CDLL:
    """dlopen of the backend library; `DyLibNotFound` when it has not been built
    (the status the reference returns when libamdhip64.so is missing, hip.rs:137-148)."""
    global _lib
    if _lib is not None:
        return _lib
    path = library_path()
    if not os.path.exists(path):
        raise BackendError(ErrorStatus.DyLibNotFound,
                           f"{path} not found; build it with `python -c 'import __graft_entry__ as g; g.build()'`")
    try:
        lib = C.CDLL(path)
    except OSError as e:
        raise BackendError(ErrorStatus.DyLibNotFound, f"cannot load {path}: {e}") from e
    lib.zhip_last_error.restype = C.c_char_p
    lib.zhip_last_error.argtypes = [C.c_void_p]
    lib.zhip_free_bytes.restype = C.c_uint64
    lib.zhip_free_bytes.argtypes = [C.c_void_p]
    lib.zhip_free_compute.restype = C.c_uint64
    lib.zhip_free_compute.argtypes = [C.c_void_p]
    _lib = lib
    return lib


def _host_span(obj, writable: bool):
    """(address, byte count) of a C-contiguous ndarray or bytes-like object; no copy is made."""
    a = obj if isinstance(obj, np.ndarray) else np.frombuffer(obj, np.uint8)
    if not a.flags["C_CONTIGUOUS"]:
        raise ValueError("host buffer must be C-contiguous")
    if writable and not a.flags["WRITEABLE"]:
        raise ValueError("destination buffer is read-only")
    return (C.c_void_p(a.ctypes.data) if a.nbytes else None), a.nbytes


def _events_array(events: Sequence[Event]):
    n = len(events)
    arr = (C.c_uint64 * max(n, 1))(*[e.handle for e in events])
    return arr, C.c_size_t(n)


class _Context:
    """One `zhip_ctx`: shared by the pool and the device the reference creates per GPU."""

    def __init__(self, device_id: int, debug: int, cache_bytes: int):
        self.lib = load_library()
        self.ptr = C.c_void_p()
        cfg = _Config(device_id, debug, cache_bytes)
        rc = self.lib.zhip_init(C.byref(cfg), C.byref(self.ptr))
        if rc != 0:
            raise BackendError(ErrorStatus(rc), self.lib.zhip_last_error(None).decode())
        self.device_id = device_id

    def check(self, rc: int):
        if rc != 0:
            raise BackendError(ErrorStatus(rc), self.lib.zhip_last_error(self.ptr).decode())

    def close(self):
        if self.ptr:
            self.lib.zhip_deinit(self.ptr)
            self.ptr = C.c_void_p()


class HIPMemoryPool:
    """zyx/src/backend/hip.rs:35-49, 340-465"""

    def __init__(self, ctx: _Context):
        self._ctx = ctx

    def deinitialize(self):
        self._ctx.close()

    def free_bytes(self) -> int:
        return int(self._ctx.lib.zhip_free_bytes(self._ctx.ptr))

    def allocate(self, bytes_: int):
        """-> (PoolBufferId, Event); `MemoryAllocation` if bytes > free_bytes (hip.rs:354-370)."""
        buf, ev = C.c_uint32(), C.c_uint64()
        self._ctx.check(self._ctx.lib.zhip_alloc(self._ctx.ptr, C.c_uint64(bytes_), C.byref(buf), C.byref(ev)))
        return buf.value, Event(ev.value)

    def deallocate(self, buffer_id: int, event_wait_list: Sequence[Event] = ()):
        arr, n = _events_array(event_wait_list)
        self._ctx.check(self._ctx.lib.zhip_free(self._ctx.ptr, C.c_uint32(buffer_id), arr, n))

    def store_variable(self, dtype: DType, value) -> int:
        raw = np.array([value], dtype=_NP_OF[DType(dtype)]).tobytes().ljust(8, b"\0")
        buf = C.c_uint32()
        self._ctx.check(self._ctx.lib.zhip_store_variable(self._ctx.ptr, int(dtype), raw, C.byref(buf)))
        return buf.value

    def get_variable(self, buffer_id: int):
        """-> (dtype, value) or None for memory buffers (backend/mod.rs:609-621)."""
        found, dt = C.c_int32(), C.c_int32()
        raw = (C.c_uint8 * 8)()
        self._ctx.check(self._ctx.lib.zhip_get_variable(self._ctx.ptr, C.c_uint32(buffer_id), C.byref(found),
                                                        C.byref(dt), raw))
        if not found.value:
            return None
        d = DType(dt.value)
        return d, np.frombuffer(bytes(raw)[:d.byte_size()], dtype=_NP_OF[d])[0].item()

    def host_to_pool(self, src, dst: int, event_wait_list: Sequence[Event] = ()) -> Event:
        """Async: `src` (bytes-like / C-contiguous ndarray) must stay alive until the event is synced."""
        addr, nbytes = _host_span(src, writable=False)
        arr, n = _events_array(event_wait_list)
        ev = C.c_uint64()
        self._ctx.check(self._ctx.lib.zhip_h2d(self._ctx.ptr, addr, C.c_uint64(nbytes), C.c_uint32(dst), arr, n,
                                               C.byref(ev)))
        return Event(ev.value)

    def pool_to_host(self, src: int, dst, event_wait_list: Sequence[Event] = ()):
        """Blocking copy into a writable buffer (hip.rs:411-434)."""
        addr, nbytes = _host_span(dst, writable=True)
        arr, n = _events_array(event_wait_list)
        self._ctx.check(self._ctx.lib.zhip_d2h(self._ctx.ptr, C.c_uint32(src), addr, C.c_uint64(nbytes), arr, n))

    def pool_to_pool(self, src_pool, src, dst: int, event_wait_list: Sequence[Event] = ()) -> Event:
        """backend/mod.rs:743-764. `src_pool` is this pool (device copy) or a host source:
        any bytes-like object standing for a HostMemoryPool buffer."""
        if src_pool is self:
            arr, n = _events_array(event_wait_list)
            ev = C.c_uint64()
            nbytes = min(self.buffer_bytes(src), self.buffer_bytes(dst))
            self._ctx.check(self._ctx.lib.zhip_d2d(self._ctx.ptr, C.c_uint32(src), C.c_uint64(0), C.c_uint32(dst),
                                                   C.c_uint64(0), C.c_uint64(nbytes), arr, n, C.byref(ev)))
            return Event(ev.value)
        return self.host_to_pool(src, dst, event_wait_list)

    def copy_range(self, src: int, src_offset: int, dst: int, dst_offset: int, nbytes: int,
                   event_wait_list: Sequence[Event] = ()) -> Event:
        """Device-to-device copy of a byte range between two buffers of this pool (the data movement a
        narrowed / sliced view needs; the reference has no HIP pool_to_pool yet)."""
        arr, n = _events_array(event_wait_list)
        ev = C.c_uint64()
        self._ctx.check(self._ctx.lib.zhip_d2d(self._ctx.ptr, C.c_uint32(src), C.c_uint64(src_offset), C.c_uint32(dst),
                                               C.c_uint64(dst_offset), C.c_uint64(nbytes), arr, n, C.byref(ev)))
        return Event(ev.value)

    def sync_events(self, events: Sequence[Event]):
        arr, n = _events_array(events)
        self._ctx.check(self._ctx.lib.zhip_sync_events(self._ctx.ptr, arr, n))

    def release_events(self, events: Sequence[Event]):
        arr, n = _events_array(events)
        self._ctx.check(self._ctx.lib.zhip_release_events(self._ctx.ptr, arr, n))

    def buffer_ptr(self, buffer_id: int):
        p, b = C.c_void_p(), C.c_uint64()
        self._ctx.check(self._ctx.lib.zhip_buffer_ptr(self._ctx.ptr, C.c_uint32(buffer_id), C.byref(p), C.byref(b)))
        return p.value, b.value

    def buffer_bytes(self, buffer_id: int) -> int:
        return self.buffer_ptr(buffer_id)[1]


class HIPDevice:
    """zyx/src/backend/hip.rs:66-83, 487-728"""

    def __init__(self, ctx: _Context, memory_pool_id: int):
        self._ctx = ctx
        self._memory_pool_id = memory_pool_id
        raw = _DeviceInfo()
        ctx.check(ctx.lib.zhip_get_device_info(ctx.ptr, C.byref(raw)))
        self._info = DeviceInfo(
            compute=raw.compute, max_global_work_dims=list(raw.max_global_work_dims),
            max_local_threads=raw.max_local_threads, max_local_work_dims=list(raw.max_local_work_dims),
            preferred_vector_size=raw.preferred_vector_size, local_mem_size=raw.local_mem_size,
            max_register_bytes=raw.max_register_bytes, tensor_cores=bool(raw.tensor_cores), warp_size=raw.warp_size,
            dtype_capability=list(raw.dtype_capability), has_native_exp2=bool(raw.has_native_exp2),
            supported_vec_lens=list(raw.supported_vec_lens)[:raw.n_supported_vec_lens], total_bytes=raw.total_bytes,
            compute_units=raw.compute_units, clock_khz=raw.clock_khz, name=raw.name.decode(), arch=raw.arch.decode())

    def deinitialize(self):
        pass  # the pool owns the context

    def info(self) -> DeviceInfo:
        return self._info

    def memory_pool_id(self) -> int:
        return self._memory_pool_id

    def free_compute(self) -> int:
        return int(self._ctx.lib.zhip_free_compute(self._ctx.ptr))

    def aot_only(self) -> bool:
        """backend/mod.rs:892-894: false, the device also compiles linearized kernels."""
        return False

    def compile(self, kernel_ir: bytes = b"", debug_asm: bool = False) -> int:
        """Device::compile (backend/mod.rs:899-933) on the image of a linearized kernel (zyx_amd.ir.Kernel.to_bytes());
        `KernelCompilation` when the image is malformed or holds an op the backend has no code for."""
        prog = C.c_uint32()
        self._ctx.check(self._ctx.lib.zhip_compile_ir(self._ctx.ptr, kernel_ir, C.c_uint64(len(kernel_ir)), C.byref(prog)))
        if debug_asm:
            print(self.program_source(prog.value))
        return prog.value

    def program_source(self, program_id: int) -> str:
        n = C.c_uint64()
        self._ctx.check(self._ctx.lib.zhip_program_source(self._ctx.ptr, C.c_uint32(program_id), None, C.c_uint64(0), C.byref(n)))
        buf = C.create_string_buffer(n.value + 1)
        self._ctx.check(self._ctx.lib.zhip_program_source(self._ctx.ptr, C.c_uint32(program_id), buf, C.c_uint64(n.value + 1), C.byref(n)))
        return buf.value.decode()

    def register_kernel(self, desc: KernelDesc) -> int:
        """AOT program registration: what `match_graph` does before pushing Node::Kernel (cblas.rs:225)."""
        prog = C.c_uint32()
        self._ctx.check(self._ctx.lib.zhip_register_kernel(self._ctx.ptr, C.byref(desc), C.byref(prog)))
        return prog.value

    def launch(self, program_id: int, memory_pool: HIPMemoryPool, args: Sequence[int],
               event_wait_list: Sequence[Event] = ()) -> Event:
        """hip.rs:654-719. args = load buffers then store buffers."""
        assert memory_pool._ctx is self._ctx, "device and pool must belong to the same GPU"
        a = (C.c_uint32 * max(len(args), 1))(*args)
        arr, n = _events_array(event_wait_list)
        ev = C.c_uint64()
        self._ctx.check(self._ctx.lib.zhip_launch(self._ctx.ptr, C.c_uint32(program_id), a, C.c_size_t(len(args)), arr,
                                                  n, C.byref(ev)))
        return Event(ev.value)

    def reduce_static(self, dtype: DType, op: int, axis0: bool, rows: int, cols: int, x_ptr: int, out_ptr: int,
                      stream: int = 0):
        """zhip_reduce_static: sum (op 0) / max (op 1) of x[rows, cols] given as raw device addresses, enqueued on the
        caller's hipStream_t (0 = null stream) without any device allocation; asynchronous."""
        self._ctx.check(self._ctx.lib.zhip_reduce_static(self._ctx.ptr, C.c_int32(int(dtype)), C.c_int32(op),
                                                         C.c_int32(int(bool(axis0))), C.c_int64(rows), C.c_int64(cols),
                                                         C.c_void_p(x_ptr), C.c_void_p(out_ptr), C.c_void_p(stream)))

    def measure_ceilings(self, nbytes: int = 128 << 20) -> dict:
        """zhip_measure_ceilings: streaming and matrix-instruction rates this device sustains right now."""
        raw = _Ceilings()
        self._ctx.check(self._ctx.lib.zhip_measure_ceilings(self._ctx.ptr, C.c_uint64(nbytes), C.byref(raw)))
        return {name: round(float(getattr(raw, name)), 1) for name, _ in _Ceilings._fields_}

    def release(self, program_id: int):
        self._ctx.check(self._ctx.lib.zhip_release_program(self._ctx.ptr, C.c_uint32(program_id)))

    def time_kernel(self, program_id: int, args: Sequence[int]) -> int:
        """launch_with_timings (zyx/src/kernel/autotune.rs:775-798): wall-clock ns of launch + sync."""
        a = (C.c_uint32 * max(len(args), 1))(*args)
        ns = C.c_uint64()
        self._ctx.check(self._ctx.lib.zhip_time_kernel(self._ctx.ptr, C.c_uint32(program_id), a, C.c_size_t(len(args)),
                                                       C.byref(ns)))
        return ns.value

    def create_plan(self, nodes: Sequence) -> int:
        """Record a fixed list of Launch nodes [(program_id, [buffer ids: loads then stores]), ...] as
        one replayable unit: the cached ExecPlan of zyx/src/graph/plan.rs:58-237 kept as a HIP graph."""
        progs = (C.c_uint32 * len(nodes))(*[n[0] for n in nodes])
        flat = [b for n in nodes for b in n[1]]
        args = (C.c_uint32 * max(len(flat), 1))(*flat)
        counts = (C.c_uint32 * len(nodes))(*[len(n[1]) for n in nodes])
        plan = C.c_uint32()
        self._ctx.check(self._ctx.lib.zhip_plan_create(self._ctx.ptr, progs, args, counts, C.c_size_t(len(nodes)),
                                                       C.byref(plan)))
        return plan.value

    def launch_plan(self, plan_id: int, event_wait_list: Sequence[Event] = ()) -> Event:
        """execute_plan (zyx/src/graph/plan.rs:271-361) for a plan whose buffers are already allocated."""
        arr, n = _events_array(event_wait_list)
        ev = C.c_uint64()
        self._ctx.check(self._ctx.lib.zhip_plan_launch(self._ctx.ptr, C.c_uint32(plan_id), arr, n, C.byref(ev)))
        return Event(ev.value)

    def destroy_plan(self, plan_id: int):
        self._ctx.check(self._ctx.lib.zhip_plan_destroy(self._ctx.ptr, C.c_uint32(plan_id)))

    def profile_kernel(self, program_id: int, arg_sets: Sequence[Sequence[int]], iters: int) -> float:
        """Mean device microseconds per launch, HIP events on the launch stream."""
        n_args = len(arg_sets[0])
        flat = [b for s in arg_sets for b in s]
        a = (C.c_uint32 * len(flat))(*flat)
        us = C.c_float()
        self._ctx.check(self._ctx.lib.zhip_profile_kernel(self._ctx.ptr, C.c_uint32(program_id), a, C.c_size_t(n_args),
                                                          C.c_size_t(len(arg_sets)), C.c_int32(iters), C.byref(us)))
        return us.value


_NP_OF = {DType.BF16: np.uint16, DType.F16: np.float16, DType.F32: np.float32, DType.F64: np.float64,
          DType.U8: np.uint8, DType.U16: np.uint16, DType.U32: np.uint32, DType.U64: np.uint64, DType.I8: np.int8,
          DType.I16: np.int16, DType.I32: np.int32, DType.I64: np.int64, DType.Bool: np.bool_}


def generate_source(kernel_ir: bytes) -> str:
    """The HIP source `HIPDevice.compile` would build for this image; needs no GPU. `KernelCompilation` with the
    reason when the image is refused."""
    lib = load_library()
    n = C.c_uint64()
    lib.zhip_ir_generate(kernel_ir, C.c_uint64(len(kernel_ir)), None, C.c_uint64(0), C.byref(n))
    buf = C.create_string_buffer(n.value + 1)
    rc = lib.zhip_ir_generate(kernel_ir, C.c_uint64(len(kernel_ir)), buf, C.c_uint64(n.value + 1), C.byref(n))
    if rc != 0:
        raise BackendError(ErrorStatus(rc), buf.value.decode())
    return buf.value.decode()


def compile_cache_stats() -> dict:
    """Run-time compilations, in-memory hits and on-disk hits of this process (zhip_compile_cache_stats)."""
    lib = load_library()
    raw = (C.c_uint64 * 3)()
    lib.zhip_compile_cache_stats(raw)
    return {"compiled": raw[0], "memory_hits": raw[1], "disk_hits": raw[2]}


def device_count() -> int:
    lib = load_library()
    n = C.c_int32()
    rc = lib.zhip_device_count(C.byref(n))
    if rc != 0:
        raise BackendError(ErrorStatus(rc), lib.zhip_last_error(None).decode())
    return n.value


def initialize_device(config: HIPConfig = HIPConfig(), debug: int = 0):
    """hip.rs:122-339: one (pool, device) pair per selected GPU; the device's
    `memory_pool_id` is the index of its pool. `device_ids == []` disables the backend."""
    if config.device_ids is not None and len(config.device_ids) == 0:
        raise BackendError(ErrorStatus.Initialization, "HIP won't be used, as it was configured out")
    ids = config.device_ids if config.device_ids is not None else list(range(device_count()))
    pools, devices = [], []
    for dev in ids:
        ctx = _Context(dev, debug, config.cache_bytes)
        pools.append(HIPMemoryPool(ctx))
        devices.append(HIPDevice(ctx, len(pools) - 1))
    if not devices:
        raise BackendError(ErrorStatus.DeviceEnumeration, "no HIP devices found")
    return pools, devices
