// Drop-in replacement for zyx/src/backend/hip.rs: the HIP slot of zyx's backend plugin interface
// (`MemoryPool::HIP` / `Device::HIP`, zyx/src/backend/mod.rs:533-1028) implemented over the C ABI of
// include/zyx_hip.h (libzyx_hip.so) instead of raw libamdhip64 calls.
//
// No Rust toolchain exists where this library is built and tested, so this file has never been compiled; it is written
// against the reference's types as they stand (paths cited per item) and every call it makes is exercised through the
// same C symbols by zyx_amd/backend.py (ctypes), tests/cabi/client.c (plain C) and tests/fakehip/harness.cpp.
//
// Changes needed outside this file, all in zyx/src/backend/mod.rs:
//   :604  MemoryPool::store_variable   `MemoryPool::HIP(_) => todo!()`      -> `MemoryPool::HIP(pool) => pool.store_variable(scalar)`
//   :618  MemoryPool::get_variable     `MemoryPool::HIP(_) => None`         -> `MemoryPool::HIP(pool) => pool.get_variable(buffer_id)`
//   :756  MemoryPool::pool_to_pool     `MemoryPool::HIP(_) => todo!()`      -> `MemoryPool::HIP(pool) => pool.pool_to_pool(src_pool, src, dst, event_wait_list)?`
//   :957  Device::match_graph          add `Device::HIP(dev) => dev.match_graph(graph, outputs),`
// and `mod hip;` in zyx/src/vendor/mod.rs for the matchers of vendor_hip.rs (saved as zyx/src/vendor/hip.rs).

#![allow(non_snake_case)]
#![allow(clippy::question_mark)]

use super::{DTypeCapability, Device, DeviceInfo, MemoryPool};
use crate::backend::{DeviceId, DeviceProgramId, Event, PoolBufferId, PoolId, ProgramId};
use crate::dtype::Constant;
use crate::error::{BackendError, ErrorStatus};
use crate::graph::{ClassId, Graph, Node, NodeData};
use crate::kernel::{IdxKind, Kernel, MemLayout, Op, OpId};
use crate::shape::Dim;
use crate::slab::Slab;
use crate::{DType, Map, Set};
use libloading::Library;
use nanoserde::DeJson;
use std::collections::BTreeSet;
use std::ffi::{c_char, c_void, CStr};
use std::ptr;
use std::sync::Arc;

#[derive(Debug, Default, DeJson)]
#[nserde(default)]
pub struct HIPConfig {
    device_ids: Option<Vec<i32>>,
}

// ---- C ABI mirror (include/zyx_hip.h) ---------------------------------------------------------------------------

type Ctx = *mut c_void;

#[repr(C)]
struct ZhipConfig {
    device_id: i32,
    debug: u32,
    cache_bytes: u64,
}

/// zhip_device_info: 272 bytes, offsets checked by tests/cabi/client.c against the C header.
#[repr(C)]
struct ZhipDeviceInfo {
    compute: u64,
    max_global_work_dims: [u64; 3],
    max_local_threads: u32,
    max_local_work_dims: [u32; 3],
    preferred_vector_size: u32,
    local_mem_size: u64,
    max_register_bytes: u64,
    tensor_cores: u32,
    warp_size: u32,
    dtype_capability: [u32; 13],
    has_native_exp2: u32,
    n_supported_vec_lens: u32,
    supported_vec_lens: [u32; 4],
    total_bytes: u64,
    compute_units: u32,
    clock_khz: u32,
    name: [c_char; 64],
    arch: [c_char; 32],
}

/// zhip_kernel_desc: 208 bytes.
#[repr(C)]
#[derive(Clone, Copy)]
pub(crate) struct ZhipKernelDesc {
    pub kind: i32,
    pub dtype: i32,
    pub out_dtype: i32,
    pub flags: i32,
    pub dims: [i64; 8],
    pub fparams: [f32; 8],
    pub iparams: [i32; 24],
}

impl ZhipKernelDesc {
    pub(crate) const fn zeroed() -> Self {
        Self { kind: 0, dtype: 0, out_dtype: 0, flags: 0, dims: [0; 8], fparams: [0.0; 8], iparams: [0; 24] }
    }
}

/// zhip_ir_header / zhip_ir_op: 16 and 32 bytes, little endian.
#[repr(C)]
struct ZhipIrHeader {
    magic: u32,
    n_ops: u32,
    n_extra: u32,
    reserved: u32,
}
#[repr(C)]
#[derive(Clone, Copy)]
struct ZhipIrOp {
    id: u32,
    opcode: u16,
    dtype: u16,
    a: u32,
    b: u32,
    c: u32,
    aux: u32,
    imm: u64,
}
const ZHIP_IR_MAGIC: u32 = 0x3152_495a;
const ZHIP_NULL: u32 = u32::MAX;

/// zhip_kernel_kind
pub(crate) mod kind {
    pub const SOFTMAX_ROWS: i32 = 1;
    pub const ELEMENTWISE: i32 = 2;
    pub const REDUCE: i32 = 3;
    pub const GEMM: i32 = 4;
    pub const NORM_ROWS: i32 = 5;
    pub const CROSS_ENTROPY: i32 = 6;
    pub const CONV2D: i32 = 7;
    pub const MAX_POOL2D: i32 = 8;
    pub const INDEX: i32 = 9;
    pub const ATTENTION: i32 = 10;
    pub const ATTENTION_BWD: i32 = 11;
    pub const NORM_ROWS_BWD: i32 = 12;
    pub const ARGMAX: i32 = 13;
}

/// Every export of libzyx_hip.so, resolved once (the style of the reference's backends, hip.rs:122-188).
pub(crate) struct Zhip {
    _lib: Library,
    device_count: unsafe extern "C" fn(*mut i32) -> i32,
    init: unsafe extern "C" fn(*const ZhipConfig, *mut Ctx) -> i32,
    deinit: unsafe extern "C" fn(Ctx) -> i32,
    last_error: unsafe extern "C" fn(Ctx) -> *const c_char,
    get_device_info: unsafe extern "C" fn(Ctx, *mut ZhipDeviceInfo) -> i32,
    free_bytes: unsafe extern "C" fn(Ctx) -> u64,
    free_compute: unsafe extern "C" fn(Ctx) -> u64,
    alloc: unsafe extern "C" fn(Ctx, u64, *mut u32, *mut u64) -> i32,
    free: unsafe extern "C" fn(Ctx, u32, *const u64, usize) -> i32,
    store_variable: unsafe extern "C" fn(Ctx, i32, *const u8, *mut u32) -> i32,
    get_variable: unsafe extern "C" fn(Ctx, u32, *mut i32, *mut i32, *mut u8) -> i32,
    h2d: unsafe extern "C" fn(Ctx, *const c_void, u64, u32, *const u64, usize, *mut u64) -> i32,
    d2h: unsafe extern "C" fn(Ctx, u32, *mut c_void, u64, *const u64, usize) -> i32,
    d2d: unsafe extern "C" fn(Ctx, u32, u64, u32, u64, u64, *const u64, usize, *mut u64) -> i32,
    sync_events: unsafe extern "C" fn(Ctx, *const u64, usize) -> i32,
    release_events: unsafe extern "C" fn(Ctx, *const u64, usize) -> i32,
    buffer_ptr: unsafe extern "C" fn(Ctx, u32, *mut *mut c_void, *mut u64) -> i32,
    register_kernel: unsafe extern "C" fn(Ctx, *const ZhipKernelDesc, *mut u32) -> i32,
    compile_ir: unsafe extern "C" fn(Ctx, *const c_void, u64, *mut u32) -> i32,
    compile_cache_stats: unsafe extern "C" fn(*mut u64),
    ir_generate: unsafe extern "C" fn(*const c_void, u64, *mut c_char, u64, *mut u64) -> i32,
    program_source: unsafe extern "C" fn(Ctx, u32, *mut c_char, u64, *mut u64) -> i32,
    launch: unsafe extern "C" fn(Ctx, u32, *const u32, usize, *const u64, usize, *mut u64) -> i32,
    release_program: unsafe extern "C" fn(Ctx, u32) -> i32,
    time_kernel: unsafe extern "C" fn(Ctx, u32, *const u32, usize, *mut u64) -> i32,
    profile_kernel: unsafe extern "C" fn(Ctx, u32, *const u32, usize, usize, i32, *mut f32) -> i32,
    plan_create: unsafe extern "C" fn(Ctx, *const u32, *const u32, *const u32, usize, *mut u32) -> i32,
    plan_launch: unsafe extern "C" fn(Ctx, u32, *const u64, usize, *mut u64) -> i32,
    plan_destroy: unsafe extern "C" fn(Ctx, u32) -> i32,
    // zhip_rng_*, zhip_reduce_static and zhip_measure_ceilings have no caller inside zyx: its random tensors come
    // from its own Rng, and nothing in the runtime launches on foreign streams or asks for measured ceilings.
}

impl std::fmt::Debug for Zhip {
    fn fmt(&self, f: &mut std::fmt::Formatter<'_>) -> std::fmt::Result {
        f.write_str("Zhip")
    }
}

impl Zhip {
    fn resolve(lib: Library) -> Result<Self, BackendError> {
        macro_rules! sym {
            ($name:literal) => {
                *unsafe { lib.get($name) }.map_err(|e| BackendError {
                    status: ErrorStatus::DyLibNotFound,
                    context: format!("libzyx_hip.so lacks {}: {e}", String::from_utf8_lossy($name)).into(),
                })?
            };
        }
        Ok(Self {
            device_count: sym!(b"zhip_device_count\0"),
            init: sym!(b"zhip_init\0"),
            deinit: sym!(b"zhip_deinit\0"),
            last_error: sym!(b"zhip_last_error\0"),
            get_device_info: sym!(b"zhip_get_device_info\0"),
            free_bytes: sym!(b"zhip_free_bytes\0"),
            free_compute: sym!(b"zhip_free_compute\0"),
            alloc: sym!(b"zhip_alloc\0"),
            free: sym!(b"zhip_free\0"),
            store_variable: sym!(b"zhip_store_variable\0"),
            get_variable: sym!(b"zhip_get_variable\0"),
            h2d: sym!(b"zhip_h2d\0"),
            d2h: sym!(b"zhip_d2h\0"),
            d2d: sym!(b"zhip_d2d\0"),
            sync_events: sym!(b"zhip_sync_events\0"),
            release_events: sym!(b"zhip_release_events\0"),
            buffer_ptr: sym!(b"zhip_buffer_ptr\0"),
            register_kernel: sym!(b"zhip_register_kernel\0"),
            compile_ir: sym!(b"zhip_compile_ir\0"),
            compile_cache_stats: sym!(b"zhip_compile_cache_stats\0"),
            ir_generate: sym!(b"zhip_ir_generate\0"),
            program_source: sym!(b"zhip_program_source\0"),
            launch: sym!(b"zhip_launch\0"),
            release_program: sym!(b"zhip_release_program\0"),
            time_kernel: sym!(b"zhip_time_kernel\0"),
            profile_kernel: sym!(b"zhip_profile_kernel\0"),
            plan_create: sym!(b"zhip_plan_create\0"),
            plan_launch: sym!(b"zhip_plan_launch\0"),
            plan_destroy: sym!(b"zhip_plan_destroy\0"),
            _lib: lib,
        })
    }

    /// A non-zero return is `ErrorStatus` ordinal + 1 with the text in zhip_last_error: the BackendError callers expect.
    fn check(&self, ctx: Ctx, rc: i32) -> Result<(), BackendError> {
        if rc == 0 {
            return Ok(());
        }
        let status = match rc {
            1 => ErrorStatus::DyLibNotFound,
            2 => ErrorStatus::Initialization,
            3 => ErrorStatus::Deinitialization,
            4 => ErrorStatus::DeviceEnumeration,
            5 => ErrorStatus::DeviceQuery,
            6 => ErrorStatus::MemoryAllocation,
            7 => ErrorStatus::MemoryDeallocation,
            8 => ErrorStatus::MemoryCopyH2P,
            9 => ErrorStatus::MemoryCopyP2H,
            10 => ErrorStatus::IncorrectKernelArg,
            11 => ErrorStatus::KernelCompilation,
            12 => ErrorStatus::KernelLaunch,
            _ => ErrorStatus::KernelSync,
        };
        let msg = unsafe { CStr::from_ptr((self.last_error)(ctx)) }.to_string_lossy().into_owned();
        Err(BackendError { status, context: msg.into() })
    }
}

// ---- the slot's types ------------------------------------------------------------------------------------------------

/// One `zhip_ctx` stands for the pool + device pair of a GPU; the pool owns it (it is deinitialised last).
#[derive(Debug)]
pub struct HIPMemoryPool {
    z: Arc<Zhip>,
    ctx: Ctx,
}

#[derive(Debug)]
pub struct HIPDevice {
    z: Arc<Zhip>,
    ctx: Ctx,
    device_id: DeviceId,
    memory_pool_id: PoolId,
    dev_info: DeviceInfo,
}

/// `handle == 0` is the null event (already signalled), the analogue of a null `hipEvent_t` (hip.rs:375,396).
#[derive(Debug, Clone)]
pub struct HIPEvent {
    handle: u64,
}

// The library serialises calls on a context itself and is callable from any thread.
unsafe impl Send for HIPMemoryPool {}
unsafe impl Send for HIPDevice {}

fn handles(events: Vec<Event>) -> Vec<u64> {
    events
        .into_iter()
        .filter_map(|e| match e {
            Event::HIP(HIPEvent { handle }) if handle != 0 => Some(handle),
            _ => None,
        })
        .collect()
}

pub(super) fn initialize_device(
    config: &HIPConfig,
    memory_pools: &mut Slab<PoolId, MemoryPool>,
    devices: &mut Slab<DeviceId, Device>,
    debug_dev: bool,
) -> Result<(), BackendError> {
    if let Some(device_ids) = &config.device_ids
        && device_ids.is_empty()
    {
        return Err(BackendError { status: ErrorStatus::Initialization, context: "HIP won't be used, as it was configured out".into() });
    }
    let lib = ["libzyx_hip.so", "/usr/lib/zyx/libzyx_hip.so", "/usr/local/lib/libzyx_hip.so"]
        .iter()
        .find_map(|p| unsafe { Library::new(p) }.ok())
        .ok_or(BackendError { status: ErrorStatus::DyLibNotFound, context: "libzyx_hip.so not found.".into() })?;
    let z = Arc::new(Zhip::resolve(lib)?);
    let mut n = 0i32;
    z.check(ptr::null_mut(), unsafe { (z.device_count)(&raw mut n) })?;
    let ids: Vec<i32> = config.device_ids.clone().unwrap_or_else(|| (0..n).collect());
    // ZYX_DEBUG reaches the library as the same bit mask (lib.rs:101-163): 1 devices, 32 launches, 64 memory, 128 compile
    let debug = std::env::var("ZYX_DEBUG").ok().and_then(|x| x.parse::<u32>().ok()).unwrap_or(u32::from(debug_dev));
    let mut found = false;
    for dev in ids {
        if dev < 0 || dev >= n {
            continue;
        }
        let mut ctx: Ctx = ptr::null_mut();
        let cfg = ZhipConfig { device_id: dev, debug, cache_bytes: 0 };
        z.check(ptr::null_mut(), unsafe { (z.init)(&raw const cfg, &raw mut ctx) })?;
        let mut raw: ZhipDeviceInfo = unsafe { std::mem::zeroed() };
        z.check(ctx, unsafe { (z.get_device_info)(ctx, &raw mut raw) })?;
        let dev_info = DeviceInfo {
            compute: u128::from(raw.compute),
            max_global_work_dims: raw.max_global_work_dims.iter().map(|&d| d as Dim).collect(),
            max_local_threads: raw.max_local_threads,
            max_local_work_dims: raw.max_local_work_dims.to_vec(),
            preferred_vector_size: raw.preferred_vector_size as u8,
            local_mem_size: raw.local_mem_size as Dim,
            max_register_bytes: raw.max_register_bytes as Dim,
            tensor_cores: raw.tensor_cores != 0,
            warp_size: raw.warp_size as u16,
            // one u32 bit mask per dtype, the layout of DTypeCapability (mod.rs:416-471); the field is private to
            // backend/mod.rs, of which this file is a submodule
            dtype_capability: std::array::from_fn(|i| if raw.dtype_capability[i] == u32::MAX { DTypeCapability::all() } else { DTypeCapability::none() }),
            has_native_exp2: raw.has_native_exp2 != 0,
            supported_vec_lens: raw.supported_vec_lens[..raw.n_supported_vec_lens as usize].iter().map(|&v| v as u8).collect(),
        };
        if debug_dev {
            let name = unsafe { CStr::from_ptr(raw.name.as_ptr()) }.to_string_lossy();
            println!("Using HIP device {name} with {} B of memory through libzyx_hip.so", raw.total_bytes);
        }
        let pool_id = memory_pools.push(MemoryPool::HIP(HIPMemoryPool { z: z.clone(), ctx }));
        let device_id = devices.push(Device::HIP(HIPDevice { z: z.clone(), ctx, device_id: DeviceId::NULL, memory_pool_id: pool_id, dev_info }));
        if let Device::HIP(d) = &mut devices[device_id] {
            d.device_id = device_id; // as CblasDevice learns its id, cblas.rs:151-177
        }
        found = true;
    }
    if !found {
        return Err(BackendError { status: ErrorStatus::DeviceEnumeration, context: "No HIP devices found.".into() });
    }
    Ok(())
}

impl HIPMemoryPool {
    pub(super) fn deinitialize(&mut self) {
        if !self.ctx.is_null() {
            let _ = unsafe { (self.z.deinit)(self.ctx) };
            self.ctx = ptr::null_mut();
        }
    }

    pub(super) fn free_bytes(&self) -> Dim {
        unsafe { (self.z.free_bytes)(self.ctx) as Dim }
    }

    pub(super) fn allocate(&mut self, bytes: Dim) -> Result<(PoolBufferId, Event), BackendError> {
        let (mut id, mut ev) = (ZHIP_NULL, 0u64);
        self.z.check(self.ctx, unsafe { (self.z.alloc)(self.ctx, bytes as u64, &raw mut id, &raw mut ev) })?;
        Ok((PoolBufferId::from(id as usize), Event::HIP(HIPEvent { handle: ev })))
    }

    pub(super) fn deallocate(&mut self, buffer_id: PoolBufferId, event_wait_list: Vec<Event>) {
        let evs = handles(event_wait_list);
        let id = usize::from(buffer_id) as u32;
        self.z.check(self.ctx, unsafe { (self.z.free)(self.ctx, id, evs.as_ptr(), evs.len()) }).unwrap();
    }

    /// MemoryPool::store_variable (mod.rs:597-607): scalar kernel arguments live in the buffer id space.
    pub(super) fn store_variable(&mut self, scalar: Constant) -> PoolBufferId {
        let mut value = [0u8; 8];
        let bytes = scalar.to_le_bytes();
        value[..bytes.len()].copy_from_slice(&bytes);
        let mut id = ZHIP_NULL;
        self.z.check(self.ctx, unsafe { (self.z.store_variable)(self.ctx, scalar.dtype() as i32, value.as_ptr(), &raw mut id) }).unwrap();
        PoolBufferId::from(id as usize)
    }

    /// MemoryPool::get_variable (mod.rs:609-621): `None` for memory buffers and unknown ids.
    pub(super) fn get_variable(&mut self, buffer_id: PoolBufferId) -> Option<Constant> {
        let (mut found, mut dtype, mut value) = (0i32, 0i32, [0u8; 8]);
        let id = usize::from(buffer_id) as u32;
        if unsafe { (self.z.get_variable)(self.ctx, id, &raw mut found, &raw mut dtype, value.as_mut_ptr()) } != 0 || found == 0 {
            return None;
        }
        Some(Constant::from_le_bytes(&value, dtype_from_ordinal(dtype)?))
    }

    /// Async: `src` must stay valid until the returned event is synced (runtime.rs:1-5). The wait list is consumed.
    pub(super) fn host_to_pool(&mut self, src: &[u8], dst: PoolBufferId, event_wait_list: Vec<Event>) -> Result<Event, BackendError> {
        let evs = handles(event_wait_list);
        let mut ev = 0u64;
        let id = usize::from(dst) as u32;
        self.z.check(self.ctx, unsafe { (self.z.h2d)(self.ctx, src.as_ptr().cast(), src.len() as u64, id, evs.as_ptr(), evs.len(), &raw mut ev) })?;
        Ok(Event::HIP(HIPEvent { handle: ev }))
    }

    /// Blocks until the bytes are in `dst` (hip.rs:411-434).
    pub(super) fn pool_to_host(&mut self, src: PoolBufferId, dst: &mut [u8], event_wait_list: Vec<Event>) -> Result<(), BackendError> {
        let evs = handles(event_wait_list);
        let id = usize::from(src) as u32;
        self.z.check(self.ctx, unsafe { (self.z.d2h)(self.ctx, id, dst.as_mut_ptr().cast(), dst.len() as u64, evs.as_ptr(), evs.len()) })
    }

    /// MemoryPool::pool_to_pool (mod.rs:743-764), the sources the CUDA pool accepts (cuda.rs:951-967) plus this pool.
    pub(super) fn pool_to_pool(
        &mut self,
        src_pool: &mut MemoryPool,
        src: PoolBufferId,
        dst: PoolBufferId,
        event_wait_list: Vec<Event>,
    ) -> Result<Event, BackendError> {
        match src_pool {
            MemoryPool::Host(src_pool) => self.host_to_pool(src_pool.get_buffer(src), dst, event_wait_list),
            MemoryPool::Disk(src_pool) => {
                let mut byte_slice = vec![0u8; src_pool.buffer_bytes(src) as usize];
                src_pool.pool_to_host(src, &mut byte_slice, Vec::new())?;
                let event = self.host_to_pool(&byte_slice, dst, event_wait_list)?;
                // the staging vector dies with this frame: the copy has to be complete before that
                self.sync_events(vec![event])?;
                Ok(Event::HIP(HIPEvent { handle: 0 }))
            }
            MemoryPool::HIP(src_pool) if src_pool.ctx == self.ctx => {
                let (mut p, mut sb, mut db) = (ptr::null_mut(), 0u64, 0u64);
                let (s, d) = (usize::from(src) as u32, usize::from(dst) as u32);
                self.z.check(self.ctx, unsafe { (self.z.buffer_ptr)(self.ctx, s, &raw mut p, &raw mut sb) })?;
                self.z.check(self.ctx, unsafe { (self.z.buffer_ptr)(self.ctx, d, &raw mut p, &raw mut db) })?;
                let evs = handles(event_wait_list);
                let mut ev = 0u64;
                self.z.check(self.ctx, unsafe { (self.z.d2d)(self.ctx, s, 0, d, 0, sb.min(db), evs.as_ptr(), evs.len(), &raw mut ev) })?;
                Ok(Event::HIP(HIPEvent { handle: ev }))
            }
            other => {
                // another device's pool: staged through the host like the reference's cross-device copies
                let bytes = match other {
                    MemoryPool::HIP(p) => {
                        let (mut ptr_, mut b) = (ptr::null_mut(), 0u64);
                        p.z.check(p.ctx, unsafe { (p.z.buffer_ptr)(p.ctx, usize::from(src) as u32, &raw mut ptr_, &raw mut b) })?;
                        b as usize
                    }
                    _ => return Err(BackendError { status: ErrorStatus::MemoryCopyH2P, context: "pool_to_pool: unsupported source pool".into() }),
                };
                let mut byte_slice = vec![0u8; bytes];
                other.pool_to_host(src, &mut byte_slice, Vec::new())?;
                let event = self.host_to_pool(&byte_slice, dst, event_wait_list)?;
                self.sync_events(vec![event])?;
                Ok(Event::HIP(HIPEvent { handle: 0 }))
            }
        }
    }

    pub fn sync_events(&mut self, events: Vec<Event>) -> Result<(), BackendError> {
        let evs = handles(events);
        self.z.check(self.ctx, unsafe { (self.z.sync_events)(self.ctx, evs.as_ptr(), evs.len()) })
    }

    pub fn release_events(&mut self, events: Vec<Event>) {
        let evs = handles(events);
        self.z.check(self.ctx, unsafe { (self.z.release_events)(self.ctx, evs.as_ptr(), evs.len()) }).unwrap();
    }
}

impl Drop for HIPMemoryPool {
    fn drop(&mut self) {
        self.deinitialize();
    }
}

fn dtype_from_ordinal(d: i32) -> Option<DType> {
    // discriminant order of zyx/src/dtype.rs:20-47
    Some(match d {
        0 => DType::BF16,
        1 => DType::F16,
        2 => DType::F32,
        3 => DType::F64,
        4 => DType::U8,
        5 => DType::U16,
        6 => DType::U32,
        7 => DType::U64,
        8 => DType::I8,
        9 => DType::I16,
        10 => DType::I32,
        11 => DType::I64,
        12 => DType::Bool,
        _ => return None,
    })
}

impl HIPDevice {
    pub(super) const fn deinitialize(&mut self) {} // the pool owns the context

    pub(super) const fn info(&self) -> &DeviceInfo {
        &self.dev_info
    }

    pub(super) const fn memory_pool_id(&self) -> PoolId {
        self.memory_pool_id
    }

    /// Device-selection weight (runtime.rs:2152-2163); the C backend reports 10 * 2^40, an MI355X about 8e14.
    pub fn free_compute(&self) -> u128 {
        u128::from(unsafe { (self.z.free_compute)(self.ctx) })
    }

    /// Device::compile (mod.rs:899-933): the linearized kernel goes to the library as a flat image, which generates
    /// HIP source for it and compiles it with hiprtc (cached by source hash). `KernelCompilation` when the kernel holds
    /// an op the library has no code for (Wmma, tile ops, Asm): autotune then moves on, as for any failing candidate.
    pub fn compile(&mut self, kernel: &Kernel, debug_asm: bool) -> Result<DeviceProgramId, BackendError> {
        let image = kernel_image(kernel);
        let mut prog = ZHIP_NULL;
        self.z.check(self.ctx, unsafe { (self.z.compile_ir)(self.ctx, image.as_ptr().cast(), image.len() as u64, &raw mut prog) })?;
        if debug_asm {
            let mut len = 0u64;
            unsafe { (self.z.program_source)(self.ctx, prog, ptr::null_mut(), 0, &raw mut len) };
            let mut buf = vec![0u8; len as usize + 1];
            unsafe { (self.z.program_source)(self.ctx, prog, buf.as_mut_ptr().cast(), buf.len() as u64, &raw mut len) };
            println!("{}", String::from_utf8_lossy(&buf[..len as usize]));
        }
        Ok(DeviceProgramId::from(prog as usize))
    }

    /// `args` = one id per `Op::Param` in head order, loads before stores (linearize.rs:138-155; AOT kernels: inputs
    /// then outputs, cblas.rs:260-263). Variables are `store_variable` ids; the library reads grid sizes that come from
    /// a Variable (`GwsDim::Param`) out of them at launch. The wait list is consumed.
    pub fn launch(
        &mut self,
        program_id: DeviceProgramId,
        memory_pool: &mut HIPMemoryPool,
        args: &[PoolBufferId],
        event_wait_list: Vec<Event>,
    ) -> Result<Event, BackendError> {
        debug_assert_eq!(memory_pool.ctx, self.ctx);
        let ids: Vec<u32> = args.iter().map(|&a| usize::from(a) as u32).collect();
        let evs = handles(event_wait_list);
        let mut ev = 0u64;
        let prog = usize::from(program_id) as u32;
        self.z.check(self.ctx, unsafe { (self.z.launch)(self.ctx, prog, ids.as_ptr(), ids.len(), evs.as_ptr(), evs.len(), &raw mut ev) })?;
        Ok(Event::HIP(HIPEvent { handle: ev }))
    }

    pub fn release(&mut self, program_id: DeviceProgramId) {
        let _ = unsafe { (self.z.release_program)(self.ctx, usize::from(program_id) as u32) };
    }

    /// Registers one hand-written kernel and measures it on scratch buffers of the sizes its arguments need
    /// (`arg_bytes`, loads then stores, each with the runtime's one element of slack already included), the way
    /// `launch_with_timings` times a candidate (autotune.rs:775-798). Returns the program and nanoseconds.
    pub(crate) fn register_and_time(&mut self, desc: &ZhipKernelDesc, arg_bytes: &[u64]) -> Option<(DeviceProgramId, u64)> {
        let mut prog = ZHIP_NULL;
        if unsafe { (self.z.register_kernel)(self.ctx, desc, &raw mut prog) } != 0 {
            return None; // a shape or dtype no kernel covers: the fused zyx kernels keep the class
        }
        let mut bufs = Vec::with_capacity(arg_bytes.len());
        let mut evs = Vec::new();
        for &bytes in arg_bytes {
            let (mut id, mut ev) = (ZHIP_NULL, 0u64);
            if unsafe { (self.z.alloc)(self.ctx, bytes, &raw mut id, &raw mut ev) } != 0 {
                for &b in &bufs {
                    unsafe { (self.z.free)(self.ctx, b, ptr::null(), 0) };
                }
                unsafe { (self.z.release_program)(self.ctx, prog) };
                return None;
            }
            bufs.push(id);
            if ev != 0 {
                evs.push(ev);
            }
        }
        unsafe { (self.z.sync_events)(self.ctx, evs.as_ptr(), evs.len()) };
        let mut best = u64::MAX;
        for _ in 0..3 {
            let mut ns = 0u64;
            if unsafe { (self.z.time_kernel)(self.ctx, prog, bufs.as_ptr(), bufs.len(), &raw mut ns) } == 0 {
                best = best.min(ns);
            }
        }
        for &b in &bufs {
            unsafe { (self.z.free)(self.ctx, b, ptr::null(), 0) };
        }
        if best == u64::MAX {
            unsafe { (self.z.release_program)(self.ctx, prog) };
            return None;
        }
        Some((DeviceProgramId::from(prog as usize), best.max(1)))
    }

    /// Device::match_graph (mod.rs:952-961): every subgraph a hand-written kernel computes gets a `Node::Kernel` in
    /// its output class, with the measured time, so that it competes with the fused zyx kernels in extraction
    /// (cblas.rs:213-238 does this for sgemm with `time = 1`). The matchers live in zyx/src/vendor/hip.rs.
    pub fn match_graph(&mut self, graph: &mut Graph, outputs: &BTreeSet<ClassId>) {
        let order = graph.topo_sort_classes_without_kernels(&Set::default(), outputs, None);
        for &cid in &order {
            // the first matcher that recognises the class wins; wider fusions are tried before their parts
            let Some(m) = graph
                .match_hip_linear(cid)
                .or_else(|| graph.match_hip_softmax(cid))
                .or_else(|| graph.match_hip_cross_entropy(cid))
                .or_else(|| graph.match_hip_norm_rows(cid))
                .or_else(|| graph.match_hip_attention(cid))
                .or_else(|| graph.match_hip_reduce(cid))
            else {
                continue;
            };
            let Some((program, time)) = self.register_and_time(&m.desc, &m.arg_bytes) else {
                continue;
            };
            let nid = graph.nodes.push(NodeData {
                node: Node::Kernel {
                    inputs: m.inputs.clone().into_boxed_slice(),
                    outputs: m.outputs.clone().into_boxed_slice(),
                    program_id: ProgramId { device: self.device_id, program },
                    time,
                },
                class_of: m.outputs[0],
            });
            // the node id goes into every output class (cblas.rs:227-236)
            for &out in &m.outputs {
                graph.classes[out].nodes.push(nid);
            }
        }
    }
}

/// What a matcher hands to `match_graph`: the descriptor to register, the operand classes in launch order (inputs then
/// outputs, the ORIGINAL operand classes: no transposes materialised, vendor/matmul.rs:35-42) and the bytes of each.
pub(crate) struct HipMatch {
    pub desc: ZhipKernelDesc,
    pub inputs: Vec<ClassId>,
    pub outputs: Vec<ClassId>,
    pub arg_bytes: Vec<u64>,
}

// ---- the flat image of a linearized kernel ---------------------------------------------------------------------------

fn vlen(layout: &MemLayout) -> u32 {
    match layout {
        MemLayout::Scalar => 0,
        MemLayout::Vector(n) => u32::from(*n),
        MemLayout::Tile { .. } => u32::MAX, // refused by the library
    }
}

/// `zhip_ir_header | zhip_ir_op[n] in head -> next order | u32 extra[]`, little endian (include/zyx_hip.h). Enum
/// discriminants (DType, UOp, BOp, ParamKind, MemScope) are the reference's own order, so they are cast.
fn kernel_image(kernel: &Kernel) -> Vec<u8> {
    let mut ops: Vec<ZhipIrOp> = Vec::new();
    let mut extra: Vec<u32> = Vec::new();
    let raw = |id: OpId| -> u32 { if id.is_null() { ZHIP_NULL } else { usize::from(id) as u32 } };
    let mut id = kernel.head;
    while !id.is_null() {
        let mut o = ZhipIrOp { id: raw(id), opcode: 0, dtype: 0, a: ZHIP_NULL, b: ZHIP_NULL, c: ZHIP_NULL, aux: 0, imm: 0 };
        match &kernel.ops[id].op {
            Op::Const(c) => {
                o.opcode = 0;
                o.dtype = c.dtype() as u16;
                let mut v = [0u8; 8];
                let b = c.to_le_bytes();
                v[..b.len()].copy_from_slice(&b);
                o.imm = u64::from_le_bytes(v);
            }
            // `shape` is nulled by linearize (ops.rs:33-35): the element count is left 0 = unchecked unless the
            // caller resolved it before (Kernel::alloc_buffers); the library then only checks liveness and kind
            Op::Param { dtype, kind, .. } => {
                o.opcode = 1;
                o.dtype = *dtype as u16;
                o.aux = *kind as u32;
            }
            Op::Storage { dtype, scope, len } => {
                o.opcode = 2;
                o.dtype = *dtype as u16;
                o.aux = *scope as u32;
                o.imm = *len as u64;
            }
            Op::Load { src, index, layout } => {
                o.opcode = 3;
                o.a = raw(*src);
                o.b = raw(*index);
                o.aux = vlen(layout);
            }
            Op::Store { dst, src, index, layout } => {
                o.opcode = 4;
                o.a = raw(*dst);
                o.b = raw(*src);
                o.c = raw(*index);
                o.aux = vlen(layout);
            }
            Op::Cast { x, dtype } => {
                o.opcode = 5;
                o.a = raw(*x);
                o.dtype = *dtype as u16;
            }
            Op::Unary { x, uop } => {
                o.opcode = 6;
                o.a = raw(*x);
                o.aux = *uop as u32;
            }
            Op::Binary { x, y, bop } => {
                o.opcode = 7;
                o.a = raw(*x);
                o.b = raw(*y);
                o.aux = *bop as u32;
            }
            Op::Mad { x, y, z } => {
                o.opcode = 8;
                o.a = raw(*x);
                o.b = raw(*y);
                o.c = raw(*z);
            }
            Op::Stack { ops: v } => {
                o.opcode = 9;
                o.a = extra.len() as u32;
                o.b = v.len() as u32;
                extra.extend(v.iter().map(|&x| raw(x)));
            }
            Op::Devectorize { vec, idx } => {
                o.opcode = 10;
                o.a = raw(*vec);
                o.aux = *idx as u32;
            }
            Op::Index { axis, kind: IdxKind::Group(len) } => {
                o.opcode = 11;
                o.a = raw(*len);
                o.aux = *axis;
            }
            Op::Index { axis, kind: IdxKind::Local(len) } => {
                o.opcode = 11;
                o.aux = *axis | (1 << 8);
                o.imm = u64::from(*len);
            }
            Op::Index { axis, kind: IdxKind::Warp(_) } => {
                o.opcode = 11;
                o.aux = *axis | (2 << 8); // refused, `todo!()` in the reference's emitters too
            }
            Op::Loop { len } => {
                o.opcode = 12;
                o.a = raw(*len);
            }
            Op::EndLoop => o.opcode = 13,
            Op::If { condition } => {
                o.opcode = 14;
                o.a = raw(*condition);
            }
            Op::EndIf => o.opcode = 15,
            Op::Barrier => o.opcode = 16,
            Op::Wmma { .. } => o.opcode = 17,
            Op::ReduceTile { .. } => o.opcode = 18,
            Op::MatmulTile { .. } => o.opcode = 19,
            Op::TransposeTile { .. } => o.opcode = 20,
            Op::Asm { .. } => o.opcode = 21,
            Op::Move { .. } => o.opcode = 22,
            Op::Reduce { .. } => o.opcode = 23,
        }
        ops.push(o);
        id = kernel.next_op(id);
    }
    let mut out = Vec::with_capacity(16 + ops.len() * 32 + extra.len() * 4);
    let header = ZhipIrHeader { magic: ZHIP_IR_MAGIC, n_ops: ops.len() as u32, n_extra: extra.len() as u32, reserved: 0 };
    for w in [header.magic, header.n_ops, header.n_extra, header.reserved] {
        out.extend_from_slice(&w.to_le_bytes());
    }
    for o in &ops {
        out.extend_from_slice(&o.id.to_le_bytes());
        out.extend_from_slice(&o.opcode.to_le_bytes());
        out.extend_from_slice(&o.dtype.to_le_bytes());
        for w in [o.a, o.b, o.c, o.aux] {
            out.extend_from_slice(&w.to_le_bytes());
        }
        out.extend_from_slice(&o.imm.to_le_bytes());
    }
    for w in &extra {
        out.extend_from_slice(&w.to_le_bytes());
    }
    out
}

#[allow(unused)]
fn _layout_checks() {
    // the sizes the C header fixes (tests/cabi/client.c prints the same from C)
    const _: () = assert!(std::mem::size_of::<ZhipKernelDesc>() == 208);
    const _: () = assert!(std::mem::size_of::<ZhipIrOp>() == 32);
    const _: () = assert!(std::mem::size_of::<ZhipIrHeader>() == 16);
    const _: () = assert!(std::mem::size_of::<ZhipConfig>() == 16);
    const _: () = assert!(std::mem::size_of::<ZhipDeviceInfo>() == 272);
    let _ = Map::<u32, u32>::default();
}
