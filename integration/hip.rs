//! `src/hip.rs`: the HIP twin of the reference's `src/cuda.rs` for the MoE FFN path.
//!
//! The reference's Rust operators (`src/ffn.rs`, `src/moe.rs`, `src/expert_packing.rs`, `src/fp8_linear.rs`) reach the
//! GPU through a thin wrapper over the CUDA driver API that `src/cuda.rs` loads from `libcuda.so.1` with `libloading`
//! (`src/cuda.rs:240-327`).  This file is the same wrapper over the HIP runtime (`libamdhip64.so`): the public types the
//! FFN path uses keep their names and method signatures (`Cuda` is kept as an alias of `Hip`, so `use crate::hip as cuda;`
//! is the whole change at the call sites), the entry points are the HIP runtime's.
//!
//! Covered (what `src/ffn.rs:52-84, 340-413, 1007-1124`, `src/moe.rs:286-372, 584-595, 972-1289`,
//! `src/expert_packing.rs:46-259` and `src/probe.rs:1527-1542` call): `open`, `allocate` / `allocate_rows`, `Buffer::{ptr,
//! len, upload, download, zero, view}`, `stream` / `auxiliary_stream` / `hint_stream`, `Stream::{raw, synchronize, capture}`,
//! `Event::{record, wait, synchronize, elapsed_since}`, `fence_event` / `event`, `module`, `Module::function`,
//! `Function::{launch, handle}`, `Graph::launch`, `capturing`, `capture_serial`, `copy_device`, `zero_device`, `owns_buffer`.
//! Not carried over, on purpose: graph node surgery (`graph_swap`, re-gridding: `src/cuda.rs:2154-2347`; the native
//! front-end is in the graph from the start), virtual-memory reservations, programmatic dependent launch, shared-memory
//! carve-out attributes, stream priorities (every stream stays at the default priority).
//!
//! This source has not been compiled: the build image of the kernel library has no Rust toolchain.  The C++ host mirror
//! (`titanic-flash-41_amd/host/hip_rt.hpp`, `ffn_host.cpp`) makes the same runtime calls in the same order and is what
//! the GPU tests run.
#![allow(dead_code)]
use anyhow::{anyhow, ensure, Context as _, Result};
use libloading::Library;
use std::cell::{Cell, RefCell};
use std::ffi::{c_char, c_int, c_uint, c_void, CStr, CString};
use std::marker::PhantomData;
use std::ptr;
use std::rc::{Rc, Weak};

type Handle = *mut c_void;
type HipResult = c_int; // 0 = hipSuccess

macro_rules! api {
    ($($field:ident : $ty:ty = $sym:literal;)+) => {
        struct Api { _library: Library, $($field: $ty,)+ }
        impl Api {
            unsafe fn load() -> Result<Self> {
                let lib = unsafe { Library::new("libamdhip64.so") }.context("load the HIP runtime")?;
                $(let $field: $ty = *unsafe { lib.get(concat!($sym, "\0").as_bytes()) }.with_context(|| concat!("HIP runtime symbol ", $sym))?;)+
                Ok(Self { _library: lib, $($field,)+ })
            }
        }
    };
}
api! {
    init: unsafe extern "C" fn(c_uint) -> HipResult = "hipInit";
    device_count: unsafe extern "C" fn(*mut c_int) -> HipResult = "hipGetDeviceCount";
    device_attribute: unsafe extern "C" fn(*mut c_int, c_int, c_int) -> HipResult = "hipDeviceGetAttribute";
    set_device: unsafe extern "C" fn(c_int) -> HipResult = "hipSetDevice";
    device_sync: unsafe extern "C" fn() -> HipResult = "hipDeviceSynchronize";
    alloc: unsafe extern "C" fn(*mut u64, usize) -> HipResult = "hipMalloc";
    free: unsafe extern "C" fn(u64) -> HipResult = "hipFree";
    mem_info: unsafe extern "C" fn(*mut usize, *mut usize) -> HipResult = "hipMemGetInfo";
    memset: unsafe extern "C" fn(u64, c_int, usize) -> HipResult = "hipMemset";
    memset_async: unsafe extern "C" fn(u64, c_int, usize, Handle) -> HipResult = "hipMemsetAsync";
    memcpy: unsafe extern "C" fn(*mut c_void, *const c_void, usize, c_int) -> HipResult = "hipMemcpy";
    memcpy_async: unsafe extern "C" fn(*mut c_void, *const c_void, usize, c_int, Handle) -> HipResult = "hipMemcpyAsync";
    stream_create: unsafe extern "C" fn(*mut Handle, c_uint) -> HipResult = "hipStreamCreateWithFlags";
    stream_destroy: unsafe extern "C" fn(Handle) -> HipResult = "hipStreamDestroy";
    stream_sync: unsafe extern "C" fn(Handle) -> HipResult = "hipStreamSynchronize";
    stream_wait_event: unsafe extern "C" fn(Handle, Handle, c_uint) -> HipResult = "hipStreamWaitEvent";
    module_load: unsafe extern "C" fn(*mut Handle, *const c_void) -> HipResult = "hipModuleLoadData";
    module_unload: unsafe extern "C" fn(Handle) -> HipResult = "hipModuleUnload";
    get_function: unsafe extern "C" fn(*mut Handle, Handle, *const c_char) -> HipResult = "hipModuleGetFunction";
    launch: unsafe extern "C" fn(Handle, c_uint, c_uint, c_uint, c_uint, c_uint, c_uint, c_uint, Handle, *mut *mut c_void, *mut *mut c_void) -> HipResult = "hipModuleLaunchKernel";
    error_string: unsafe extern "C" fn(HipResult) -> *const c_char = "hipGetErrorString";
    event_create: unsafe extern "C" fn(*mut Handle, c_uint) -> HipResult = "hipEventCreateWithFlags";
    event_destroy: unsafe extern "C" fn(Handle) -> HipResult = "hipEventDestroy";
    event_record: unsafe extern "C" fn(Handle, Handle) -> HipResult = "hipEventRecord";
    event_sync: unsafe extern "C" fn(Handle) -> HipResult = "hipEventSynchronize";
    event_elapsed: unsafe extern "C" fn(*mut f32, Handle, Handle) -> HipResult = "hipEventElapsedTime";
    capture_begin: unsafe extern "C" fn(Handle, c_int) -> HipResult = "hipStreamBeginCapture";
    capture_end: unsafe extern "C" fn(Handle, *mut Handle) -> HipResult = "hipStreamEndCapture";
    graph_instantiate: unsafe extern "C" fn(*mut Handle, Handle, u64) -> HipResult = "hipGraphInstantiateWithFlags";
    graph_destroy: unsafe extern "C" fn(Handle) -> HipResult = "hipGraphDestroy";
    exec_destroy: unsafe extern "C" fn(Handle) -> HipResult = "hipGraphExecDestroy";
    graph_launch: unsafe extern "C" fn(Handle, Handle) -> HipResult = "hipGraphLaunch";
}
const MEMCPY_HOST_TO_DEVICE: c_int = 1;
const MEMCPY_DEVICE_TO_HOST: c_int = 2;
const MEMCPY_DEVICE_TO_DEVICE: c_int = 3;
const STREAM_NON_BLOCKING: c_uint = 1;
const EVENT_TIMING: c_uint = 0;
const EVENT_DISABLE_TIMING: c_uint = 2;
const CAPTURE_MODE_THREAD_LOCAL: c_int = 1;
const ATTRIBUTE_MULTIPROCESSOR_COUNT: c_int = 63;

impl Api {
    fn check(&self, status: HipResult, what: &str) -> Result<()> {
        if status == 0 {
            return Ok(());
        }
        let text = unsafe {
            let p = (self.error_string)(status);
            if p.is_null() { "unknown".into() } else { CStr::from_ptr(p).to_string_lossy().into_owned() }
        };
        Err(anyhow!("{what}: HIP error {status} ({text})"))
    }
}

thread_local! {
    static CAPTURE_DEPTH: Cell<usize> = const { Cell::new(0) };
    static CAPTURE_SERIAL: Cell<u64> = const { Cell::new(0) };
}
/// Advances at every `Stream::capture` begin on this thread (same meaning as `cuda::capture_serial`).
pub(crate) fn capture_serial() -> u64 { CAPTURE_SERIAL.with(|s| s.get()) }
/// Whether this thread is inside exactly one `Stream::capture` body.
pub(crate) fn capturing() -> bool { CAPTURE_DEPTH.with(|d| d.get() == 1) }

/// One device, one OS thread: every handle below stays on the thread that opened it (`Rc`, not `Send`), as in `cuda.rs`.
struct Owner {
    api: Api,
    device: c_int,
    compute_units: c_int,
    auxiliary: RefCell<Option<(usize, Weak<Stream>)>>,
    hints: RefCell<Option<(usize, Weak<Stream>)>>,
    allocations: RefCell<Vec<(u64, usize)>>,
}
impl Owner {
    fn current(&self) -> Result<()> { self.api.check(unsafe { (self.api.set_device)(self.device) }, "select device") }
}
#[derive(Clone)]
pub struct Hip { owner: Rc<Owner> }
pub type Cuda = Hip;

impl Hip {
    pub fn open(device: usize) -> Result<Self> {
        let api = unsafe { Api::load() }?;
        api.check(unsafe { (api.init)(0) }, "initialise HIP")?;
        let mut count = 0;
        api.check(unsafe { (api.device_count)(&mut count) }, "count devices")?;
        ensure!((device as c_int) < count, "HIP device {device} of {count}");
        api.check(unsafe { (api.set_device)(device as c_int) }, "select device")?;
        let mut compute_units = 0;
        api.check(unsafe { (api.device_attribute)(&mut compute_units, ATTRIBUTE_MULTIPROCESSOR_COUNT, device as c_int) }, "compute unit count")?;
        Ok(Self { owner: Rc::new(Owner { api, device: device as c_int, compute_units, auxiliary: RefCell::new(None), hints: RefCell::new(None),
            allocations: RefCell::new(Vec::new()) }) })
    }
    /// 256 on MI355X; what `native.json`'s `physical_cus` is checked against (`physical_sms == 48` in the reference, `src/ffn.rs:71-74`).
    pub fn compute_units(&self) -> usize { self.owner.compute_units as usize }
    pub fn allocate<T: Copy>(&self, len: usize) -> Result<Buffer<T>> {
        ensure!(len > 0, "empty device allocation");
        self.owner.current()?;
        let bytes = len.checked_mul(std::mem::size_of::<T>()).context("allocation size")?;
        let mut ptr = 0u64;
        self.owner.api.check(unsafe { (self.owner.api.alloc)(&mut ptr, bytes) }, "allocate device memory")?;
        self.owner.allocations.borrow_mut().push((ptr, bytes));
        Ok(Buffer { owner: self.owner.clone(), ptr, len, owned: true, _marker: PhantomData })
    }
    /// Row buffers of the decode / verify profiles (`Cuda::allocate_rows`): the same allocation, kept as a separate name.
    pub fn allocate_rows<T: Copy>(&self, len: usize) -> Result<Buffer<T>> { self.allocate(len) }
    pub fn owns_buffer<T>(&self, buffer: &Buffer<T>) -> bool { Rc::ptr_eq(&self.owner, &buffer.owner) }
    pub fn owns_stream(&self, stream: &Stream) -> bool { Rc::ptr_eq(&self.owner, &stream.owner) }
    pub fn stream(&self) -> Result<Stream> {
        self.owner.current()?;
        let mut raw = ptr::null_mut();
        // default priority: streams of different priorities are not used on this part
        self.owner.api.check(unsafe { (self.owner.api.stream_create)(&mut raw, STREAM_NON_BLOCKING) }, "create nonblocking stream")?;
        Ok(Stream { owner: self.owner.clone(), raw })
    }
    /// The shared expert's branch beside the routed experts (`src/ffn.rs:518-522, 1007-1036`): one per parent stream.
    pub(crate) fn auxiliary_stream(&self, parent: &Stream) -> Result<Rc<Stream>> { self.cached(parent, &self.owner.auxiliary) }
    /// The expert-weight prefetch window (`ca_expert_prefetch`) runs on a stream of its own beside both.
    pub(crate) fn hint_stream(&self, parent: &Stream) -> Result<Rc<Stream>> { self.cached(parent, &self.owner.hints) }
    fn cached(&self, parent: &Stream, cache: &RefCell<Option<(usize, Weak<Stream>)>>) -> Result<Rc<Stream>> {
        ensure!(self.owns_stream(parent), "auxiliary parent context");
        if let Some((bound, weak)) = cache.borrow().as_ref() {
            if let Some(stream) = weak.upgrade() {
                ensure!(*bound == parent.raw() as usize, "auxiliary stream requires one ordered parent");
                return Ok(stream);
            }
        }
        let stream = Rc::new(self.stream()?);
        *cache.borrow_mut() = Some((parent.raw() as usize, Rc::downgrade(&stream)));
        Ok(stream)
    }
    pub fn event(&self) -> Result<Event> { self.make_event(EVENT_TIMING, "create timing event") }
    pub(crate) fn fence_event(&self) -> Result<Event> { self.make_event(EVENT_DISABLE_TIMING, "create dependency event") }
    fn make_event(&self, flags: c_uint, what: &str) -> Result<Event> {
        self.owner.current()?;
        let mut raw = ptr::null_mut();
        self.owner.api.check(unsafe { (self.owner.api.event_create)(&mut raw, flags) }, what)?;
        Ok(Event { owner: self.owner.clone(), raw })
    }
    /// `artifact`: the bytes of a code object (`titanic_moe_gfx950.hsaco`, `titanic_moe_gfx950_reference_layer.hsaco`).
    pub fn module(&self, artifact: &[u8]) -> Result<Module> {
        ensure!(!artifact.is_empty(), "empty kernel artifact");
        self.owner.current()?;
        let mut raw = ptr::null_mut();
        self.owner.api.check(unsafe { (self.owner.api.module_load)(&mut raw, artifact.as_ptr().cast()) }, "load code object")?;
        Ok(Module { inner: Rc::new(ModuleOwner { owner: self.owner.clone(), raw }) })
    }
    pub fn copy_device<T: Copy>(&self, from: &Buffer<T>, to: &mut Buffer<T>, stream: &Stream) -> Result<()> {
        ensure!(from.len == to.len && self.owns_buffer(from) && self.owns_buffer(to), "device copy shape/context");
        self.owner.api.check(unsafe { (self.owner.api.memcpy_async)(to.ptr as *mut c_void, from.ptr as *const c_void, from.bytes(), MEMCPY_DEVICE_TO_DEVICE, stream.raw) },
            "device copy")
    }
    /// Outside captures only: inside a capture a fill kernel clears memory (memset nodes are not recorded into graphs here).
    pub fn zero_device<T: Copy>(&self, buffer: &mut Buffer<T>, stream: &Stream) -> Result<()> {
        ensure!(!capturing(), "memset inside a capture: use the library's fill kernel");
        self.owner.api.check(unsafe { (self.owner.api.memset_async)(buffer.ptr, 0, buffer.bytes(), stream.raw) }, "zero device memory")
    }
    pub fn synchronize(&self) -> Result<()> { self.owner.api.check(unsafe { (self.owner.api.device_sync)() }, "device synchronize") }
}

/// Device memory owned by the host code (the native library never allocates or frees: `include/titanic_moe.h`).
pub struct Buffer<T> { owner: Rc<Owner>, ptr: u64, len: usize, owned: bool, _marker: PhantomData<T> }
impl<T: Copy> Buffer<T> {
    pub fn ptr(&self) -> u64 { self.ptr }
    pub fn len(&self) -> usize { self.len }
    pub fn is_empty(&self) -> bool { self.len == 0 }
    fn bytes(&self) -> usize { self.len * std::mem::size_of::<T>() }
    pub fn upload(&mut self, host: &[T]) -> Result<()> {
        ensure!(host.len() == self.len, "upload length");
        self.owner.current()?;
        self.owner.api.check(unsafe { (self.owner.api.memcpy)(self.ptr as *mut c_void, host.as_ptr().cast(), self.bytes(), MEMCPY_HOST_TO_DEVICE) }, "upload")
    }
    pub fn download(&self) -> Result<Vec<T>> {
        self.owner.current()?;
        let mut host = Vec::<T>::with_capacity(self.len);
        self.owner.api.check(unsafe { (self.owner.api.memcpy)(host.as_mut_ptr().cast(), self.ptr as *const c_void, self.bytes(), MEMCPY_DEVICE_TO_HOST) }, "download")?;
        unsafe { host.set_len(self.len) };
        Ok(host)
    }
    pub fn zero(&mut self) -> Result<()> {
        self.owner.current()?;
        self.owner.api.check(unsafe { (self.owner.api.memset)(self.ptr, 0, self.bytes()) }, "zero")
    }
    /// Safety: the view must not outlive `self` and must not be written through while `self` is read elsewhere.
    pub unsafe fn view(&self, first: usize, len: usize) -> Result<Buffer<T>> {
        ensure!(first.checked_add(len).is_some_and(|end| end <= self.len) && len > 0, "device view range");
        Ok(Buffer { owner: self.owner.clone(), ptr: self.ptr + (first * std::mem::size_of::<T>()) as u64, len, owned: false, _marker: PhantomData })
    }
}
impl<T> Drop for Buffer<T> {
    fn drop(&mut self) {
        if self.owned {
            let _ = self.owner.current();
            unsafe { (self.owner.api.free)(self.ptr) };
            self.owner.allocations.borrow_mut().retain(|(p, _)| *p != self.ptr);
        }
    }
}

pub struct Stream { owner: Rc<Owner>, raw: Handle }
impl Stream {
    pub fn raw(&self) -> Handle { self.raw }
    pub fn synchronize(&self) -> Result<()> { self.owner.api.check(unsafe { (self.owner.api.stream_sync)(self.raw) }, "stream synchronize") }
    /// Records everything `body` enqueues on this stream (and on streams forked from it with events) into a graph.
    pub fn capture(&self, body: impl FnOnce() -> Result<()>) -> Result<Graph> {
        self.owner.current()?;
        self.owner.api.check(unsafe { (self.owner.api.capture_begin)(self.raw, CAPTURE_MODE_THREAD_LOCAL) }, "begin capture")?;
        CAPTURE_DEPTH.with(|d| d.set(d.get() + 1));
        CAPTURE_SERIAL.with(|s| s.set(s.get() + 1));
        let outcome = body();
        CAPTURE_DEPTH.with(|d| d.set(d.get() - 1));
        let mut graph = ptr::null_mut();
        let ended = self.owner.api.check(unsafe { (self.owner.api.capture_end)(self.raw, &mut graph) }, "end capture");
        outcome?;
        ended?;
        let mut exec = ptr::null_mut();
        let made = self.owner.api.check(unsafe { (self.owner.api.graph_instantiate)(&mut exec, graph, 0) }, "instantiate graph");
        unsafe { (self.owner.api.graph_destroy)(graph) };
        made?;
        Ok(Graph { owner: self.owner.clone(), exec })
    }
}
impl Drop for Stream {
    fn drop(&mut self) { unsafe { (self.owner.api.stream_destroy)(self.raw) }; }
}

pub struct Event { owner: Rc<Owner>, raw: Handle }
impl Event {
    pub fn record(&self, stream: &Stream) -> Result<()> { self.owner.api.check(unsafe { (self.owner.api.event_record)(self.raw, stream.raw) }, "record event") }
    /// Makes `stream` wait for this event (a fork or a join between the layer's streams).
    pub fn wait(&self, stream: &Stream) -> Result<()> { self.owner.api.check(unsafe { (self.owner.api.stream_wait_event)(stream.raw, self.raw, 0) }, "wait for event") }
    pub fn synchronize(&self) -> Result<()> { self.owner.api.check(unsafe { (self.owner.api.event_sync)(self.raw) }, "event synchronize") }
    pub fn elapsed_since(&self, begin: &Event) -> Result<f32> {
        let mut ms = 0f32;
        self.owner.api.check(unsafe { (self.owner.api.event_elapsed)(&mut ms, begin.raw, self.raw) }, "elapsed time")?;
        Ok(ms)
    }
}
impl Drop for Event {
    fn drop(&mut self) { unsafe { (self.owner.api.event_destroy)(self.raw) }; }
}

struct ModuleOwner { owner: Rc<Owner>, raw: Handle }
impl Drop for ModuleOwner {
    fn drop(&mut self) { unsafe { (self.owner.api.module_unload)(self.raw) }; }
}
#[derive(Clone)]
pub struct Module { inner: Rc<ModuleOwner> }
impl Module {
    pub fn function(&self, name: &str) -> Result<Function> {
        let symbol = CString::new(name)?;
        let mut raw = ptr::null_mut();
        let api = &self.inner.owner.api;
        api.check(unsafe { (api.get_function)(&mut raw, self.inner.raw, symbol.as_ptr()) }, &format!("resolve kernel {name}"))?;
        Ok(Function { module: self.inner.clone(), raw })
    }
}
pub struct Function { module: Rc<ModuleOwner>, raw: Handle }
impl Function {
    pub fn handle(&self) -> usize { self.raw as usize }
    /// Safety: `args` point at values of the kernel's parameter types, in order; buffers outlive the launch.
    /// Blocks are whole wavefronts of 64 lanes on this part: a launch width taken from a 32-lane manifest is `64 * waves`.
    pub unsafe fn launch(&self, grid: [u32; 3], block: [u32; 3], shared: u32, stream: &Stream, args: &mut [*mut c_void]) -> Result<()> {
        let api = &self.module.owner.api;
        api.check(unsafe { (api.launch)(self.raw, grid[0], grid[1], grid[2], block[0], block[1], block[2], shared, stream.raw, args.as_mut_ptr(), ptr::null_mut()) },
            "launch kernel")
    }
    /// LDS is not traded against cache on this part: nothing to opt into (kept for the call sites).
    pub fn opt_in_shared_memory(&self, _bytes: u32) -> Result<()> { Ok(()) }
}

pub struct Graph { owner: Rc<Owner>, exec: Handle }
impl Graph {
    pub fn launch(&self, stream: &Stream) -> Result<()> { self.owner.api.check(unsafe { (self.owner.api.graph_launch)(self.exec, stream.raw) }, "launch graph") }
}
impl Drop for Graph {
    fn drop(&mut self) { unsafe { (self.owner.api.exec_destroy)(self.exec) }; }
}
