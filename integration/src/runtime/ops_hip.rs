//! `HIP` device for AMD Instinct MI355X (gfx950): the counterpart of `ops_cuda.rs`, bound to
//! `libarhip.so` (C ABI in `include/arhip.h`) with `libloading`.
//!
//! This file is shipped as source for the reference's maintainers; it is written against the
//! reference's own traits (`BackendAllocator`, `Comp`, `Prog`, `Compiled`,
//! `src/runtime/device.rs:39-62,239-251,295-311`) and mirrors the composition of the CUDA
//! device (`src/runtime/ops_cuda.rs:1132-1169`).  It was not compiled in the environment that
//! produced the library (no Rust toolchain there); the same entry points are exercised through
//! ctypes and through a C++ restatement of this layer in that repository's tests.
//!
//! What runs on this device: hand-written host kernels (`Compiled::run_host_kernel`), i.e. the
//! fused attention kernels of `hip_flash.rs`.  The "source" of such a kernel is the path of a
//! prebuilt gfx950 code object (`attn_kernels.hsaco`); "compiling" it means reading the file.
//! There is no uop renderer for HIP in this change: generated kernels keep running on the
//! device they run on today.

use std::cell::RefCell;
use std::ffi::{c_char, c_int, c_uint, c_void, CStr, CString};
use std::rc::Rc;

use libloading::Library;

use crate::runtime::buffer::OpaqueT;
use crate::runtime::device::{
    register_device, register_device_family, BackendAllocator, Comp, Compiled, LruAllocator,
    MemoryInfo, Prog, TinyElf,
};

/// `ARHIP_EUNSUPPORTED`: a capability gap, never a panic (the dispatcher returns `None`).
pub const EUNSUPPORTED: c_int = -2;

type FnLastError = unsafe extern "C" fn() -> *const c_char;
type FnDeviceCount = unsafe extern "C" fn(*mut c_int) -> c_int;
type FnOpen = unsafe extern "C" fn(c_int, *mut *mut c_void) -> c_int;
type FnClose = unsafe extern "C" fn(*mut c_void) -> c_int;
type FnArch = unsafe extern "C" fn(*mut c_void) -> *const c_char;
type FnCus = unsafe extern "C" fn(*mut c_void) -> c_int;
type FnAlloc = unsafe extern "C" fn(*mut c_void, usize, *mut *mut c_void) -> c_int;
type FnFree = unsafe extern "C" fn(*mut c_void, *mut c_void) -> c_int;
type FnCopyIn = unsafe extern "C" fn(*mut c_void, *mut c_void, *const c_void, usize) -> c_int;
type FnCopyOut = unsafe extern "C" fn(*mut c_void, *mut c_void, *const c_void, usize) -> c_int;
type FnCopyD2D = unsafe extern "C" fn(*mut c_void, *mut c_void, *const c_void, usize) -> c_int;
type FnMemInfo = unsafe extern "C" fn(*mut c_void, *mut usize, *mut usize) -> c_int;
type FnSync = unsafe extern "C" fn(*mut c_void) -> c_int;
type FnModuleLoad = unsafe extern "C" fn(*mut c_void, *const c_void, usize, *mut *mut c_void) -> c_int;
type FnLaunch = unsafe extern "C" fn(
    *mut c_void,      // device
    *mut c_void,      // module
    *const c_char,    // entry point
    *const c_uint,    // grid[3], in workgroups
    *const c_uint,    // block[3]
    *const *mut c_void, // buffers
    c_int,
    *const i64,       // scalars
    *const c_int,     // their widths in bits (32 / 64)
    c_int,
    c_int,            // wait
    *mut f64,         // elapsed seconds when wait
) -> c_int;

/// The loaded library and one open device (one stream, default priority).
pub struct HipInner {
    lib: Library,
    dev: *mut c_void,
    /// "gfx950"
    pub arch: String,
    /// compute units (256 on MI355X): the dispatcher sizes its grids against it
    pub compute_units: i64,
}

impl HipInner {
    fn sym<T: Copy>(&self, name: &[u8]) -> T {
        unsafe { *self.lib.get::<T>(name).unwrap_or_else(|e| panic!("TGERR: libarhip: {e}")) }
    }

    /// Panics with the library's message unless `rc` is success; `EUNSUPPORTED` is the caller's
    /// business (AGENTS.md: capability gaps are never panics).
    pub fn check(&self, rc: c_int) {
        if rc != 0 {
            let msg = unsafe { CStr::from_ptr(self.sym::<FnLastError>(b"arhip_last_error")()) };
            panic!("TGERR: arhip {rc}: {}", msg.to_string_lossy());
        }
    }

    /// `HIP` / `HIP:N` -> ordinal N (`ops_cuda.rs:140-174`).
    pub fn open(name: &str) -> HipInner {
        let ordinal: c_int = name.split(':').nth(1).and_then(|s| s.parse().ok()).unwrap_or(0);
        let lib = unsafe { Library::new("libarhip.so") }
            .unwrap_or_else(|e| panic!("TGERR: cannot load libarhip.so: {e}"));
        let mut dev = std::ptr::null_mut();
        let open: FnOpen = unsafe { *lib.get::<FnOpen>(b"arhip_open").expect("arhip_open") };
        let rc = unsafe { open(ordinal, &mut dev) };
        let mut me = HipInner { lib, dev, arch: String::new(), compute_units: 0 };
        me.check(rc);
        me.arch = unsafe { CStr::from_ptr(me.sym::<FnArch>(b"arhip_arch")(dev)) }
            .to_string_lossy()
            .into_owned();
        me.compute_units = unsafe { me.sym::<FnCus>(b"arhip_compute_units")(dev) } as i64;
        me
    }
}

impl Drop for HipInner {
    fn drop(&mut self) {
        unsafe { self.sym::<FnClose>(b"arhip_close")(self.dev) };
    }
}

/// Number of usable gfx950 devices; 0 when the library or the driver is absent
/// (`ops_cuda.rs:1118-1129`).
pub fn device_count() -> usize {
    let Ok(lib) = (unsafe { Library::new("libarhip.so") }) else { return 0 };
    let Ok(f) = (unsafe { lib.get::<FnDeviceCount>(b"arhip_device_count") }) else { return 0 };
    let mut n: c_int = 0;
    unsafe { f(&mut n) };
    n.max(0) as usize
}

/// Device memory window: base pointer, byte offset, size.  Views share the base
/// (`ops_cuda.rs:595-621`).
pub struct HipOpaque {
    base: *mut c_void,
    offset: usize,
    size: usize,
    id: u64,
}

impl HipOpaque {
    /// The device address kernels receive.
    pub fn ptr(&self) -> *mut c_void {
        (self.base as usize + self.offset) as *mut c_void
    }
}

impl OpaqueT for HipOpaque {
    fn size(&self) -> usize {
        self.size
    }
    fn storage_id(&self) -> u64 {
        self.id
    }
    fn as_any(&self) -> &dyn std::any::Any {
        self
    }
}

fn hip_of(o: &dyn OpaqueT) -> &HipOpaque {
    o.as_any().downcast_ref::<HipOpaque>().unwrap_or_else(|| panic!("TGERR: buffer is not on a HIP device"))
}

/// `BackendAllocator` over `arhip_alloc` & co.; wrapped in `LruAllocator` like every device
/// (`device.rs:128-203`).
pub struct HipAllocator {
    inner: Rc<HipInner>,
    next_id: std::cell::Cell<u64>,
}

impl BackendAllocator for HipAllocator {
    fn _alloc(&self, size: usize) -> Rc<dyn OpaqueT> {
        let mut p = std::ptr::null_mut();
        self.inner.check(unsafe { self.inner.sym::<FnAlloc>(b"arhip_alloc")(self.inner.dev, size, &mut p) });
        let id = self.next_id.get();
        self.next_id.set(id + 1);
        Rc::new(HipOpaque { base: p, offset: 0, size, id })
    }
    fn _free(&self, o: Rc<dyn OpaqueT>) {
        let h = hip_of(&*o);
        if h.offset == 0 {
            self.inner.check(unsafe { self.inner.sym::<FnFree>(b"arhip_free")(self.inner.dev, h.base) });
        }
    }
    fn _copyin(&self, dest: &dyn OpaqueT, src: &[u8]) {
        let d = hip_of(dest);
        self.inner.check(unsafe {
            self.inner.sym::<FnCopyIn>(b"arhip_copyin")(self.inner.dev, d.ptr(), src.as_ptr() as *const c_void, src.len())
        });
    }
    fn _copyout(&self, dest: &mut [u8], src: &dyn OpaqueT) {
        // syncs the stream first, like `ops_cuda.rs:662-667`
        let s = hip_of(src);
        self.inner.check(unsafe {
            self.inner.sym::<FnCopyOut>(b"arhip_copyout")(self.inner.dev, dest.as_mut_ptr() as *mut c_void, s.ptr(), dest.len())
        });
    }
    fn _offset(&self, buf: &dyn OpaqueT, size: usize, offset: usize) -> Rc<dyn OpaqueT> {
        let b = hip_of(buf);
        Rc::new(HipOpaque { base: b.base, offset: b.offset + offset, size, id: b.id })
    }
    fn _copy_into(&self, dest: &dyn OpaqueT, src: &dyn OpaqueT) {
        // asynchronous on the device's stream, no sync (`ops_cuda.rs:668-685`)
        let (d, s) = (hip_of(dest), hip_of(src));
        self.inner.check(unsafe {
            self.inner.sym::<FnCopyD2D>(b"arhip_copy_d2d")(self.inner.dev, d.ptr(), s.ptr(), s.size.min(d.size))
        });
    }
    fn memory_info(&self) -> Option<MemoryInfo> {
        let (mut free, mut total) = (0usize, 0usize);
        let rc = unsafe { self.inner.sym::<FnMemInfo>(b"arhip_mem_info")(self.inner.dev, &mut free, &mut total) };
        (rc == 0).then_some(MemoryInfo { free, total })
    }
}

/// The "compiler": a host kernel's source is the path of a prebuilt code object; compiling it
/// is reading the file.  The in-memory cache is keyed by the path, as `compile_cached` keys by
/// source text (`ops_cuda.rs:756-771`).
#[derive(Default)]
pub struct HipCompiler {
    cache: RefCell<std::collections::HashMap<String, Vec<u8>>>,
}

impl Comp for HipCompiler {
    fn compile(&self, src: &str) -> Vec<u8> {
        std::fs::read(src).unwrap_or_else(|e| panic!("TGERR: HIP code object {src}: {e}"))
    }
    fn compile_cached(&self, src: &str) -> Vec<u8> {
        if let Some(v) = self.cache.borrow().get(src) {
            return v.clone();
        }
        let v = self.compile(src);
        self.cache.borrow_mut().insert(src.to_string(), v.clone());
        v
    }
}

/// A loaded entry point: `arhip_module_load` (cached by content inside the library) +
/// `arhip_launch`.
pub struct HipProgram {
    inner: Rc<HipInner>,
    module: *mut c_void,
    name: CString,
    signature: Vec<(i64, crate::dtype::DTypeId)>,
    /// Content hash of the code object (FNV-1a), printed by KPROF so that two kernels that share a
    /// name can be told apart (`ops_cuda.rs:873-876`).
    key: u64,
}

/// `AUTORUST_KPROF=1` synchronises after each kernel and prints its name/time (`ops_cuda.rs:879-885`).
fn kprof_enabled() -> bool {
    static ON: std::sync::OnceLock<bool> = std::sync::OnceLock::new();
    *ON.get_or_init(|| crate::helpers::env::get("AUTORUST_KPROF").is_some())
}

impl HipProgram {
    pub fn new(inner: Rc<HipInner>, elf: &TinyElf) -> HipProgram {
        let mut module = std::ptr::null_mut();
        inner.check(unsafe {
            inner.sym::<FnModuleLoad>(b"arhip_module_load")(inner.dev, elf.lib.as_ptr() as *const c_void, elf.lib.len(), &mut module)
        });
        if crate::helpers::env::get_os("AUTORUST_KERNEL_INFO").is_some() {
            eprintln!("[hip] {}: code object of {} bytes loaded for {}", elf.name, elf.lib.len(), inner.arch);
        }
        let key = elf.lib.iter().fold(0xcbf29ce484222325u64, |h, b| (h ^ *b as u64).wrapping_mul(0x100000001b3));
        HipProgram { inner, module, name: CString::new(elf.name.clone()).unwrap(), signature: elf.signature.clone(), key }
    }
}

impl Prog for HipProgram {
    fn call(
        &mut self,
        bufs: &[Rc<dyn OpaqueT>],
        global_size: [usize; 3],
        local_size: Option<[usize; 3]>,
        vals: &[i64],
        wait: bool,
    ) -> Option<f64> {
        // Argument encoding of `CudaProgram::call` (`ops_cuda.rs:943-990`): a slot below
        // `bufs.len()` is that buffer's device pointer, any other slot is
        // `vals[slot - bufs.len()]` narrowed to the width of its dtype.  The library takes the
        // pointers first and the scalars after them, which is the order every host kernel uses.
        let mut ptrs: Vec<*mut c_void> = Vec::new();
        let mut scalars: Vec<i64> = Vec::new();
        let mut bits: Vec<c_int> = Vec::new();
        for (slot, dt) in self.signature.iter() {
            let slot = *slot as usize;
            if slot < bufs.len() {
                assert!(scalars.is_empty(), "TGERR: HIP host kernels take their buffers first");
                ptrs.push(hip_of(&*bufs[slot]).ptr());
            } else {
                scalars.push(vals[slot - bufs.len()]);
                bits.push(match dt.bitsize() {
                    64 => 64,
                    32 => 32,
                    b => panic!("TGERR: HIP val arg bitsize {b}"),
                });
            }
        }
        let ls = local_size.unwrap_or([1, 1, 1]);
        let grid = [global_size[0] as c_uint, global_size[1] as c_uint, global_size[2] as c_uint];
        let block = [ls[0] as c_uint, ls[1] as c_uint, ls[2] as c_uint];
        // KPROF (`ops_cuda.rs:1004-1012`): a launch that would not wait is synchronised and reported
        let kprof = kprof_enabled() && !wait;
        let mut secs = 0f64;
        let rc = unsafe {
            self.inner.sym::<FnLaunch>(b"arhip_launch")(
                self.inner.dev,
                self.module,
                self.name.as_ptr(),
                grid.as_ptr(),
                block.as_ptr(),
                ptrs.as_ptr(),
                ptrs.len() as c_int,
                scalars.as_ptr(),
                bits.as_ptr(),
                scalars.len() as c_int,
                (wait || kprof) as c_int,
                &mut secs,
            )
        };
        self.inner.check(rc);
        if kprof {
            eprintln!("KPROF\t{}\t{secs:.6}\t{:016x}", self.name.to_string_lossy(), self.key);
            return Some(secs);
        }
        wait.then_some(secs)
    }

    fn flush(&mut self) {
        unsafe { self.inner.sym::<FnSync>(b"arhip_sync")(self.inner.dev) };
    }
}

/// A factory for the device named `name` (`HIP` or `HIP:N`), the composition of
/// `ops_cuda.rs:1132-1159` without a uop renderer of its own: generated kernels are not
/// rendered for this device by this change, host kernels are.
fn factory(name: String) -> crate::runtime::device::DeviceFactory {
    Rc::new(move || {
        let inner = Rc::new(HipInner::open(&name));
        let compiler: Rc<dyn Comp> = Rc::new(HipCompiler::default());
        let allocator = LruAllocator::with_backend(Box::new(HipAllocator {
            inner: inner.clone(),
            next_id: std::cell::Cell::new(1),
        }));
        let ctor: crate::runtime::device::RuntimeCtor = {
            let inner = inner.clone();
            Rc::new(move |elf| Rc::new(RefCell::new(HipProgram::new(inner.clone(), elf))))
        };
        // NOTE for the maintainer: `Compiled::new` wants a `UopRenderer`.  This change brings none for
        // HIP; `host_kernels_only_renderer` stands for a renderer whose `render` panics with
        // "TGERR: HIP renders no generated kernels yet" (a few lines next to `CudaUopRenderer`).
        let renderer = crate::runtime::device::host_kernels_only_renderer("HIP");
        Compiled::new(&name, renderer, allocator, compiler, ctor)
    })
}

/// `Device._DeviceMap["HIP"]` + the `HIP:N` family (`ops_cuda.rs:1161-1169`).
pub fn register() {
    if device_count() == 0 {
        return;
    }
    register_device("HIP", factory("HIP".into()));
    register_device_family("HIP", Rc::new(|name| factory(name.to_string())));
}

/// Compute units of the opened device `name`, for grid sizing in the dispatcher.
pub fn compute_units(name: &str) -> i64 {
    thread_local! { static CUS: RefCell<std::collections::HashMap<String, i64>> = RefCell::new(Default::default()); }
    CUS.with(|m| *m.borrow_mut().entry(name.to_string()).or_insert_with(|| HipInner::open(name).compute_units))
}
