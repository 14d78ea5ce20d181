//! Handle of the MI355X (gfx950) backend: the `Gpu` of `handle/cuda/mod.rs`, over `libophip.so`.
//!
//! Everything on the device side (kernels, module loading, kernel choice, workspace planning)
//! lives behind the C ABI declared in [`ffi`]; this module only adapts types:
//! `Hip` / `Stream` / `DevByte` / `DevMem` for [`Hardware`] and [`QueueAlloc`], `TensorLayout` ->
//! `ophip_tensor_layout`, status codes -> `SchemeError` / `LaunchError`, and a macro that writes
//! the `Operator` impl every `<op>/hip/mod.rs` shares.

pub(crate) mod ffi;

use crate::{
    Alloc, Hardware, LaunchError, LaunchErrorKind, QueueAlloc, QueueOf, SchemeError,
    SchemeErrorKind, TensorLayout,
};
use digit_layout::{types as ty, DigitLayout};
use std::{
    cell::RefCell,
    collections::HashMap,
    ffi::{c_void, CStr},
    mem::forget,
    ops::{Deref, DerefMut},
    ptr::null_mut,
    slice::{from_raw_parts, from_raw_parts_mut},
    sync::Arc,
};

/// The hardware handle operators are created on.
pub struct Hip(pub(crate) Arc<Handle>);

pub struct Handle {
    raw: *mut ffi::ophip_device,
}

// The device object is reference counted and thread safe on the C side.
unsafe impl Send for Handle {}
unsafe impl Sync for Handle {}

impl Drop for Handle {
    #[inline]
    fn drop(&mut self) {
        unsafe { ffi::ophip_device_release(self.raw) }
    }
}

impl Handle {
    #[inline]
    pub(crate) fn raw(&self) -> *mut ffi::ophip_device {
        self.raw
    }
}

/// Same knobs as the CUDA backend's `Config`.
#[derive(Clone, Debug)]
pub struct Config {
    pub low_diversity_cache: usize,
    pub medium_diversity_cache: usize,
    pub high_diversity_cache: usize,
}

impl Default for Config {
    fn default() -> Self {
        Self {
            low_diversity_cache: 4,
            medium_diversity_cache: 16,
            high_diversity_cache: 64,
        }
    }
}

/// One byte of device memory; never read or written from the host.
#[repr(transparent)]
pub struct DevByte(#[allow(dead_code)] u8);

impl Hardware for Hip {
    type Byte = DevByte;
    type Queue<'ctx> = Stream<'ctx>;
}

impl Hip {
    /// `None` when the machine has no such device (or no HIP runtime).
    pub fn new(ordinal: i32, config: Config) -> Option<Self> {
        if unsafe { ffi::ophip_device_count() } <= ordinal {
            return None;
        }
        let cfg = ffi::ophip_config {
            low_diversity_cache: config.low_diversity_cache,
            medium_diversity_cache: config.medium_diversity_cache,
            high_diversity_cache: config.high_diversity_cache,
        };
        let mut raw = null_mut();
        match unsafe { ffi::ophip_device_create(ordinal, &cfg, &mut raw) } {
            0 => Some(Self(Arc::new(Handle { raw }))),
            _ => None,
        }
    }

    /// Device 0 with the default configuration; what the tests use.
    #[inline]
    pub fn init() -> Option<Self> {
        Self::new(0, Config::default())
    }

    pub fn info(&self) -> ffi::ophip_device_info {
        let mut info = unsafe { std::mem::zeroed() };
        let status = unsafe { ffi::ophip_device_get_info(self.0.raw, &mut info) };
        assert_eq!(status, 0, "{}", last_error());
        info
    }

    /// A new stream on this device.
    pub fn stream(&self) -> Stream<'_> {
        let mut raw = null_mut();
        let status = unsafe { ffi::ophip_stream_create(self.0.raw, &mut raw) };
        assert_eq!(status, 0, "{}", last_error());
        let mut vtable = ffi::ophip_queue_alloc {
            ctx: null_mut(),
            stream: raw,
            alloc: unreachable_alloc,
            free: unreachable_free,
        };
        let status = unsafe { ffi::ophip_queue_alloc_from_stream(self.0.raw, raw, &mut vtable) };
        assert_eq!(status, 0, "{}", last_error());
        Stream {
            raw,
            vtable,
            hip: self,
        }
    }

    /// Memory that lives until the returned object is dropped (a synchronous allocation).
    pub fn malloc(&self, len: usize) -> DevMem<'_> {
        let mut ptr = null_mut();
        let status = unsafe { ffi::ophip_malloc(self.0.raw, len, &mut ptr) };
        assert_eq!(status, 0, "{}", last_error());
        DevMem {
            ptr: ptr.cast(),
            len,
            hip: self,
        }
    }

    pub fn from_host(&self, data: &[u8], stream: &Stream) -> DevMem<'_> {
        let mem = self.malloc(data.len());
        let status = unsafe {
            ffi::ophip_memcpy_h2d(self.0.raw, mem.ptr.cast(), data.as_ptr().cast(), data.len(), stream.raw)
        };
        assert_eq!(status, 0, "{}", last_error());
        stream.synchronize();
        mem
    }

    pub fn to_host(&self, mem: &[DevByte], out: &mut [u8], stream: &Stream) {
        assert_eq!(mem.len(), out.len());
        let status = unsafe {
            ffi::ophip_memcpy_d2h(self.0.raw, out.as_mut_ptr().cast(), mem.as_ptr().cast(), out.len(), stream.raw)
        };
        assert_eq!(status, 0, "{}", last_error());
        stream.synchronize();
    }
}

extern "C" fn unreachable_alloc(_: *mut c_void, _: usize) -> *mut c_void {
    null_mut()
}
extern "C" fn unreachable_free(_: *mut c_void, _: *mut c_void) {}

/// A HIP stream together with the stream-ordered allocator the library binds to it.
pub struct Stream<'ctx> {
    raw: ffi::ophip_stream,
    vtable: ffi::ophip_queue_alloc,
    hip: &'ctx Hip,
}

impl Stream<'_> {
    #[inline]
    pub fn as_raw(&self) -> ffi::ophip_stream {
        self.raw
    }
    #[inline]
    pub fn hip(&self) -> &Hip {
        self.hip
    }
    pub fn synchronize(&self) {
        let status = unsafe { ffi::ophip_stream_synchronize(self.hip.0.raw, self.raw) };
        assert_eq!(status, 0, "{}", last_error());
    }
}

impl Drop for Stream<'_> {
    fn drop(&mut self) {
        unsafe { ffi::ophip_stream_destroy(self.hip.0.raw, self.raw) };
    }
}

/// Ownership of a range of device memory.
pub struct DevMem<'ctx> {
    ptr: *mut DevByte,
    len: usize,
    hip: &'ctx Hip,
}

impl Deref for DevMem<'_> {
    type Target = [DevByte];
    #[inline]
    fn deref(&self) -> &Self::Target {
        if self.len == 0 {
            &[]
        } else {
            unsafe { from_raw_parts(self.ptr, self.len) }
        }
    }
}

impl DerefMut for DevMem<'_> {
    #[inline]
    fn deref_mut(&mut self) -> &mut Self::Target {
        if self.len == 0 {
            &mut []
        } else {
            unsafe { from_raw_parts_mut(self.ptr, self.len) }
        }
    }
}

impl Drop for DevMem<'_> {
    fn drop(&mut self) {
        if !self.ptr.is_null() {
            unsafe { ffi::ophip_free(self.hip.0.raw, self.ptr.cast()) };
        }
    }
}

/// `impl QueueAlloc for Stream` of `handle/cuda/alloc.rs`: stream-ordered allocation.
impl<'ctx> Alloc<DevMem<'ctx>> for Stream<'ctx> {
    fn alloc(&self, size: usize) -> DevMem<'ctx> {
        let ptr = (self.vtable.alloc)(self.vtable.ctx, size);
        assert!(size == 0 || !ptr.is_null(), "{}", last_error());
        DevMem {
            ptr: ptr.cast(),
            len: size,
            hip: self.hip,
        }
    }

    fn free(&self, mem: DevMem<'ctx>) {
        (self.vtable.free)(self.vtable.ctx, mem.ptr.cast());
        forget(mem)
    }
}

impl<'ctx> QueueAlloc for Stream<'ctx> {
    type Hardware = Hip;
    type DevMem = DevMem<'ctx>;
    #[inline]
    fn queue(&self) -> &QueueOf<Self::Hardware> {
        self
    }
}

// ---------------------------------------------------------------- adapters --

pub(crate) fn last_error() -> String {
    let ptr = unsafe { ffi::ophip_last_error() };
    if ptr.is_null() {
        String::new()
    } else {
        unsafe { CStr::from_ptr(ptr) }.to_string_lossy().into_owned()
    }
}

fn scheme_kind(status: i32) -> Option<SchemeErrorKind> {
    use SchemeErrorKind::*;
    Some(match status {
        1 => TypeNotSupport,
        2 => TypeMismatch,
        3 => RankNotSupport,
        4 => RankMismatch,
        5 => ShapeNotSupport,
        6 => ShapeMismatch,
        7 => StridesNotSupport,
        8 => ArgsNotSupport,
        9 => DynamicNotSupport,
        _ => return None,
    })
}

pub(crate) fn check_scheme(status: i32) -> Result<(), SchemeError> {
    match status {
        0 => Ok(()),
        s => Err(SchemeError {
            // a scheme call cannot fail to execute; keep the closest kind if it ever reports so
            kind: scheme_kind(s).unwrap_or(SchemeErrorKind::ArgsNotSupport),
            info: last_error(),
        }),
    }
}

pub(crate) fn check_launch(status: i32) -> Result<(), LaunchError> {
    match status {
        0 => Ok(()),
        s => Err(LaunchError {
            kind: match scheme_kind(s) {
                Some(kind) => LaunchErrorKind::Scheme(kind),
                None => LaunchErrorKind::ExecutionFailed,
            },
            info: last_error(),
        }),
    }
}

/// `DigitLayout` -> the library's type code; 0 (which every operator rejects) if it has none.
pub(crate) fn dt_code(dt: DigitLayout) -> u64 {
    const TABLE: [(DigitLayout, u64); 13] = [
        (ty::F16, 1),
        (ty::BF16, 2),
        (ty::F32, 3),
        (ty::F64, 4),
        (ty::U8, 5),
        (ty::U16, 6),
        (ty::U32, 7),
        (ty::U64, 8),
        (ty::I8, 9),
        (ty::I16, 10),
        (ty::I32, 11),
        (ty::I64, 12),
        (ty::Bool, 13),
    ];
    if dt == crate::random_sample::KVPair::<()>::LAYOUT {
        return 14;
    }
    TABLE.iter().find(|(d, _)| *d == dt).map_or(0, |(_, c)| *c)
}

/// Borrows a `TensorLayout` for the duration of one call.  `MaybeDyn<T>` is `repr(transparent)` and
/// its dynamic values (`usize::MAX`, `isize::MAX`) are the library's sentinels.
#[inline]
pub(crate) fn layout_of(layout: &TensorLayout) -> ffi::ophip_tensor_layout {
    ffi::ophip_tensor_layout {
        dt: dt_code(layout.dt()),
        ndim: layout.ndim() as _,
        shape: layout.shape().as_ptr().cast(),
        strides: layout.strides().as_ptr().cast(),
    }
}

/// What the vtable's `ctx` points at while a launch runs: the caller's allocator and the blocks it
/// has handed out (the library frees a block before `launch` returns, or never asks for one).
struct Bridge<'a, QA: QueueAlloc<Hardware = Hip>> {
    qa: &'a QA,
    live: RefCell<HashMap<usize, QA::DevMem>>,
}

extern "C" fn bridge_alloc<QA: QueueAlloc<Hardware = Hip>>(ctx: *mut c_void, size: usize) -> *mut c_void {
    let bridge = unsafe { &*ctx.cast::<Bridge<QA>>() };
    let mut mem = bridge.qa.alloc(size);
    let ptr = mem.as_mut_ptr();
    bridge.live.borrow_mut().insert(ptr as usize, mem);
    ptr.cast()
}

extern "C" fn bridge_free<QA: QueueAlloc<Hardware = Hip>>(ctx: *mut c_void, ptr: *mut c_void) {
    let bridge = unsafe { &*ctx.cast::<Bridge<QA>>() };
    if let Some(mem) = bridge.live.borrow_mut().remove(&(ptr as usize)) {
        bridge.qa.free(mem)
    }
}

/// Runs `f` with a C view of `queue_alloc`.
pub(crate) fn with_queue_alloc<QA, T>(queue_alloc: &QA, f: impl FnOnce(&ffi::ophip_queue_alloc) -> T) -> T
where
    QA: QueueAlloc<Hardware = Hip>,
{
    let bridge = Bridge {
        qa: queue_alloc,
        live: RefCell::new(HashMap::new()),
    };
    let vtable = ffi::ophip_queue_alloc {
        ctx: (&bridge as *const Bridge<QA>).cast_mut().cast(),
        stream: queue_alloc.queue().as_raw(),
        alloc: bridge_alloc::<QA>,
        free: bridge_free::<QA>,
    };
    let ans = f(&vtable);
    // the library frees what it allocates before it returns; anything left goes back now
    for (_, mem) in bridge.live.into_inner() {
        queue_alloc.free(mem)
    }
    ans
}

/// Uploads `data` into a fresh block from `queue_alloc` (the helper behind `Rope::build_pos` and
/// `RandomSample::build_indices`).
pub(crate) fn upload<QA>(data: &[u8], queue_alloc: &QA) -> QA::DevMem
where
    QA: QueueAlloc<Hardware = Hip>,
{
    let mut mem = queue_alloc.alloc(data.len());
    let stream = queue_alloc.queue();
    let status = unsafe {
        ffi::ophip_memcpy_h2d(
            stream.hip().0.raw(),
            mem.as_mut_ptr().cast(),
            data.as_ptr().cast(),
            data.len(),
            stream.as_raw(),
        )
    };
    assert_eq!(status, 0, "{}", last_error());
    // `data` may be pageable host memory that the caller drops right away
    stream.synchronize();
    mem
}

/// Writes `pub struct Operator` and its `Operator` / operator-trait impls for one operator.
///
/// ```ignore
/// hip_operator! {
///     RmsNorm, ffi::ophip_rms_norm, ffi::ophip_rms_norm_args,
///     ophip_rms_norm_create, ophip_rms_norm_scheme, ophip_rms_norm_launch, ophip_rms_norm_destroy,
///     |a| ffi::ophip_rms_norm_args { .. };
///     // items of the operator trait (`build_pos`, ...), if it has any
/// }
/// ```
macro_rules! hip_operator {
    ($trait:ident, $raw:ty, $cargs:ty, $create:ident, $scheme:ident, $launch:ident, $destroy:ident,
     |$a:ident| $conv:expr; $($items:item)*) => {
        pub struct Operator {
            raw: *mut $raw,
            _handle: std::sync::Arc<$crate::hip::Handle>,
        }

        // the C object is immutable after `scheme` and `launch` takes it by const pointer
        unsafe impl Send for Operator {}
        unsafe impl Sync for Operator {}

        impl Drop for Operator {
            #[inline]
            fn drop(&mut self) {
                unsafe { $crate::hip::ffi::$destroy(self.raw) }
            }
        }

        impl Operator {
            #[inline]
            fn c_args($a: &Args<$crate::hip::Hip>) -> $cargs {
                $conv
            }
        }

        impl $trait<$crate::hip::Hip> for Operator {
            $($items)*
        }

        impl $crate::Operator for Operator {
            type Hardware = $crate::hip::Hip;
            type TopoNode = $crate::hip::Hip;
            type Args = Args<$crate::hip::Hip>;

            fn new(node: &Self::TopoNode) -> Self {
                let mut raw = std::ptr::null_mut();
                let status = unsafe { $crate::hip::ffi::$create(node.0.raw(), &mut raw) };
                assert_eq!(status, 0, "{}", $crate::hip::last_error());
                Self {
                    raw,
                    _handle: node.0.clone(),
                }
            }

            fn scheme(
                &mut self,
                args: &Self::Args,
                max_workspace_size: usize,
            ) -> Result<usize, $crate::SchemeError> {
                let c = Self::c_args(args);
                let mut workspace = 0;
                $crate::hip::check_scheme(unsafe {
                    $crate::hip::ffi::$scheme(self.raw, &c, max_workspace_size, &mut workspace)
                })?;
                Ok(workspace)
            }

            fn launch<QA>(
                &self,
                args: &Self::Args,
                workspace: &mut [$crate::ByteOf<Self::Hardware>],
                queue_alloc: &QA,
            ) -> Result<(), $crate::LaunchError>
            where
                QA: $crate::QueueAlloc<Hardware = Self::Hardware>,
            {
                let c = Self::c_args(args);
                $crate::hip::with_queue_alloc(queue_alloc, |qa| {
                    $crate::hip::check_launch(unsafe {
                        $crate::hip::ffi::$launch(
                            self.raw,
                            &c,
                            workspace.as_mut_ptr().cast(),
                            workspace.len(),
                            qa,
                        )
                    })
                })
            }
        }
    };
}

pub(crate) use hip_operator;
