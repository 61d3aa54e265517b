//! Minimal HIP backend for fusor on MI355X: it owns device buffers and streams and runs the attention operator
//! through `libfusor_hip` (`fusor-hip-sys`).
//!
//! The types mirror what `fusor_core` offers for WGPU so that `fusor::Tensor` can carry a third variant:
//!   * [`Device`]: adapter + stream + grow-only workspace (reference: `fusor_core::Device`,
//!     fusor-ml/core/src/device.rs:89-354);
//!   * [`HipTensor`]: a shared device buffer plus `{offset, shape, strides}` in elements, the layout contract
//!     `TensorLayoutInfo` already has (fusor-ml/core/src/mir/inputs.rs:164-173, fusor-ml/types/src/layout.rs:88-129);
//!   * [`HipTensor::flash_attention`]: same signature as `fusor_core::Tensor::flash_attention`
//!     (fusor-ml/core/src/composite/flash_attention.rs:28-52), plus `MaskKind::BatchKeyMask` natively;
//!   * [`KvCache`], [`MaskCache`]: device-side counterparts of fusor-ml/fusor/src/cache/{kv_cache,mask_cache}.rs.
//!
//! Failures that are `assert!` panics in the reference (head divisibility, mask shape) panic here with the same
//! text, so `#[should_panic(expected = ...)]` tests keep holding; HIP failures are `Error::Hip`.
use std::ffi::{CStr, c_void};
use std::marker::PhantomData;
use std::ptr;
use std::sync::{Arc, Mutex};

pub use fusor_hip_sys as sys;
use sys::*;

/// Element types the kernels take (reference: `DataTypeEnum`, fusor-ml/core/src/tensor.rs:110-134).
pub trait HipDataType: Copy + 'static {
    const FHIP_DTYPE: fhip_dtype;
}
impl HipDataType for f32 {
    const FHIP_DTYPE: fhip_dtype = FHIP_F32;
}
impl HipDataType for half::f16 {
    const FHIP_DTYPE: fhip_dtype = FHIP_F16;
}
impl HipDataType for half::bf16 {
    const FHIP_DTYPE: fhip_dtype = FHIP_BF16;
}

#[derive(Debug)]
pub enum Error {
    /// A HIP runtime call failed (maps to `fusor::Error::Gpu`).
    Hip(String),
    /// The request is valid but no kernel serves it.
    Unsupported(String),
    /// The workspace is missing or too small.
    Workspace(String),
}
impl std::fmt::Display for Error {
    fn fmt(&self, f: &mut std::fmt::Formatter<'_>) -> std::fmt::Result {
        match self {
            Error::Hip(m) | Error::Unsupported(m) | Error::Workspace(m) => f.write_str(m),
        }
    }
}
impl std::error::Error for Error {}
pub type Result<T> = std::result::Result<T, Error>;

fn last_error() -> String {
    unsafe { CStr::from_ptr(fhip_last_error()) }.to_string_lossy().into_owned()
}

/// Status -> `Result`; what the reference asserts panics with the reference's message.
fn check(status: i32) -> Result<()> {
    match status {
        FHIP_OK => Ok(()),
        FHIP_ERR_INVALID_ARG => panic!("{}", last_error()),
        FHIP_ERR_UNSUPPORTED => Err(Error::Unsupported(last_error())),
        FHIP_ERR_WORKSPACE => Err(Error::Workspace(last_error())),
        _ => Err(Error::Hip(last_error())),
    }
}

struct DeviceInner {
    dev: *mut fhip_device,
    stream: *mut fhip_stream,
    compute_units: i32,
    /// grow-only scratch for split-KV partials, mask intervals and prefill key shares
    workspace: Mutex<(*mut c_void, usize)>,
}
// the library keeps its mutable state in the handles; one stream is used by one thread at a time (the Mutex
// above serialises the attention calls that share the workspace)
unsafe impl Send for DeviceInner {}
unsafe impl Sync for DeviceInner {}
impl Drop for DeviceInner {
    fn drop(&mut self) {
        unsafe {
            fhip_stream_synchronize(self.stream);
            let ws = self.workspace.lock().unwrap();
            if !ws.0.is_null() {
                fhip_free(self.dev, ws.0);
            }
            fhip_stream_destroy(self.stream);
            fhip_device_destroy(self.dev);
        }
    }
}

/// One GPU with one stream of default priority.
#[derive(Clone)]
pub struct Device(Arc<DeviceInner>);

impl Device {
    pub fn new(ordinal: i32) -> Result<Self> {
        unsafe {
            let mut dev = ptr::null_mut();
            check(fhip_device_create(ordinal, &mut dev))?;
            let mut info: fhip_device_info = std::mem::zeroed();
            check(fhip_device_get_info(dev, &mut info))?;
            let mut stream = ptr::null_mut();
            check(fhip_stream_create(dev, &mut stream))?;
            Ok(Device(Arc::new(DeviceInner {
                dev,
                stream,
                compute_units: info.compute_units,
                workspace: Mutex::new((ptr::null_mut(), 0)),
            })))
        }
    }
    pub fn compute_units(&self) -> i32 {
        self.0.compute_units
    }
    pub fn raw(&self) -> *mut fhip_device {
        self.0.dev
    }
    pub fn stream(&self) -> *mut fhip_stream {
        self.0.stream
    }
    pub fn synchronize(&self) -> Result<()> {
        check(unsafe { fhip_stream_synchronize(self.0.stream) })
    }
    pub fn alloc(&self, bytes: usize) -> Result<Arc<Buffer>> {
        let mut p = ptr::null_mut();
        check(unsafe { fhip_malloc(self.0.dev, bytes.max(1), &mut p) })?;
        Ok(Arc::new(Buffer { device: self.clone(), ptr: p, bytes }))
    }
}

/// Device memory, freed when the last tensor that views it goes away.
pub struct Buffer {
    device: Device,
    ptr: *mut c_void,
    bytes: usize,
}
unsafe impl<const R: usize, D: Send> Send for HipTensor<R, D> {}
unsafe impl<const R: usize, D: Sync> Sync for HipTensor<R, D> {}
unsafe impl Send for Buffer {}
unsafe impl Sync for Buffer {}
impl Buffer {
    pub fn ptr(&self) -> *mut c_void {
        self.ptr
    }
    pub fn len(&self) -> usize {
        self.bytes
    }
    pub fn is_empty(&self) -> bool {
        self.bytes == 0
    }
}
impl Drop for Buffer {
    fn drop(&mut self) {
        unsafe {
            // the stream may still read the buffer
            fhip_stream_synchronize(self.device.0.stream);
            fhip_free(self.device.0.dev, self.ptr);
        }
    }
}

impl<D: HipDataType> HipTensor<2, D> {
    /// For a mask tensor whose contents will not change (a block-diagonal or padding mask built once and passed to
    /// every layer of a forward pass): computes its interval table once, so that the attention calls it is passed
    /// to skip their scan of the tensor.
    pub fn with_mask_intervals(mut self) -> Result<Self> {
        let mut bytes = 0usize;
        check(unsafe { fhip_mask_intervals_bytes(self.shape[0] as u32, &mut bytes) })?;
        let table = self.device.alloc(bytes)?;
        let view = self.as_ffi();
        check(unsafe { fhip_mask_intervals(self.device.stream(), &view, D::FHIP_DTYPE, table.ptr(), bytes) })?;
        self.intervals = Some(table);
        Ok(self)
    }
}

/// Describes how to interpret a 2D attention mask (reference: fusor flash_attention.rs:11-19).
#[derive(Debug, Clone, Copy, PartialEq, Eq)]
pub enum MaskKind {
    QKMask,
    BatchKeyMask,
}
impl MaskKind {
    fn ffi(self) -> fhip_mask_kind {
        match self {
            MaskKind::QKMask => FHIP_MASK_QK,
            MaskKind::BatchKeyMask => FHIP_MASK_BATCH_KEY,
        }
    }
}

/// A strided view of rank `R` into a device buffer; offset and strides in elements.
#[derive(Clone)]
pub struct HipTensor<const R: usize, D> {
    device: Device,
    ptr: *mut c_void,
    /// the allocation `ptr` points into; `None` for views into memory a `KvCache` owns
    #[allow(dead_code)]
    keep: Option<Arc<Buffer>>,
    offset: u64,
    shape: [usize; R],
    strides: [i64; R],
    /// Set by `MaskCache::get_mask`: the formula this (mask) tensor was built from.
    analytic: Option<fhip_analytic_mask>,
    /// Set by `with_mask_intervals`: the interval table of this (mask) tensor (`fhip_mask_intervals`).
    intervals: Option<Arc<Buffer>>,
    _elem: PhantomData<D>,
}

fn contiguous_strides<const R: usize>(shape: [usize; R]) -> [i64; R] {
    let mut strides = [0i64; R];
    let mut acc = 1i64;
    for i in (0..R).rev() {
        strides[i] = acc;
        acc *= shape[i] as i64;
    }
    strides
}

impl<const R: usize, D: HipDataType> HipTensor<R, D> {
    /// A fresh tensor whose contents are whatever the allocation holds.
    pub fn uninit(device: &Device, shape: [usize; R]) -> Result<Self> {
        let n: usize = shape.iter().product();
        let buffer = device.alloc(n * std::mem::size_of::<D>())?;
        Ok(HipTensor {
            device: device.clone(),
            ptr: buffer.ptr(),
            keep: Some(buffer),
            offset: 0,
            shape,
            strides: contiguous_strides(shape),
            analytic: None,
            intervals: None,
            _elem: PhantomData,
        })
    }
    /// Upload (reference: `Tensor::new`, fusor-ml/core/src/tensor.rs).
    pub fn from_slice(device: &Device, shape: [usize; R], data: &[D]) -> Result<Self> {
        assert_eq!(data.len(), shape.iter().product::<usize>(), "data length does not match the shape");
        let t = Self::uninit(device, shape)?;
        check(unsafe {
            fhip_memcpy_h2d(device.stream(), t.ptr, data.as_ptr().cast(), std::mem::size_of_val(data))
        })?;
        Ok(t)
    }
    /// Read back a contiguous tensor (reference: `as_slice`, fusor-ml/core/src/tensor.rs:797-896); synchronises.
    pub fn to_vec(&self) -> Result<Vec<D>> {
        assert_eq!(self.strides, contiguous_strides(self.shape), "to_vec needs a contiguous tensor");
        let n: usize = self.shape.iter().product();
        let mut out = Vec::<D>::with_capacity(n);
        let src = unsafe { self.ptr.cast::<D>().add(self.offset as usize) };
        check(unsafe {
            fhip_memcpy_d2h(self.device().stream(), out.as_mut_ptr().cast(), src.cast(), n * std::mem::size_of::<D>())
        })?;
        unsafe { out.set_len(n) };
        Ok(out)
    }
    pub fn device(&self) -> &Device {
        &self.device
    }
    pub fn shape(&self) -> [usize; R] {
        self.shape
    }
    pub fn strides(&self) -> [i64; R] {
        self.strides
    }
    /// A view that swaps two dimensions (no copy).
    pub fn transpose(&self, a: usize, b: usize) -> Self {
        let mut t = self.clone();
        t.shape.swap(a, b);
        t.strides.swap(a, b);
        t
    }
    /// A view of `len` entries of dimension `dim` starting at `start` (no copy).
    pub fn narrow(&self, dim: usize, start: usize, len: usize) -> Self {
        assert!(start + len <= self.shape[dim], "narrow out of range");
        let mut t = self.clone();
        t.offset = (t.offset as i64 + start as i64 * t.strides[dim]) as u64;
        t.shape[dim] = len;
        t
    }
}

impl<D: HipDataType> HipTensor<4, D> {
    pub fn as_ffi(&self) -> fhip_tensor4 {
        fhip_tensor4 {
            ptr: self.ptr,
            offset: self.offset,
            shape: self.shape.map(|x| x as u32),
            stride: self.strides,
        }
    }
    /// A view into memory somebody else owns (a KV cache's rows).
    fn from_ffi(device: &Device, t: &fhip_tensor4) -> Self {
        HipTensor {
            device: device.clone(),
            ptr: t.ptr,
            keep: None,
            offset: t.offset,
            shape: t.shape.map(|x| x as usize),
            strides: t.stride,
            analytic: None,
            intervals: None,
            _elem: PhantomData,
        }
    }

    /// `softmax(q k^T * scale + mask) v` with GQA head mapping `kv_head = head / (H / Hkv)`.
    ///
    /// Same arguments as the reference operator (fusor flash_attention.rs:52-58); the result is a fresh
    /// tensor of Q's shape and type (core flash_attention.rs:505-507).  Asynchronous on the device's stream.
    pub fn flash_attention(
        &self,
        k: &Self,
        v: &Self,
        scale: f32,
        mask: Option<(&HipTensor<2, D>, MaskKind)>,
    ) -> Self {
        let dev = self.device().clone();
        let out = Self::uninit(&dev, self.shape).expect("output allocation");
        let mut a: fhip_attn_args = unsafe { std::mem::zeroed() };
        a.q = self.as_ffi();
        a.k = k.as_ffi();
        a.v = v.as_ffi();
        a.out = out.as_ffi();
        a.dtype = D::FHIP_DTYPE;
        a.out_dtype = D::FHIP_DTYPE;
        a.scale = scale;
        if let Some((m, kind)) = mask {
            match m.analytic {
                // the formula MaskCache attached means exactly this tensor: no tensor read, masked tiles skipped
                Some(desc) if kind == MaskKind::QKMask => a.analytic = desc,
                _ => {
                    a.mask = m.as_ffi();
                    a.mask_kind = kind.ffi();
                    // the table computed once for this mask: the call does not scan the tensor again
                    if let Some(table) = &m.intervals {
                        a.mask_intervals = table.ptr();
                    }
                }
            }
        }
        let mut need = 0usize;
        check(unsafe { fhip_flash_attention_workspace_bytes(&a, dev.compute_units(), &mut need) })
            .expect("workspace query");
        // one call at a time uses the device's workspace
        let mut ws = dev.0.workspace.lock().unwrap();
        if need > ws.1 {
            unsafe {
                if !ws.0.is_null() {
                    fhip_stream_synchronize(dev.stream());
                    fhip_free(dev.raw(), ws.0);
                }
                let mut p = ptr::null_mut();
                check(fhip_malloc(dev.raw(), need, &mut p)).expect("workspace allocation");
                *ws = (p, need);
            }
        }
        a.workspace = ws.0;
        a.workspace_bytes = ws.1;
        check(unsafe { fhip_flash_attention(dev.stream(), &a) }).expect("flash_attention");
        out
    }
}

impl<D: HipDataType> HipTensor<2, D> {
    pub fn as_ffi(&self) -> fhip_tensor2 {
        fhip_tensor2 {
            ptr: self.ptr,
            offset: self.offset,
            shape: self.shape.map(|x| x as u32),
            stride: self.strides,
        }
    }
}

/// Device counterpart of `fusor::cache::MaskCache::get_mask` (fusor-ml/fusor/src/cache/mask_cache.rs:36-86): the
/// tensor is written by a kernel and carries the formula it was built from.
pub struct MaskCache;
impl MaskCache {
    pub fn get_mask<D: HipDataType>(
        device: &Device,
        seq_len: usize,
        seqlen_offset: usize,
        sliding_window_size: Option<usize>,
    ) -> Result<HipTensor<2, D>> {
        let (has_window, window) = match sliding_window_size {
            Some(w) => (1, w as u64),
            None => (0, 0),
        };
        let (mut rows, mut cols) = (0u32, 0u64);
        check(unsafe {
            fhip_mask_get_mask_shape(seq_len as u32, seqlen_offset as u64, has_window, window, &mut rows, &mut cols)
        })?;
        let mut t = HipTensor::<2, D>::uninit(device, [rows as usize, cols as usize])?;
        check(unsafe {
            fhip_mask_get_mask_device(
                device.stream(),
                D::FHIP_DTYPE,
                seq_len as u32,
                seqlen_offset as u64,
                has_window,
                window,
                t.ptr,
            )
        })?;
        let mut desc = fhip_analytic_mask::default();
        check(unsafe { fhip_mask_get_analytic(seq_len as u32, seqlen_offset as u64, has_window, window, &mut desc) })?;
        t.analytic = Some(desc);
        Ok(t)
    }
}

/// Device counterpart of `fusor::cache::KvCache` for `[B, Hkv, seq, D]` tensors concatenated along dim 2
/// (fusor-ml/fusor/src/cache/kv_cache.rs:13-68, tensor_cache.rs:9-124).
pub struct KvCache<D> {
    device: Device,
    raw: *mut fhip_kv_cache,
    _elem: PhantomData<D>,
}
unsafe impl<D> Send for KvCache<D> {}

impl<D: HipDataType> KvCache<D> {
    pub fn new(device: &Device, max_sequence_len: usize) -> Result<Self> {
        let mut raw = ptr::null_mut();
        check(unsafe { fhip_kv_cache_create(device.raw(), D::FHIP_DTYPE, max_sequence_len as u64, &mut raw) })?;
        Ok(KvCache { device: device.clone(), raw, _elem: PhantomData })
    }
    pub fn reset(&mut self) -> Result<()> {
        check(unsafe { fhip_kv_cache_reset(self.raw) })
    }
    pub fn current_seq_len(&self) -> usize {
        let mut n = 0u64;
        unsafe { fhip_kv_cache_current_seq_len(self.raw, &mut n) };
        n as usize
    }
    /// Appends `[B, Hkv, n, D]` rows and returns the cached keys and values including them; the views are valid
    /// until the next append / reset (they die when the cache grows or slides for the first time).
    pub fn append(&mut self, k: &HipTensor<4, D>, v: &HipTensor<4, D>) -> Result<(HipTensor<4, D>, HipTensor<4, D>)> {
        let (kn, vn) = (k.as_ffi(), v.as_ffi());
        let mut k_all: fhip_tensor4 = unsafe { std::mem::zeroed() };
        let mut v_all: fhip_tensor4 = unsafe { std::mem::zeroed() };
        check(unsafe { fhip_kv_cache_append(self.raw, self.device.stream(), &kn, &vn, &mut k_all, &mut v_all) })?;
        Ok((HipTensor::from_ffi(&self.device, &k_all), HipTensor::from_ffi(&self.device, &v_all)))
    }
}
impl<D> Drop for KvCache<D> {
    fn drop(&mut self) {
        unsafe {
            fhip_stream_synchronize(self.device.stream());
            fhip_kv_cache_destroy(self.raw);
        }
    }
}
