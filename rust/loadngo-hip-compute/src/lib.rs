//! GPU compute for local models on AMD Instinct MI355X (gfx950), over liblng_hip.so.
//!
//! The public types keep the names and signatures of `loadngo-metal-compute` for everything the
//! gpt-oss attention path uses (`metal-compute/src/lib.rs:35-53`, `metal-compute/src/apple.rs`), so
//! `gpt-oss/src/gpu.rs` builds against either crate: work is recorded into a [`Batch`] and committed
//! whole; the GPU's completion is delivered as a job on a loadngo proactor together with the buffers
//! the batch owned, so nothing waits on the GPU and the CPU never touches a buffer the GPU may still be
//! writing.
//!
//! What differs, because device memory is not CPU-visible:
//! - the borrows `Buffer::as_bytes` / `as_f32` of metal-compute become copies: [`Buffer::read`], [`Buffer::write`] and their
//!   `f32` forms.
//! - A batch has an element type for its attention and row-copy dispatches ([`Batch::element_type`]):
//!   `F32` (the default: every call then means what it means in metal-compute) or `Bf16` (bf16 in and out,
//!   f32 accumulation; sinks stay f32).
//!
//! Additions without a counterpart in metal-compute are grouped at the end of `impl Batch`.
#![warn(unsafe_op_in_unsafe_fn)]

pub mod ffi;

use std::ffi::{c_void, CStr, CString};
use std::marker::PhantomData;
use std::panic::{catch_unwind, AssertUnwindSafe};
use std::ptr::{self, NonNull};
use std::sync::Arc;
use std::time::Duration;

use loadngo_proactor::{CompletionPort, ProactorHandle};

/// Why a GPU operation could not be set up or did not complete (`metal-compute/src/lib.rs:41-53`).
#[derive(Debug, thiserror::Error)]
pub enum Error {
    #[error("no HIP device")]
    NoDevice,
    #[error("the gfx950 code object did not load: {0}")]
    Compile(String),
    #[error("could not allocate a {0}-byte device buffer")]
    Alloc(usize),
    #[error("invalid dispatch: {0}")]
    Dispatch(String),
    #[error("GPU work failed: {0}")]
    Gpu(String),
}

/// The calling thread's most recent message from the library.
fn last_message() -> String {
    // SAFETY: the library returns a NUL-terminated string that stays valid until this thread's next call.
    unsafe { CStr::from_ptr(ffi::lng_hip_last_error()) }
        .to_string_lossy()
        .into_owned()
}

/// A status of the C ABI as a `Result`; `len` is what an `Alloc` error reports.
fn check_len(rc: i32, len: usize) -> Result<(), Error> {
    match rc {
        ffi::LNG_OK => Ok(()),
        ffi::LNG_ERR_NO_DEVICE => Err(Error::NoDevice),
        ffi::LNG_ERR_COMPILE => Err(Error::Compile(last_message())),
        ffi::LNG_ERR_ALLOC => Err(Error::Alloc(len)),
        ffi::LNG_ERR_DISPATCH => Err(Error::Dispatch(last_message())),
        _ => Err(Error::Gpu(last_message())),
    }
}

fn check(rc: i32) -> Result<(), Error> {
    check_len(rc, 0)
}

/// Whether a batch's dispatches run in order or may overlap (`apple.rs:67-70`). Both record the same
/// thing here: dispatches run in the order recorded, which is a valid execution of either mode.
#[derive(Clone, Copy, Debug, PartialEq, Eq)]
pub enum Dispatch {
    Serial,
    Concurrent,
}

/// Element type of the rows an attention or row-copy dispatch reads and writes.
#[derive(Clone, Copy, Debug, PartialEq, Eq)]
pub enum DType {
    /// The reference's only element type.
    F32 = ffi::LNG_F32 as isize,
    /// The high half of an f32, narrowed to nearest even (`weights/src/dtype.rs:95-116`).
    Bf16 = ffi::LNG_BF16 as isize,
}

impl DType {
    pub const fn size(self) -> usize {
        match self {
            DType::F32 => 4,
            DType::Bf16 => 2,
        }
    }
}

/// One MI355X, its stream and the loaded kernels (`apple.rs:73`).
pub struct Gpu {
    raw: NonNull<ffi::LngGpu>,
}

// SAFETY: the library takes its own locks around allocation, submission and completion; a handle may be
// used from any thread and from several at once.
unsafe impl Send for Gpu {}
unsafe impl Sync for Gpu {}

impl Gpu {
    /// Opens HIP device 0 (`apple.rs:105 Gpu::new`).
    pub fn new() -> Result<Self, Error> {
        Self::on_device(0)
    }

    /// Opens HIP device `device`.
    pub fn on_device(device: i32) -> Result<Self, Error> {
        let mut raw = ptr::null_mut();
        // SAFETY: `raw` is a valid place for the handle.
        check(unsafe { ffi::lng_hip_open(device, &mut raw) })?;
        NonNull::new(raw).map(|raw| Self { raw }).ok_or(Error::NoDevice)
    }

    /// The device's name (`apple.rs:235`).
    pub fn name(&self) -> String {
        let mut text = [0 as std::os::raw::c_char; 256];
        // SAFETY: the library writes at most `text.len()` bytes, NUL-terminated.
        if unsafe { ffi::lng_hip_device_name(self.raw.as_ptr(), text.as_mut_ptr(), text.len()) } != ffi::LNG_OK {
            return String::new();
        }
        // SAFETY: NUL-terminated by the call above.
        unsafe { CStr::from_ptr(text.as_ptr()) }.to_string_lossy().into_owned()
    }

    /// A development switch by its environment name (the header lists them; not part of the interface, no
    /// counterpart in metal-compute). `None` puts the default back. The environment itself is read once, in `new`.
    pub fn debug_set(&self, name: &str, value: Option<&str>) -> Result<(), Error> {
        let name = CString::new(name).map_err(|_| Error::Dispatch("a switch name holds a NUL".into()))?;
        let value = match value {
            Some(v) => Some(CString::new(v).map_err(|_| Error::Dispatch("a switch value holds a NUL".into()))?),
            None => None,
        };
        let value_ptr = value.as_ref().map_or(ptr::null(), |v| v.as_ptr());
        // SAFETY: both strings are NUL-terminated and outlive the call.
        check(unsafe { ffi::lng_hip_debug_set(self.raw.as_ptr(), name.as_ptr(), value_ptr) })
    }

    /// A development counter by name (not part of the interface): waits for submitted work, reads it and resets it.
    pub fn debug_get(&self, name: &str) -> Result<u64, Error> {
        let name = CString::new(name).map_err(|_| Error::Dispatch("a counter name holds a NUL".into()))?;
        let mut value = 0u64;
        // SAFETY: the name is NUL-terminated and `value` is a valid place for the result.
        check(unsafe { ffi::lng_hip_debug_get(self.raw.as_ptr(), name.as_ptr(), &mut value) })?;
        Ok(value)
    }

    /// Device memory of `len` bytes, contents unspecified (`apple.rs:255`). `len == 0` is `Alloc(0)`.
    pub fn buffer(&self, len: usize) -> Result<Buffer, Error> {
        let mut raw = ptr::null_mut();
        // SAFETY: `raw` is a valid place for the handle.
        check_len(unsafe { ffi::lng_hip_buffer(self.raw.as_ptr(), len, &mut raw) }, len)?;
        let raw = NonNull::new(raw).ok_or(Error::Alloc(len))?;
        // SAFETY: plain call on the handle just made.
        let len = unsafe { ffi::lng_hip_buffer_len(raw.as_ptr()) };
        Ok(Buffer { raw, len })
    }

    /// Read-only memory filled once, attachable to any number of batches (`apple.rs:297`).
    pub fn resident(&self, bytes: &[u8]) -> Result<Arc<Resident>, Error> {
        let mut raw = ptr::null_mut();
        // SAFETY: `bytes` is readable for its length; the library copies it before returning.
        check_len(
            unsafe { ffi::lng_hip_resident(self.raw.as_ptr(), bytes.as_ptr().cast(), bytes.len(), &mut raw) },
            bytes.len(),
        )?;
        NonNull::new(raw)
            .map(|raw| Arc::new(Resident { raw, len: bytes.len() }))
            .ok_or(Error::Alloc(bytes.len()))
    }

    /// [`Gpu::resident`] from 16-bit words (`apple.rs:302`).
    pub fn resident_words(&self, words: &[u16]) -> Result<Arc<Resident>, Error> {
        // SAFETY: any `u16` slice is readable as twice as many bytes.
        self.resident(unsafe { std::slice::from_raw_parts(words.as_ptr().cast(), words.len() * 2) })
    }

    /// Starts recording a batch that owns `buffers` until it completes; dispatches refer to them by
    /// position in this vector (`apple.rs:365`).
    pub fn batch(&self, buffers: Vec<Buffer>, _dispatch: Dispatch) -> Result<Batch<'_>, Error> {
        let handles: Vec<*mut ffi::LngBuffer> = buffers.iter().map(|b| b.raw.as_ptr()).collect();
        let mut raw = ptr::null_mut();
        // SAFETY: `handles` holds live buffer handles; the library copies the list.
        check(unsafe { ffi::lng_hip_batch(self.raw.as_ptr(), handles.as_ptr(), handles.len(), &mut raw) })?;
        let raw = NonNull::new(raw).ok_or_else(|| Error::Gpu("no batch".into()))?;
        Ok(Batch {
            raw: Some(raw),
            buffers,
            residents: Vec::new(),
            dtype: DType::F32,
            gpu: PhantomData,
        })
    }

    /// The plain attention operator for callers that cannot allocate (code under HIP graph capture,
    /// tight serving loops): raw device addresses, launched at once on `stream` (a `hipStream_t`; null
    /// is the default stream), no allocation of any kind. `t * heads * ceil(dim / 64) <= 2048` per call;
    /// calls that can overlap in time on one GPU race on the library's fixed scratch array.
    ///
    /// # Safety
    /// The addresses must be device memory of this GPU holding what `shape` and `dtype` imply, and must
    /// stay valid until the stream has run the call.
    #[allow(clippy::too_many_arguments)]
    pub unsafe fn attention_grouped_static(
        &self,
        stream: *mut c_void,
        (q, k, v): (*const c_void, *const c_void, *const c_void),
        sinks: *const f32,
        out: *mut c_void,
        shape: GroupedShape,
        dtype: DType,
    ) -> Result<(), Error> {
        let shape = shape.raw();
        // SAFETY: the caller's contract.
        check(unsafe {
            ffi::lng_hip_attention_grouped_static(self.raw.as_ptr(), stream, q, k, v, out, sinks, &shape, dtype as i32)
        })
    }
}

impl Drop for Gpu {
    /// Waits for submitted batches. Buffers, residents and committed batches that are still alive keep
    /// working; the device's resources go when the last of them has gone.
    fn drop(&mut self) {
        // SAFETY: the handle is live and not used again.
        unsafe { ffi::lng_hip_close(self.raw.as_ptr()) }
    }
}

/// Device memory. The GPU only touches a buffer while a [`Batch`] owns it, and a batch hands its buffers
/// back only after the GPU has finished, so a `Buffer` in hand is never being written by the GPU
/// (`apple.rs:388-396`).
pub struct Buffer {
    raw: NonNull<ffi::LngBuffer>,
    len: usize,
}

// SAFETY: the handle names device memory; access is serialized by ownership.
unsafe impl Send for Buffer {}

impl Buffer {
    pub fn len(&self) -> usize {
        self.len
    }

    pub fn is_empty(&self) -> bool {
        self.len == 0
    }

    /// Copies bytes `offset..offset + dst.len()` to the host (`as_bytes()[..]`, `apple.rs:409`). Blocking.
    pub fn read(&self, offset: usize, dst: &mut [u8]) -> Result<(), Error> {
        // SAFETY: `dst` is writable for its length.
        check(unsafe { ffi::lng_hip_download(self.raw.as_ptr(), offset, dst.as_mut_ptr().cast(), dst.len()) })
    }

    /// Copies `src` over bytes `offset..offset + src.len()` (`as_bytes_mut()[..].copy_from_slice`,
    /// `apple.rs:415`). Blocking.
    pub fn write(&mut self, offset: usize, src: &[u8]) -> Result<(), Error> {
        // SAFETY: `src` is readable for its length.
        check(unsafe { ffi::lng_hip_upload(self.raw.as_ptr(), offset, src.as_ptr().cast(), src.len()) })
    }

    /// The whole buffer as `f32` (`as_f32()`, `apple.rs:421`).
    pub fn read_f32(&self) -> Result<Vec<f32>, Error> {
        let mut values = vec![0.0f32; self.len / 4];
        // SAFETY: `values` is writable for `values.len() * 4` bytes.
        check(unsafe {
            ffi::lng_hip_download(self.raw.as_ptr(), 0, values.as_mut_ptr().cast(), values.len() * 4)
        })?;
        Ok(values)
    }

    /// Copies `src` to the `f32` elements from `first` on (`as_f32_mut()[first..]`, `apple.rs:426`).
    pub fn write_f32(&mut self, first: usize, src: &[f32]) -> Result<(), Error> {
        // SAFETY: `src` is readable for `src.len() * 4` bytes.
        check(unsafe { ffi::lng_hip_upload(self.raw.as_ptr(), first * 4, src.as_ptr().cast(), src.len() * 4) })
    }

    /// Sets every byte of `offset..offset + len` to `byte`. Blocking.
    pub fn fill(&mut self, offset: usize, byte: u8, len: usize) -> Result<(), Error> {
        // SAFETY: plain call on a live handle.
        check(unsafe { ffi::lng_hip_fill(self.raw.as_ptr(), offset, i32::from(byte), len) })
    }

    /// The raw device address, for sharing the memory with other HIP code.
    pub fn device_ptr(&self) -> *mut c_void {
        // SAFETY: plain call on a live handle.
        unsafe { ffi::lng_hip_buffer_device_ptr(self.raw.as_ptr()) }
    }
}

impl Drop for Buffer {
    fn drop(&mut self) {
        // SAFETY: the handle is live and not used again. (A buffer that a batch owns is inside that batch,
        // so the refusal for owned buffers cannot happen here.)
        let _ = unsafe { ffi::lng_hip_buffer_free(self.raw.as_ptr()) };
    }
}

/// Read-only device memory shared by any number of batches (`apple.rs:465`).
pub struct Resident {
    raw: NonNull<ffi::LngBuffer>,
    len: usize,
}

// SAFETY: never written after creation.
unsafe impl Send for Resident {}
unsafe impl Sync for Resident {}

impl Resident {
    pub fn len(&self) -> usize {
        self.len
    }

    pub fn is_empty(&self) -> bool {
        self.len == 0
    }
}

impl Drop for Resident {
    fn drop(&mut self) {
        // SAFETY: the last `Arc` is gone: no batch in flight holds the resident (each keeps a clone until
        // its completion).
        let _ = unsafe { ffi::lng_hip_buffer_free(self.raw.as_ptr()) };
    }
}

/// Bytes `offset..offset + len` of the batch's buffer number `buffer`: its own buffers first, then the
/// residents it attached, in order (`apple.rs:507-512`).
#[derive(Clone, Copy, Debug, PartialEq, Eq)]
pub struct Slice {
    pub buffer: usize,
    pub offset: usize,
    pub len: usize,
}

impl Slice {
    pub const fn new(buffer: usize, offset: usize, len: usize) -> Self {
        Self { buffer, offset, len }
    }
}

impl From<Slice> for ffi::LngSlice {
    fn from(s: Slice) -> Self {
        Self { buffer: s.buffer as u64, offset: s.offset as u64, len: s.len as u64 }
    }
}

/// The shape of one [`Batch::attention_grouped`] dispatch (`apple.rs:598-614`).
#[derive(Clone, Copy, Debug)]
pub struct GroupedShape {
    /// New positions (queries).
    pub t: usize,
    /// The absolute position of the first of them.
    pub start: usize,
    pub heads: usize,
    /// Key/value heads; `heads` is a multiple of it.
    pub kv_heads: usize,
    /// Width of every query, key and value head: a multiple of 32 (16 for the tiled form), at most 512.
    pub dim: usize,
    /// Positions each query sees, its own included; `usize::MAX` for all of them.
    pub window: usize,
    /// Rows in the key and value buffers; position `s` is in row `s % slots`.
    pub slots: usize,
    pub scale: f32,
}

impl GroupedShape {
    fn raw(&self) -> ffi::LngGroupedShape {
        ffi::LngGroupedShape {
            t: self.t as u64,
            start: self.start as u64,
            heads: self.heads as u64,
            kv_heads: self.kv_heads as u64,
            dim: self.dim as u64,
            window: if self.window == usize::MAX { ffi::LNG_WINDOW_FULL } else { self.window as u64 },
            slots: self.slots as u64,
            scale: self.scale,
        }
    }

    /// The shape rules alone, with no device: exactly the refusals of `apple.rs:1243-1272` (`tiled` false)
    /// and `apple.rs:1356-1385` (`tiled` true).
    pub fn check(&self, tiled: bool) -> Result<(), Error> {
        let raw = self.raw();
        // SAFETY: `raw` is a valid shape for the duration of the call.
        check(unsafe { ffi::lng_hip_check_grouped(&raw, i32::from(tiled)) })
    }
}

/// What a finished batch hands back on the proactor: its buffers, and how long the GPU spent on it or why
/// it failed (`apple.rs:536-539`).
pub struct Completed {
    pub buffers: Vec<Buffer>,
    pub gpu_time: Result<Duration, Error>,
}

/// One query of [`Batch::attention_decode_batched`]: byte offsets into the buffers the call names.
pub type DecodeItem = ffi::LngDecodeItem;
/// One sequence of [`Batch::prepare_attention`].
pub type PrepareItem = ffi::LngPrepareItem;

/// The buffers of [`Batch::prepare_attention`] (indices as in [`Slice::buffer`]) and the optional biases.
#[derive(Clone, Copy, Debug)]
pub struct PrepareBuffers {
    pub q: usize,
    pub k: usize,
    pub v: usize,
    pub table: usize,
    pub q_out: usize,
    pub k_cache: usize,
    pub v_cache: usize,
    pub q_bias: Option<Slice>,
    pub k_bias: Option<Slice>,
    pub v_bias: Option<Slice>,
}

/// One matrix of [`Batch::gemm_q8_0_many`]: its codes and scales, its dense output and its rows.
#[derive(Clone, Copy, Debug)]
pub struct Q8Matrix {
    pub codes: Slice,
    pub scales: Slice,
    pub y: Slice,
    pub rows: usize,
}

/// One batch being recorded (`apple.rs:541`).
pub struct Batch<'g> {
    /// `None` once committed: the completion lets go of the handle.
    raw: Option<NonNull<ffi::LngBatch>>,
    buffers: Vec<Buffer>,
    /// Attached residents, kept alive until the GPU is done with them.
    residents: Vec<Arc<Resident>>,
    dtype: DType,
    gpu: PhantomData<&'g Gpu>,
}

impl Drop for Batch<'_> {
    /// A batch dropped without [`Batch::commit`] (for example after a dispatch error) runs nothing
    /// (`apple.rs:553-561`); its buffers are then freed with it.
    fn drop(&mut self) {
        if let Some(raw) = self.raw.take() {
            // SAFETY: the handle is live and not used again; the buffers are dropped after this returns.
            unsafe { ffi::lng_hip_batch_drop(raw.as_ptr()) }
        }
    }
}

/// What travels through the library as `user` from [`Batch::commit`] to its completion.
struct Pending<P: CompletionPort, F> {
    raw: NonNull<ffi::LngBatch>,
    buffers: Vec<Buffer>,
    residents: Vec<Arc<Resident>>,
    on_done: F,
    proactor: ProactorHandle<P>,
}

/// Runs on the library's completion thread: rebuilds [`Completed`] and re-posts `on_done` to the
/// proactor, as the Metal completion handler does (`apple.rs:2213-2233`).
unsafe extern "C" fn completion<P, F>(done: *const ffi::LngCompleted, user: *mut c_void)
where
    P: CompletionPort,
    ProactorHandle<P>: Send,
    F: FnOnce(Completed) + Send + 'static,
{
    // A panic must not cross the C frames above.
    let _ = catch_unwind(AssertUnwindSafe(|| {
        // SAFETY: `user` is the box `commit` leaked, handed back exactly once.
        let pending = unsafe { Box::from_raw(user.cast::<Pending<P, F>>()) };
        // SAFETY: `done` is valid during the callback, and so is its message.
        let done = unsafe { &*done };
        let gpu_time = if done.status == ffi::LNG_OK {
            Ok(Duration::from_secs_f64(done.gpu_seconds.max(0.0)))
        } else {
            let text = if done.message.is_null() {
                format!("status {}", done.status)
            } else {
                // SAFETY: NUL-terminated, valid during the callback.
                unsafe { CStr::from_ptr(done.message) }.to_string_lossy().into_owned()
            };
            Err(Error::Gpu(text))
        };
        let Pending { raw, buffers, residents, on_done, proactor } = *pending;
        // Allowed from inside the callback: the handle is freed when the callback returns. The buffers
        // are the caller's again from here on.
        // SAFETY: the handle is live and not used again.
        unsafe { ffi::lng_hip_batch_drop(raw.as_ptr()) };
        drop(residents);
        // If the proactor has shut down, the closure and with it the buffers are dropped instead.
        let _ = proactor.enqueue_work(move |_| on_done(Completed { buffers, gpu_time }));
    }));
}

impl<'g> Batch<'g> {
    fn handle(&self) -> *mut ffi::LngBatch {
        self.raw.expect("a batch has its handle until it is committed").as_ptr()
    }

    /// Element type of the attention and row-copy dispatches recorded from here on (default `F32`).
    pub fn element_type(&mut self, dtype: DType) {
        self.dtype = dtype;
    }

    /// Dispatches recorded so far (`apple.rs:829`).
    pub fn dispatches(&self) -> usize {
        // SAFETY: plain call on a live handle.
        unsafe { ffi::lng_hip_batch_dispatches(self.handle()) }
    }

    /// Makes `resident` visible to this batch's dispatches; the slice covers all of it (`apple.rs:835`).
    pub fn attach(&mut self, resident: &Arc<Resident>) -> Slice {
        let mut whole = ffi::LngSlice { buffer: 0, offset: 0, len: 0 };
        // SAFETY: both handles are live; `whole` is a valid place for the result.
        let rc = unsafe { ffi::lng_hip_batch_attach(self.handle(), resident.raw.as_ptr(), &mut whole) };
        assert_eq!(rc, ffi::LNG_OK, "attach: {}", last_message());
        self.residents.push(Arc::clone(resident));
        Slice::new(whole.buffer as usize, whole.offset as usize, whole.len as usize)
    }

    fn grouped(
        &mut self,
        (q, k, v): (Slice, Slice, Slice),
        sinks: Option<Slice>,
        out: Slice,
        shape: GroupedShape,
        tiled: bool,
    ) -> Result<(), Error> {
        let raw = shape.raw();
        let sinks: Option<ffi::LngSlice> = sinks.map(Into::into);
        let sinks_ptr = sinks.as_ref().map_or(ptr::null(), |s| s as *const ffi::LngSlice);
        let dtype = self.dtype as i32;
        // SAFETY: `raw` and `sinks` outlive the call; the library validates every slice.
        check(unsafe {
            if tiled {
                ffi::lng_hip_attention_grouped_tiled(self.handle(), q.into(), k.into(), v.into(), out.into(), sinks_ptr, &raw, dtype)
            } else {
                ffi::lng_hip_attention_grouped(self.handle(), q.into(), k.into(), v.into(), out.into(), sinks_ptr, &raw, dtype)
            }
        })
    }

    /// Causal grouped-query attention of `t` new positions over a ring of rows (`apple.rs:1199`).
    pub fn attention_grouped(&mut self, q: Slice, k: Slice, v: Slice, out: Slice, shape: GroupedShape) -> Result<(), Error> {
        self.grouped((q, k, v), None, out, shape, false)
    }

    /// The same with a learned sink logit per head joining each softmax (`apple.rs:1213`).
    pub fn attention_grouped_with_sinks(
        &mut self,
        (q, k, v): (Slice, Slice, Slice),
        sinks: Slice,
        out: Slice,
        shape: GroupedShape,
    ) -> Result<(), Error> {
        self.grouped((q, k, v), Some(sinks), out, shape, false)
    }

    /// The prompt-pass form: `q` and `out` hold `t` rounded up to 32 rows (`apple.rs:1311`).
    pub fn attention_grouped_tiled(&mut self, q: Slice, k: Slice, v: Slice, out: Slice, shape: GroupedShape) -> Result<(), Error> {
        self.grouped((q, k, v), None, out, shape, true)
    }

    /// The prompt-pass form with sinks (`apple.rs:1324`).
    pub fn attention_grouped_tiled_with_sinks(
        &mut self,
        (q, k, v): (Slice, Slice, Slice),
        sinks: Slice,
        out: Slice,
        shape: GroupedShape,
    ) -> Result<(), Error> {
        self.grouped((q, k, v), Some(sinks), out, shape, true)
    }

    /// Copies `rows` rows of `width` elements of the batch's element type, strides in elements
    /// (`apple.rs:1762`): how `gpt-oss/src/gpu.rs:744-759` writes new key and value rows into a cache.
    pub fn copy_rows(
        &mut self,
        (src, src_stride): (Slice, usize),
        (dst, dst_stride): (Slice, usize),
        rows: usize,
        width: usize,
    ) -> Result<(), Error> {
        let dtype = self.dtype;
        self.copy_rows_converting((src, src_stride, dtype), (dst, dst_stride, dtype), rows, width)
    }

    /// `f32` rows in place: `v = w * v / sqrt(mean(v^2) + eps)` (`apple.rs:1733`).
    pub fn rmsnorm_rows(&mut self, (v, w): (Slice, Slice), rows: usize, (d, stride): (usize, usize), eps: f32) -> Result<(), Error> {
        // SAFETY: plain call; the library validates every slice.
        check(unsafe { ffi::lng_hip_rmsnorm_rows(self.handle(), v.into(), w.into(), rows as u64, d as u64, stride as u64, eps) })
    }

    /// `dst[r][i] += src[r * src_stride + i]`, `f32`; a stride of 0 adds one row to every row (`apple.rs:1886`).
    pub fn add_rows(&mut self, dst: Slice, (src, src_stride): (Slice, usize), rows: usize, width: usize) -> Result<(), Error> {
        // SAFETY: as above.
        check(unsafe { ffi::lng_hip_add_rows(self.handle(), dst.into(), src.into(), src_stride as u64, rows as u64, width as u64) })
    }

    /// Rotary by halves over all of each head, `f32`, in place (`apple.rs:1916`).
    pub fn rotate_halves(&mut self, x: Slice, table: Slice, rows: usize, (heads, dim): (usize, usize)) -> Result<(), Error> {
        self.rotate_halves_partial(x, table, rows, (heads, dim, dim))
    }

    /// Rotary by halves over the first `rotary` dimensions of each head (`apple.rs:1929`).
    pub fn rotate_halves_partial(
        &mut self,
        x: Slice,
        table: Slice,
        rows: usize,
        (heads, dim, rotary): (usize, usize, usize),
    ) -> Result<(), Error> {
        // SAFETY: as above.
        check(unsafe {
            ffi::lng_hip_rotate_halves(self.handle(), x.into(), table.into(), rows as u64, heads as u64, dim as u64, rotary as u64)
        })
    }

    /// `y = W x` with `W` in repacked `Q8_0` (`apple.rs:1812`).
    pub fn gemv_q8_0(&mut self, (codes, scales): (Slice, Slice), x: Slice, y: Slice, rows: usize, cols: usize) -> Result<(), Error> {
        // SAFETY: as above.
        check(unsafe { ffi::lng_hip_gemv_q8_0(self.handle(), codes.into(), scales.into(), x.into(), y.into(), rows as u64, cols as u64) })
    }

    /// `y[p] = W x[p]` for `n` positions (`apple.rs:1833`).
    #[allow(clippy::too_many_arguments)]
    pub fn gemm_q8_0(
        &mut self,
        (codes, scales): (Slice, Slice),
        x: Slice,
        y: Slice,
        rows: usize,
        cols: usize,
        n: usize,
        (x_stride, y_stride): (usize, usize),
    ) -> Result<(), Error> {
        // SAFETY: as above.
        check(unsafe {
            ffi::lng_hip_gemm_q8_0(
                self.handle(), codes.into(), scales.into(), x.into(), y.into(), rows as u64, cols as u64, n as u64,
                x_stride as u64, y_stride as u64,
            )
        })
    }

    /// The same product for prompt passes: `rows % 64 == 0`, `n % 32 == 0` (`apple.rs:1857`).
    #[allow(clippy::too_many_arguments)]
    pub fn gemm_q8_0_tiled(
        &mut self,
        (codes, scales): (Slice, Slice),
        x: Slice,
        y: Slice,
        rows: usize,
        cols: usize,
        n: usize,
        (x_stride, y_stride): (usize, usize),
    ) -> Result<(), Error> {
        // SAFETY: as above.
        check(unsafe {
            ffi::lng_hip_gemm_q8_0_tiled(
                self.handle(), codes.into(), scales.into(), x.into(), y.into(), rows as u64, cols as u64, n as u64,
                x_stride as u64, y_stride as u64,
            )
        })
    }

    /// Orders later dispatches after earlier ones (`apple.rs:2194`). Dispatches of a batch already run in
    /// order here.
    pub fn barrier(&mut self) {
        // SAFETY: plain call on a live handle.
        let _ = unsafe { ffi::lng_hip_batch_barrier(self.handle()) };
    }

    /// Sends the batch to the GPU. When it finishes, `on_done` runs as a job on `proactor` with the batch's
    /// buffers. Nothing blocks. If the proactor has shut down by then, the buffers are dropped instead
    /// (`apple.rs:2202`).
    pub fn commit<P, F>(mut self, proactor: &ProactorHandle<P>, on_done: F)
    where
        P: CompletionPort,
        ProactorHandle<P>: Send,
        F: FnOnce(Completed) + Send + 'static,
    {
        let raw = self.raw.take().expect("a batch is committed once");
        let pending = Box::new(Pending {
            raw,
            buffers: std::mem::take(&mut self.buffers),
            residents: std::mem::take(&mut self.residents),
            on_done,
            proactor: proactor.clone(),
        });
        let user = Box::into_raw(pending);
        // SAFETY: `user` stays valid until `completion` takes it back, which happens exactly once if the
        // call succeeds and never if it fails.
        let rc = unsafe { ffi::lng_hip_batch_commit(raw.as_ptr(), Some(completion::<P, F>), user.cast()) };
        if rc != ffi::LNG_OK {
            let why = last_message();
            // SAFETY: the library did not keep `user`.
            let Pending { raw, buffers, residents, on_done, proactor } = *unsafe { Box::from_raw(user) };
            // SAFETY: the handle is live and not used again.
            unsafe { ffi::lng_hip_batch_drop(raw.as_ptr()) };
            drop(residents);
            let _ = proactor.enqueue_work(move |_| on_done(Completed { buffers, gpu_time: Err(Error::Gpu(why)) }));
        }
    }

    /// Commits and blocks until the GPU has finished: for tools and tests that have no proactor.
    pub fn run(mut self) -> Completed {
        let raw = self.raw.take().expect("a batch is committed once");
        let buffers = std::mem::take(&mut self.buffers);
        let residents = std::mem::take(&mut self.residents);
        let mut seconds = 0.0f64;
        // SAFETY: no callback, so nothing outlives the calls; the handle is dropped last.
        let gpu_time = check(unsafe { ffi::lng_hip_batch_commit(raw.as_ptr(), None, ptr::null_mut()) })
            .and_then(|()| check(unsafe { ffi::lng_hip_batch_wait(raw.as_ptr(), &mut seconds) }))
            .map(|()| Duration::from_secs_f64(seconds.max(0.0)));
        // SAFETY: the handle is live and not used again.
        unsafe { ffi::lng_hip_batch_drop(raw.as_ptr()) };
        drop(residents);
        Completed { buffers, gpu_time }
    }

    // ---- additions without a counterpart in metal-compute ----------------------------------------------

    /// [`Batch::copy_rows`] between element types: `f32 -> bf16` rounds to nearest even, so the new rows of
    /// an `f32` projection go straight into a `bf16` cache.
    pub fn copy_rows_converting(
        &mut self,
        (src, src_stride, src_dtype): (Slice, usize, DType),
        (dst, dst_stride, dst_dtype): (Slice, usize, DType),
        rows: usize,
        width: usize,
    ) -> Result<(), Error> {
        // SAFETY: plain call; the library validates every slice.
        check(unsafe {
            ffi::lng_hip_copy_rows(
                self.handle(), src.into(), src_stride as u64, src_dtype as i32, dst.into(), dst_stride as u64,
                dst_dtype as i32, rows as u64, width as u64,
            )
        })
    }

    /// One decoding query per item, many sequences in one dispatch: each item computes what
    /// [`Batch::attention_grouped_with_sinks`] computes with `t = 1` (`gpt-oss/src/gpu.rs:794-805` records one
    /// such call per sequence and layer). The five buffers are named by index; offsets are bytes.
    #[allow(clippy::too_many_arguments)]
    pub fn attention_decode_batched(
        &mut self,
        (q, k, v): (usize, usize, usize),
        sinks: usize,
        out: usize,
        items: &[DecodeItem],
        (heads, kv_heads, dim): (usize, usize, usize),
        scale: f32,
    ) -> Result<(), Error> {
        // SAFETY: `items` is readable for its length; the library copies it before returning.
        check(unsafe {
            ffi::lng_hip_attention_decode_batched(
                self.handle(), q as u64, k as u64, v as u64, out as u64, sinks as u64, items.as_ptr(), items.len(),
                heads as u64, kv_heads as u64, dim as u64, scale, self.dtype as i32,
            )
        })
    }

    /// Biases, rotary, narrowing to the batch's element type and the ring append of new key and value rows
    /// in one dispatch: what the three `add_rows`, two `rotate_halves` and the `copy_rows` loop of
    /// `gpt-oss/src/gpu.rs:733-759` compute, in the same `f32` operations.
    pub fn prepare_attention(
        &mut self,
        buffers: PrepareBuffers,
        items: &[PrepareItem],
        (heads, kv_heads, dim, rotary): (usize, usize, usize, usize),
    ) -> Result<(), Error> {
        let bias = |s: Option<Slice>| -> Option<ffi::LngSlice> { s.map(Into::into) };
        let (qb, kb, vb) = (bias(buffers.q_bias), bias(buffers.k_bias), bias(buffers.v_bias));
        let at = |s: &Option<ffi::LngSlice>| s.as_ref().map_or(ptr::null(), |s| s as *const ffi::LngSlice);
        let raw = ffi::LngPrepareBuffers {
            q: buffers.q as u64,
            k: buffers.k as u64,
            v: buffers.v as u64,
            table: buffers.table as u64,
            q_out: buffers.q_out as u64,
            k_cache: buffers.k_cache as u64,
            v_cache: buffers.v_cache as u64,
            q_bias: at(&qb),
            k_bias: at(&kb),
            v_bias: at(&vb),
        };
        // SAFETY: `raw`, the biases and `items` outlive the call; the library copies what it keeps.
        check(unsafe {
            ffi::lng_hip_prepare_attention(
                self.handle(), &raw, items.as_ptr(), items.len(), heads as u64, kv_heads as u64, dim as u64, rotary as u64,
                self.dtype as i32,
            )
        })
    }

    /// [`Batch::gemm_q8_0`] for positions that are `bf16` already (the output of a `bf16` attention feeding the
    /// output projection, `gpt-oss/src/gpu.rs:807-817`); `y` is `f32`.
    #[allow(clippy::too_many_arguments)]
    pub fn gemm_q8_0_bf16(
        &mut self,
        (codes, scales): (Slice, Slice),
        x: Slice,
        y: Slice,
        rows: usize,
        cols: usize,
        n: usize,
        (x_stride, y_stride): (usize, usize),
    ) -> Result<(), Error> {
        // SAFETY: plain call; the library validates every slice.
        check(unsafe {
            ffi::lng_hip_gemm_q8_0_bf16(
                self.handle(), codes.into(), scales.into(), x.into(), y.into(), rows as u64, cols as u64, n as u64,
                x_stride as u64, y_stride as u64,
            )
        })
    }

    fn q8_matrices(matrices: &[Q8Matrix]) -> Vec<ffi::LngQ8Matrix> {
        matrices
            .iter()
            .map(|m| ffi::LngQ8Matrix { codes: m.codes.into(), scales: m.scales.into(), y: m.y.into(), rows: m.rows as u64 })
            .collect()
    }

    /// Up to four `Q8_0` matrices of `cols` columns times the same `n` positions, one dispatch when decoding
    /// (the q, k and v projections of `gpt-oss/src/gpu.rs:724-732`).
    pub fn gemm_q8_0_many(&mut self, matrices: &[Q8Matrix], x: Slice, cols: usize, n: usize, x_stride: usize) -> Result<(), Error> {
        let raw = Self::q8_matrices(matrices);
        // SAFETY: `raw` is readable for its length; the library copies it.
        check(unsafe { ffi::lng_hip_gemm_q8_0_many(self.handle(), raw.as_ptr(), raw.len(), x.into(), cols as u64, n as u64, x_stride as u64) })
    }

    /// The same with the RMS norm of the positions folded in (`gpt-oss/src/gpu.rs:712-732`); decoding only.
    #[allow(clippy::too_many_arguments)]
    pub fn gemm_q8_0_many_normed(
        &mut self,
        matrices: &[Q8Matrix],
        x: Slice,
        (norm_w, eps): (Slice, f32),
        cols: usize,
        n: usize,
        x_stride: usize,
    ) -> Result<(), Error> {
        let raw = Self::q8_matrices(matrices);
        // SAFETY: as above.
        check(unsafe {
            ffi::lng_hip_gemm_q8_0_many_normed(
                self.handle(), raw.as_ptr(), raw.len(), x.into(), norm_w.into(), eps, cols as u64, n as u64, x_stride as u64,
            )
        })
    }

    /// The output projection with its bias and the residual add folded in: `h[p] += (W x[p]) + bias`, rounded
    /// as the three dispatches of `gpt-oss/src/gpu.rs:807-827` round it; decoding only.
    #[allow(clippy::too_many_arguments)]
    pub fn gemm_q8_0_residual(
        &mut self,
        (codes, scales): (Slice, Slice),
        (x, x_dtype): (Slice, DType),
        bias: Option<Slice>,
        h: Slice,
        rows: usize,
        cols: usize,
        n: usize,
        (x_stride, h_stride): (usize, usize),
    ) -> Result<(), Error> {
        let bias: Option<ffi::LngSlice> = bias.map(Into::into);
        let bias_ptr = bias.as_ref().map_or(ptr::null(), |s| s as *const ffi::LngSlice);
        // SAFETY: `bias` outlives the call.
        check(unsafe {
            ffi::lng_hip_gemm_q8_0_residual(
                self.handle(), codes.into(), scales.into(), x.into(), x_dtype as i32, bias_ptr, h.into(), rows as u64,
                cols as u64, n as u64, x_stride as u64, h_stride as u64,
            )
        })
    }

    /// The XOR of every 16-byte word of `src`, written to the 16 bytes of `dst`: a plain streaming read (benchmarks
    /// and tests; no counterpart in metal-compute).
    pub fn checksum(&mut self, src: Slice, dst: Slice) -> Result<(), Error> {
        // SAFETY: plain call; the library validates the slices.
        check(unsafe { ffi::lng_hip_checksum(self.handle(), src.into(), dst.into()) })
    }

    /// Deterministic synthetic values written on the device (benchmarks and full-size tests).
    pub fn fill_synthetic(&mut self, dst: Slice, dtype: DType, seed: u64, scale: f32, period: u64) -> Result<(), Error> {
        // SAFETY: plain call; the library validates the slice.
        check(unsafe { ffi::lng_hip_fill_synthetic(self.handle(), dst.into(), dtype as i32, seed, scale, period) })
    }

    /// Records an event after every kernel of the batch, for [`Batch::run_timed`]-style accounting (the
    /// finer-grained form of the phases of `gpt-oss/src/gpu.rs:247-317`). Set before committing.
    pub fn set_timing(&mut self, enabled: bool) -> Result<(), Error> {
        // SAFETY: plain call on a live handle.
        check(unsafe { ffi::lng_hip_batch_set_timing(self.handle(), i32::from(enabled)) })
    }

    /// Commits with timing on, blocks, and returns for each of `kernels` the seconds the GPU spent in that
    /// kernel and how often it was launched, beside the usual [`Completed`].
    pub fn run_timed(mut self, kernels: &[&str]) -> (Completed, Vec<(f64, usize)>) {
        let _ = self.set_timing(true);
        let raw = self.raw.take().expect("a batch is committed once");
        let buffers = std::mem::take(&mut self.buffers);
        let residents = std::mem::take(&mut self.residents);
        let mut seconds = 0.0f64;
        // SAFETY: no callback; the handle is dropped last.
        let gpu_time = check(unsafe { ffi::lng_hip_batch_commit(raw.as_ptr(), None, ptr::null_mut()) })
            .and_then(|()| check(unsafe { ffi::lng_hip_batch_wait(raw.as_ptr(), &mut seconds) }))
            .map(|()| Duration::from_secs_f64(seconds.max(0.0)));
        let per_kernel = kernels
            .iter()
            .map(|name| {
                let (mut s, mut n) = (0.0f64, 0usize);
                if let Ok(name) = CString::new(*name) {
                    // SAFETY: `name` is NUL-terminated; `s` and `n` are valid places for the results.
                    let _ = unsafe { ffi::lng_hip_batch_kernel_seconds(raw.as_ptr(), name.as_ptr(), &mut s, &mut n) };
                }
                (s, n)
            })
            .collect();
        // SAFETY: the handle is live and not used again.
        unsafe { ffi::lng_hip_batch_drop(raw.as_ptr()) };
        drop(residents);
        (Completed { buffers, gpu_time }, per_kernel)
    }
}
