// src/device/hip/hip_shim.rs -- bindings to libx17ai_hip_shim (include/x17ai_hip_shim.h) and safe wrappers.
// UNCOMPILED HERE: no Rust toolchain in the image this was written in.
//
// Twin of src/device/cuda/cuda_shim.rs: the same 21 entry points with the same argument orders and struct layouts
// (:76-158) under x17ai_hip_* link names, the same ownership rules (a context handle whose first field is a
// reference count the C++ side maintains, :20-24; a kernel keeps its module alive, :445-449) and the same error
// convention (a null DiagnosticBuffer is success; every non-null one must be handed to x17ai_move_diagnostic,
// which appends its text to a Rust Vec<u8> through the FfiBuffer callbacks and frees it).
// What differs from CUDA without showing in the signatures: HIP has no driver context -- the shim makes the
// handle's device current for the duration of a call and restores the previous one; context_ptr() is the device
// ordinal + 1; preferred_shared_memory_carveout reads 100; get_kernel() checks the requested dynamic LDS against the
// device limit (160 KB on gfx950) instead of opting in to it.

use std::ffi::{c_char, c_void, CString};
use std::os::unix::ffi::OsStrExt;
use std::path::Path;
use std::ptr::NonNull;

use crate::device::DevicePtr;
use crate::util::ffi_buffer::FfiBuffer;
use crate::{ErrPack, TensorOpError};

type DevResult<T> = Result<T, ErrPack<TensorOpError>>;

// ---------------------------------------------------------------- opaque handles (x17ai_hip_shim.h)

macro_rules! opaque {
	($($name:ident),* $(,)?) => {$(
		#[repr(C)]
		pub struct $name { _opaque: [u8; 0] }
	)*};
}
opaque!(HipStreamHandle, HipDeviceData, HipTimerHandle, HipModuleHandle, HipKernelHandle, DiagnosticBuffer);

/// The C++ side keeps `references - 1` in the first word (cuda_shim.rs:20-24, hip_shim.cpp: HipContext).
#[repr(C)]
pub struct HipContextHandle {
	refcnt_minus_one: usize,
	_opaque: [u8; 0],
}

/// X17HipKernelAttrs: nine i32 in this order (cuda_shim.rs:51-63).  `ptx_version` / `binary_version` carry the
/// code object's ISA version on this device; `local_size_bytes != 0` means the kernel uses scratch memory.
#[repr(C)]
#[derive(Clone, Copy, Debug, Default)]
pub struct HipKernelAttrs {
	pub max_threads_per_block: i32,
	pub static_shared_size_bytes: i32,
	pub const_size_bytes: i32,
	pub local_size_bytes: i32,
	pub num_regs: i32,
	pub ptx_version: i32,
	pub binary_version: i32,
	pub max_dynamic_shared_size_bytes: i32,
	pub preferred_shared_memory_carveout: i32,
}

/// Two pointers returned by value; exactly one is non-null (cuda_shim.rs:70-74).
#[repr(C)]
struct PtrResult<T> {
	value: *mut T,
	diagnostic: *mut DiagnosticBuffer,
}

type Diag = *mut DiagnosticBuffer;

unsafe extern "C" {
	fn x17ai_move_diagnostic(diag: Diag, sink: FfiBuffer);

	#[link_name = "x17ai_hip_open_context"]
	fn open_context(device_id: usize) -> PtrResult<HipContextHandle>;
	#[link_name = "x17ai_hip_close_context"]
	fn close_context(ctx: *mut HipContextHandle) -> Diag;
	#[link_name = "x17ai_hip_context_ptr"]
	fn context_ptr(ctx: *mut HipContextHandle) -> *mut c_void;

	#[link_name = "x17ai_hip_open_stream"]
	fn open_stream(ctx: *mut HipContextHandle) -> PtrResult<HipStreamHandle>;
	#[link_name = "x17ai_hip_close_stream"]
	fn close_stream(stream: *mut HipStreamHandle) -> Diag;
	#[link_name = "x17ai_hip_synchronize"]
	fn synchronize(stream: *mut HipStreamHandle) -> Diag;

	#[link_name = "x17ai_hip_create_timer"]
	fn create_timer(ctx: *mut HipContextHandle, stream: *mut HipStreamHandle) -> PtrResult<HipTimerHandle>;
	#[link_name = "x17ai_hip_destroy_timer"]
	fn destroy_timer(timer: *mut HipTimerHandle) -> Diag;
	#[link_name = "x17ai_hip_timer_start"]
	fn timer_start(timer: *mut HipTimerHandle) -> Diag;
	#[link_name = "x17ai_hip_timer_stop"]
	fn timer_stop(timer: *mut HipTimerHandle) -> Diag;
	#[link_name = "x17ai_hip_timer_elapsed_seconds"]
	fn timer_elapsed_seconds(timer: *mut HipTimerHandle, seconds: *mut f64) -> Diag;

	#[link_name = "x17ai_hip_alloc"]
	fn alloc(stream: *mut HipStreamHandle, bytes: usize) -> PtrResult<HipDeviceData>;
	#[link_name = "x17ai_hip_free"]
	fn free(stream: *mut HipStreamHandle, ptr: *mut HipDeviceData) -> Diag;
	#[link_name = "x17ai_hip_upload_data"]
	fn upload_data(stream: *mut HipStreamHandle, src: *const u8, dst: *mut HipDeviceData, offset_bytes: usize, size_bytes: usize) -> Diag;
	#[link_name = "x17ai_hip_download_data"]
	fn download_data(stream: *mut HipStreamHandle, src: *mut HipDeviceData, dst: *mut u8, offset_bytes: usize, size_bytes: usize) -> Diag;

	#[link_name = "x17ai_hip_load_module"]
	fn load_module(ctx: *mut HipContextHandle, code_object_path: *const c_char) -> PtrResult<HipModuleHandle>;
	#[link_name = "x17ai_hip_del_module"]
	fn del_module(module: *mut HipModuleHandle) -> Diag;
	#[link_name = "x17ai_hip_get_kernel"]
	fn get_kernel(module: *mut HipModuleHandle, name: *const c_char, smem_size: usize) -> PtrResult<HipKernelHandle>;
	#[link_name = "x17ai_hip_read_kernel_attrs"]
	fn read_kernel_attrs(kernel: *mut HipKernelHandle, attrs: *mut HipKernelAttrs) -> Diag;
	#[link_name = "x17ai_hip_launch_kernel"]
	fn launch_kernel(
		stream: *mut HipStreamHandle, kernel: *mut HipKernelHandle,
		grid_x: usize, grid_y: usize, grid_z: usize,
		block_x: usize, block_y: usize, block_z: usize,
		shared_mem_bytes: usize,
		args: *mut *mut c_void,
	) -> Diag;
}

// ---------------------------------------------------------------- diagnostics

/// Moves the text out of a diagnostic (which frees it on the C++ side); `what` names the call for the case that
/// the shim had no text to give.
pub(super) fn diagnostic_text(diag: Diag, what: &str) -> String {
	let mut bytes = Vec::new();
	unsafe { x17ai_move_diagnostic(diag, FfiBuffer::new(&mut bytes)) };
	if bytes.is_empty() {
		format!("{what} failed without diagnostic")
	} else {
		String::from_utf8_lossy(&bytes).into_owned()
	}
}

#[cold]
#[inline(never)]
fn device_error(diag: Diag, what: &str) -> ErrPack<TensorOpError> {
	ErrPack::new(TensorOpError::Device, diagnostic_text(diag, what))
}

/// null = success
fn check(diag: Diag, what: &str) -> DevResult<()> {
	if diag.is_null() { Ok(()) } else { Err(device_error(diag, what)) }
}

/// for Drop impls: the diagnostic still has to be moved so that the C++ side frees it
fn ignore(diag: Diag) {
	if !diag.is_null() {
		let _ = diagnostic_text(diag, "");
	}
}

fn take<T>(result: PtrResult<T>, what: &str) -> DevResult<NonNull<T>> {
	match NonNull::new(result.value) {
		Some(value) => {
			debug_assert!(result.diagnostic.is_null());
			Ok(value)
		},
		None => Err(device_error(result.diagnostic, what)),
	}
}

fn c_string(bytes: &[u8], what: &str) -> DevResult<CString> {
	CString::new(bytes)
		.map_err(|_| ErrPack::new(TensorOpError::Device, format!("{what} contains an interior NUL byte")))
}

// ---------------------------------------------------------------- stream (+ its context)

pub struct HipStream {
	stream: NonNull<HipStreamHandle>,
	ctx: NonNull<HipContextHandle>,
}

impl HipStream {
	pub fn new(device_id: usize) -> DevResult<Self> {
		let ctx = take(unsafe { open_context(device_id) }, "x17ai_hip_open_context()")?;
		match take(unsafe { open_stream(ctx.as_ptr()) }, "x17ai_hip_open_stream()") {
			Ok(stream) => Ok(Self { stream, ctx }),
			Err(stream_err) => {
				// the context must not leak; if closing it fails too, report that with the first error nested
				let closing = unsafe { close_context(ctx.as_ptr()) };
				if closing.is_null() {
					Err(stream_err)
				} else {
					Err(ErrPack::new_with_nested(
						TensorOpError::Device,
						diagnostic_text(closing, "x17ai_hip_close_context()"),
						stream_err,
					))
				}
			},
		}
	}

	pub fn handle(&self) -> *mut HipStreamHandle {
		self.stream.as_ptr()
	}

	/// Not a driver context: the device ordinal + 1 as an opaque non-null pointer.
	pub fn hip_context(&self) -> *mut c_void {
		unsafe { context_ptr(self.ctx.as_ptr()) }
	}

	pub fn synchronize(&self) -> DevResult<()> {
		check(unsafe { synchronize(self.stream.as_ptr()) }, "x17ai_hip_synchronize()")
	}

	/// # Safety
	/// The block is uninitialised and only valid on this stream's device (stream-ordered allocation).
	pub unsafe fn alloc(&self, bytes: usize) -> DevResult<DevicePtr> {
		let data = take(unsafe { alloc(self.stream.as_ptr(), bytes) }, "x17ai_hip_alloc()")?;
		// the handle IS the device address: kernels receive it verbatim (gemm.rs:618-631)
		Ok(DevicePtr::new(data.as_ptr().cast()))
	}

	/// # Safety
	/// `ptr` came from `alloc` of this stream and is not used afterwards.
	pub unsafe fn free(&self, ptr: DevicePtr) {
		ignore(unsafe { free(self.stream.as_ptr(), ptr.as_ptr::<HipDeviceData>()) });
	}

	/// # Safety
	/// `src` points at `size_bytes` readable bytes that stay alive until the stream has been synchronized
	/// (the copy is asynchronous); `dst` + `offset_bytes` .. + `size_bytes` lies inside the allocation.
	pub unsafe fn upload_data(&self, src: NonNull<u8>, dst: DevicePtr, offset_bytes: usize, size_bytes: usize) -> DevResult<()> {
		check(
			unsafe { upload_data(self.stream.as_ptr(), src.as_ptr(), dst.as_ptr::<HipDeviceData>(), offset_bytes, size_bytes) },
			"x17ai_hip_upload_data()",
		)
	}

	/// # Safety
	/// As `upload_data`, with `dst` writable; the bytes are there after `synchronize()` (Tensor::to_cpu does not
	/// synchronize, src/tensor.rs:98-112).
	pub unsafe fn download_data(&self, src: DevicePtr, dst: NonNull<u8>, offset_bytes: usize, size_bytes: usize) -> DevResult<()> {
		check(
			unsafe { download_data(self.stream.as_ptr(), src.as_ptr::<HipDeviceData>(), dst.as_ptr(), offset_bytes, size_bytes) },
			"x17ai_hip_download_data()",
		)
	}

	/// Loads a gfx950 code object (kernel.hsaco, possibly an offload bundle as `hipcc --genco` writes it).
	pub fn load_module_from_code_object(&self, path: &Path) -> DevResult<HipModule> {
		let path = c_string(path.as_os_str().as_bytes(), "HIP code object path")?;
		let handle = take(unsafe { load_module(self.ctx.as_ptr(), path.as_ptr()) }, "x17ai_hip_load_module()")?;
		Ok(HipModule { handle })
	}
}

impl Drop for HipStream {
	fn drop(&mut self) {
		ignore(unsafe { close_stream(self.stream.as_ptr()) });
		ignore(unsafe { close_context(self.ctx.as_ptr()) });
	}
}

// ---------------------------------------------------------------- module and kernel

pub struct HipModule {
	handle: NonNull<HipModuleHandle>,
}

impl HipModule {
	/// Consumes the module: the kernel owns it from here on (every code object exports the one entry `kernel`).
	pub fn get_kernel(self, name: &str, smem_size: usize) -> DevResult<HipKernel> {
		let name = c_string(name.as_bytes(), "HIP kernel name")?;
		let handle = take(
			unsafe { get_kernel(self.handle.as_ptr(), name.as_ptr(), smem_size) },
			"x17ai_hip_get_kernel()",
		)?;
		let mut attrs = HipKernelAttrs::default();
		check(unsafe { read_kernel_attrs(handle.as_ptr(), &raw mut attrs) }, "x17ai_hip_read_kernel_attrs()")?;
		Ok(HipKernel { _module: self, handle, attrs })
	}
}

impl Drop for HipModule {
	fn drop(&mut self) {
		ignore(unsafe { del_module(self.handle.as_ptr()) });
	}
}

pub struct HipKernel {
	_module: HipModule,
	handle: NonNull<HipKernelHandle>,
	pub attrs: HipKernelAttrs,
}

impl HipKernel {
	pub fn handle(&self) -> *mut HipKernelHandle {
		self.handle.as_ptr()
	}

	/// scratch memory in use (register spills or a stack object)
	pub fn has_spills(&self) -> bool {
		self.attrs.local_size_bytes != 0
	}

	/// # Safety
	/// One pointer per kernel parameter, each to a host value of the parameter's exact layout.  The operator layer
	/// passes 8-byte `usize` slots for the kernels' `u32` parameters (gemm.rs:618-631); the kernels read the low half.
	pub unsafe fn launch(
		&self,
		stream: &HipStream,
		grid_dim: [usize; 3],
		block_dim: [usize; 3],
		shared_mem_bytes: usize,
		args: &mut [*mut c_void],
	) -> DevResult<()> {
		let [gx, gy, gz] = grid_dim;
		let [bx, by, bz] = block_dim;
		check(
			unsafe {
				launch_kernel(stream.stream.as_ptr(), self.handle.as_ptr(), gx, gy, gz, bx, by, bz, shared_mem_bytes, args.as_mut_ptr())
			},
			"x17ai_hip_launch_kernel()",
		)
	}
}

// ---------------------------------------------------------------- event timer

pub struct HipEventTimer {
	timer: NonNull<HipTimerHandle>,
}

impl HipEventTimer {
	pub fn new(stream: &HipStream) -> DevResult<Self> {
		let timer = take(
			unsafe { create_timer(stream.ctx.as_ptr(), stream.stream.as_ptr()) },
			"x17ai_hip_create_timer()",
		)?;
		Ok(Self { timer })
	}

	pub fn start(&self) -> DevResult<()> {
		check(unsafe { timer_start(self.timer.as_ptr()) }, "x17ai_hip_timer_start()")
	}

	pub fn stop(&self) -> DevResult<()> {
		check(unsafe { timer_stop(self.timer.as_ptr()) }, "x17ai_hip_timer_stop()")
	}

	/// Waits for the stop event; seconds between the two events on the device's stream.
	pub fn elapsed_seconds(&self) -> DevResult<f64> {
		let mut seconds = 0.0_f64;
		check(
			unsafe { timer_elapsed_seconds(self.timer.as_ptr(), &raw mut seconds) },
			"x17ai_hip_timer_elapsed_seconds()",
		)?;
		Ok(seconds)
	}
}

impl Drop for HipEventTimer {
	fn drop(&mut self) {
		ignore(unsafe { destroy_timer(self.timer.as_ptr()) });
	}
}
