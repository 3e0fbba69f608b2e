// src/device/hip.rs -- the HIP device of the tensor API (twin of src/device/cuda.rs:25-101).
// UNCOMPILED HERE: no Rust toolchain in the image this was written in.
//
// One stream per device object; allocation, copies and launches are ordered on it.  Memory is stream-ordered
// (hipMallocAsync / hipFreeAsync inside the shim), copies are asynchronous, and nothing here synchronizes behind the
// caller's back: src/main.rs synchronizes once before it reads results (main.rs:265).

use std::ptr::NonNull;
use std::rc::Rc;

use hip_shim::{HipEventTimer, HipStream};
use crate::{DeviceAllocError, ErrPack, TensorOpError};

use super::{Device, DevicePtr};

pub mod hip_shim;
pub mod attn;            // src/device/cuda/attn.rs with Cuda* -> Hip*; kernel source attn_fwd_i8.hip / attn_meta.cpp
pub mod gemm;            // src/device/cuda/gemm.rs likewise; kernel source gemm_b8.hip / gemm_meta.cpp
pub mod gemm_templates;  // renders common.h (#define list) instead of the askama templates
mod kernel_build;        // integration/rust/kernel_build_hip.rs
mod tensor_check;        // unchanged

pub struct HipDevice {
	name: String,
	stream: HipStream,
}

impl HipDevice {
	/// `device_id` is the HIP device ordinal (HIP_VISIBLE_DEVICES applies).
	pub fn new(device_id: usize) -> Result<Rc<Self>, ErrPack<TensorOpError>> {
		Self::new_named(device_id, format!("HIP:{device_id}"))
	}

	pub fn new_named(device_id: usize, name: String) -> Result<Rc<Self>, ErrPack<TensorOpError>> {
		Ok(Rc::new(Self { name, stream: HipStream::new(device_id)? }))
	}

	pub fn synchronize(&self) -> Result<(), ErrPack<TensorOpError>> {
		self.stream.synchronize()
	}

	/// for the operator modules (gemm, attn): kernels are loaded into and launched on this stream
	pub(crate) fn stream(&self) -> &HipStream {
		&self.stream
	}
}

impl Device for HipDevice {
	fn name(&self) -> &str {
		&self.name
	}

	unsafe fn new_buffer(&self, bytes: usize) -> Result<DevicePtr, DeviceAllocError> {
		match unsafe { self.stream.alloc(bytes) } {
			Ok(ptr) => Ok(ptr),
			Err(_) => Err(DeviceAllocError),
		}
	}

	unsafe fn drop_buffer(&self, device_ptr: DevicePtr, _bytes: usize) {
		unsafe { self.stream.free(device_ptr) }
	}

	unsafe fn upload_data(&self, src: NonNull<u8>, dst: DevicePtr, bytes: usize) -> Result<(), ErrPack<TensorOpError>> {
		unsafe { self.stream.upload_data(src, dst, 0, bytes) }
	}

	unsafe fn download_data(&self, src: DevicePtr, dst: NonNull<u8>, bytes: usize) -> Result<(), ErrPack<TensorOpError>> {
		unsafe { self.stream.download_data(src, dst, 0, bytes) }
	}
}

/// A pair of events on the device's stream (start .. stop), as src/main.rs uses CudaTimer around each launch.
pub struct HipTimer<'d> {
	_device: &'d HipDevice,
	events: HipEventTimer,
}

impl<'d> HipTimer<'d> {
	pub fn new(device: &'d HipDevice) -> Result<Self, ErrPack<TensorOpError>> {
		Ok(Self { _device: device, events: HipEventTimer::new(&device.stream)? })
	}

	pub fn start(&self) -> Result<(), ErrPack<TensorOpError>> {
		self.events.start()
	}

	pub fn stop(&self) -> Result<(), ErrPack<TensorOpError>> {
		self.events.stop()
	}

	pub fn elapsed_seconds(&self) -> Result<f64, ErrPack<TensorOpError>> {
		self.events.elapsed_seconds()
	}
}
