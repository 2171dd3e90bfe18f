// Device memory and the stream for the GPU ops: the few HIP runtime calls the host side needs.
// UNCOMPILED in this repository (no Rust toolchain in the image it was written in).
//
// `DeviceBuf<T>` owns one hipMalloc block.  With the crate as it is (host-resident ndarray
// storage, src/evaluation.rs:183-223) every op uploads its inputs and downloads its outputs; once
// the evaluator's storage holds `DeviceBuf`s the copies disappear and the `compute` bodies in
// gpu_ops.rs stay as they are.
use crate::ndarray_ext::{NdArray, NdArrayView};
use std::os::raw::{c_int, c_void};

#[link(name = "amdhip64")]
extern "C" {
    fn hipMalloc(ptr: *mut *mut c_void, bytes: usize) -> c_int;
    fn hipFree(ptr: *mut c_void) -> c_int;
    fn hipMemcpyAsync(dst: *mut c_void, src: *const c_void, bytes: usize, kind: c_int, stream: *mut c_void) -> c_int;
    fn hipStreamSynchronize(stream: *mut c_void) -> c_int;
}
const HIP_MEMCPY_HOST_TO_DEVICE: c_int = 1;
const HIP_MEMCPY_DEVICE_TO_HOST: c_int = 2;

/// The stream every op of one graph evaluation enqueues on (the null stream: one evaluator thread
/// per graph, src/graph.rs:17-20).
pub fn stream() -> super::hip_ffi::AgStream {
    std::ptr::null_mut()
}

pub struct DeviceBuf<T> {
    ptr: *mut T,
    len: usize,
}

impl<T: Copy> DeviceBuf<T> {
    pub fn alloc(len: usize) -> Self {
        let mut raw: *mut c_void = std::ptr::null_mut();
        let bytes = std::cmp::max(len, 1) * std::mem::size_of::<T>();
        assert_eq!(unsafe { hipMalloc(&mut raw, bytes) }, 0, "hipMalloc({bytes}) failed");
        DeviceBuf { ptr: raw as *mut T, len }
    }
    /// Contiguous copy of a (possibly strided) view, as the reference's ops make before calling
    /// BLAS (conv2d.rs:436-452), then host -> device.
    pub fn upload(view: &NdArrayView<T>) -> Self {
        let owned = view.as_standard_layout();
        let host = owned.as_slice().expect("standard layout");
        let buf = Self::alloc(host.len());
        let bytes = host.len() * std::mem::size_of::<T>();
        assert_eq!(unsafe { hipMemcpyAsync(buf.ptr as *mut c_void, host.as_ptr() as *const c_void, bytes,
                                           HIP_MEMCPY_HOST_TO_DEVICE, stream()) }, 0);
        assert_eq!(unsafe { hipStreamSynchronize(stream()) }, 0); // `owned` may be a temporary
        buf
    }
    /// Device -> host into a new array of `shape`; waits for the stream.
    pub fn download(&self, shape: &[usize]) -> NdArray<T> where T: Default {
        let mut host = vec![T::default(); self.len];
        let bytes = self.len * std::mem::size_of::<T>();
        assert_eq!(unsafe { hipMemcpyAsync(host.as_mut_ptr() as *mut c_void, self.ptr as *const c_void, bytes,
                                           HIP_MEMCPY_DEVICE_TO_HOST, stream()) }, 0);
        assert_eq!(unsafe { hipStreamSynchronize(stream()) }, 0);
        NdArray::from_shape_vec(ndarray::IxDyn(shape), host).expect("shape matches the buffer")
    }
    pub fn len(&self) -> usize { self.len }
    pub fn ptr(&self) -> *const T { self.ptr }
    pub fn ptr_mut(&self) -> *mut T { self.ptr }
    pub fn void(&self) -> *mut c_void { self.ptr as *mut c_void }
    pub fn bytes(&self) -> usize { self.len * std::mem::size_of::<T>() }
}

impl<T> Drop for DeviceBuf<T> {
    fn drop(&mut self) {
        unsafe { hipFree(self.ptr as *mut c_void) };
    }
}
