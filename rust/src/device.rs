// Device memory and the stream for the GPU ops: the few HIP runtime calls the host side needs.
// UNCOMPILED in this repository (no Rust toolchain in the image it was written in).
//
// `DeviceBuf<T>` owns one hipMalloc block; `DeviceArray<T>` is a shared `DeviceBuf<T>` with extents, the
// value that travels between GPU ops.  The ops in gpu_ops.rs take their inputs and hand back their
// outputs through the `DeviceIo` trait, which has two implementations for `ComputeContext<f32>`:
//   * without the cargo feature `device_storage` (the crate as it is: host-resident ndarray storage,
//     src/evaluation.rs:183-223) an input is uploaded when it is taken and an output downloaded when
//     it is appended -- every op stages through host arrays;
//   * with the feature, the evaluator's storage and the contexts hold `DeviceArray`s
//     (device_storage.rs has those changes to op.rs / evaluation.rs / variable.rs): consecutive GPU
//     ops pass pointers, and nothing crosses PCIe until a CPU op or the caller asks for a value.
// The `compute` bodies in gpu_ops.rs are the same either way.
use crate::ndarray_ext::{NdArray, NdArrayView};
use crate::op::ComputeContext;
use std::os::raw::{c_int, c_void};
use std::rc::Rc;

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
    pub fn download(&self, shape: &[usize]) -> NdArray<T> where T: num_traits::Zero {
        let mut host = vec![T::zero(); self.len];
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

/// A contiguous row-major array in device memory: one shared allocation plus its extents.
/// Clones share the allocation (a view in the sense of `append_output_view`, src/op.rs:265-287).
pub struct DeviceArray<T> {
    buf: Rc<DeviceBuf<T>>,
    shape: Vec<usize>,
}

impl<T> Clone for DeviceArray<T> {
    fn clone(&self) -> Self {
        DeviceArray { buf: self.buf.clone(), shape: self.shape.clone() }
    }
}

impl<T: Copy> DeviceArray<T> {
    pub fn new(buf: DeviceBuf<T>, shape: &[usize]) -> Self {
        assert_eq!(buf.len(), shape.iter().product::<usize>(), "extents {shape:?} for {} elements", buf.len());
        DeviceArray { buf: Rc::new(buf), shape: shape.to_vec() }
    }
    /// Host -> device (a contiguous copy of a possibly strided view, conv2d.rs:436-452).
    pub fn from_host(view: &NdArrayView<T>) -> Self {
        DeviceArray { buf: Rc::new(DeviceBuf::upload(view)), shape: view.shape().to_vec() }
    }
    /// Device -> host; waits for the stream.
    pub fn to_host(&self) -> NdArray<T> where T: num_traits::Zero {
        self.buf.download(&self.shape)
    }
    pub fn shape(&self) -> &[usize] { &self.shape }
    pub fn ndim(&self) -> usize { self.shape.len() }
    pub fn len(&self) -> usize { self.buf.len() }
    pub fn ptr(&self) -> *const T { self.buf.ptr() }
    /// For the in-place update ops (AdamOp).  The caller holds the array mutably in the evaluator's
    /// sense: a variable registered with allow_mut (src/tensor.rs:735-739) and taken with `dev_in_mut`.
    pub fn ptr_mut(&self) -> *mut T { self.buf.ptr_mut() }
    /// Same storage, other extents (Reshape is a view, array_ops.rs:183-239).
    pub fn reshaped(&self, shape: &[usize]) -> Self {
        assert_eq!(shape.iter().product::<usize>(), self.shape.iter().product::<usize>());
        DeviceArray { buf: self.buf.clone(), shape: shape.to_vec() }
    }
    /// True if nothing else holds the allocation (an op may then overwrite it as its output).
    pub fn is_unique(&self) -> bool { Rc::strong_count(&self.buf) == 1 }
}

/// How a GPU op takes its inputs and hands back its outputs.
pub trait DeviceIo {
    /// The `i`th input on the device.  Like `input(i)` it may be taken once (src/op.rs:206-217).
    fn dev_in(&mut self, i: usize) -> DeviceArray<f32>;
    /// The `i`th input, a variable registered as mutable, for an update in place (`input_mut(i)`,
    /// src/op.rs:239-262).  Every array taken this way is given back with `dev_commit`.
    fn dev_in_mut(&mut self, i: usize) -> DeviceArray<f32>;
    /// Ends the in-place update of input `i`.
    fn dev_commit(&mut self, i: usize, a: DeviceArray<f32>);
    /// A new array as the next output (`append_output`, src/op.rs:300-302).
    fn dev_out(&mut self, buf: DeviceBuf<f32>, shape: &[usize]);
    /// An input handed on unchanged as the next output (`append_output_view`, src/op.rs:265-287).
    fn dev_out_shared(&mut self, a: DeviceArray<f32>);
}

// The crate as it is: everything stages through host arrays.
#[cfg(not(feature = "device_storage"))]
thread_local! {
    // One evaluation runs one op at a time on its thread (src/evaluation.rs:268-345), so the views an
    // op took mutably are parked here between dev_in_mut and dev_commit.  They are 'static only in
    // name: dev_commit removes each one before `compute` returns, while the evaluator's borrow of the
    // variable is still alive.
    static PENDING: std::cell::RefCell<Vec<(usize, crate::ndarray_ext::NdArrayViewMut<'static, f32>)>> =
        std::cell::RefCell::new(Vec::new());
}

#[cfg(not(feature = "device_storage"))]
impl<'v> DeviceIo for ComputeContext<'v, f32> {
    fn dev_in(&mut self, i: usize) -> DeviceArray<f32> {
        DeviceArray::from_host(&self.input(i))
    }
    fn dev_in_mut(&mut self, i: usize) -> DeviceArray<f32> {
        let view = self.input_mut(i);
        let a = DeviceArray::from_host(&view.view());
        let parked: crate::ndarray_ext::NdArrayViewMut<'static, f32> = unsafe { std::mem::transmute(view) };
        PENDING.with(|p| p.borrow_mut().push((i, parked)));
        a
    }
    fn dev_commit(&mut self, i: usize, a: DeviceArray<f32>) {
        let mut view = PENDING.with(|p| {
            let mut p = p.borrow_mut();
            let at = p.iter().position(|(j, _)| *j == i).expect("dev_commit without dev_in_mut");
            p.swap_remove(at).1
        });
        view.assign(&a.to_host());
    }
    fn dev_out(&mut self, buf: DeviceBuf<f32>, shape: &[usize]) {
        self.append_output(buf.download(shape));
    }
    fn dev_out_shared(&mut self, a: DeviceArray<f32>) {
        self.append_output(a.to_host());
    }
}

/// Device-resident storage: the calls below are the ones device_storage.rs adds to ComputeContext.
#[cfg(feature = "device_storage")]
impl<'v> DeviceIo for ComputeContext<'v, f32> {
    fn dev_in(&mut self, i: usize) -> DeviceArray<f32> {
        self.input_device(i) // uploads only what still lives on the host
    }
    fn dev_in_mut(&mut self, i: usize) -> DeviceArray<f32> {
        self.input_device_mut(i) // the variable's device copy; its host copy becomes stale
    }
    fn dev_commit(&mut self, _i: usize, _a: DeviceArray<f32>) {} // updated where it lives
    fn dev_out(&mut self, buf: DeviceBuf<f32>, shape: &[usize]) {
        self.append_device_output(DeviceArray::new(buf, shape));
    }
    fn dev_out_shared(&mut self, a: DeviceArray<f32>) {
        self.append_device_output(a);
    }
}
