// Device-resident evaluation: what the crate gains under the cargo feature `device_storage`, so that
// consecutive GPU ops (gpu_ops.rs) pass device pointers and nothing crosses PCIe until a CPU op or
// the caller asks for a value.  UNCOMPILED in this repository (no Rust toolchain in the image it was
// written in); meant to live at src/tensor_ops/device_storage.rs.
//
// The storage the evaluator keeps per node (src/evaluation.rs:183-223) and the two enums an op sees
// (src/op.rs:125-136) each get a device kind; a variable gets a device copy that the update ops write
// in place (src/variable.rs:152-155, :685-703).  Three kinds of change:
//
//  (1) edits in place -- a field or an enum variant cannot be added from another module:
//        src/op.rs:125-129     enum OpInput    + Device(Option<DeviceArray<T>>)
//                                               + Variable { env: &'v VariableEnvironment<T>, vid: VariableID,
//                                                            allow_mut: bool, taken: bool }
//        src/op.rs:133-136     enum OpOutput   + Device(DeviceArray<T>)
//        src/op.rs:186-191     struct ComputeContext: `xs` becomes pub(crate);
//                                               + pub(crate) host_copies: Vec<Box<NdArray<T>>>
//                                               + pub(crate) uploads: Option<&'v UploadCache<T>>
//                                               + pub(crate) keys: SmallVec<InputKey>
//        src/op.rs:206-262     `input` / `input_mut`: first `self.make_host(i)` (below), which turns a
//                              Device or Variable input into the host kind those functions know
//        src/variable.rs:152-155  struct VariableEnvironment + pub(crate) device: RefCell<DeviceCopies<F>>
//        src/variable.rs:549, :539, :663, :385, :393  `save`, `iter`, `get_array_by_id` and the namespace
//                              iterators: first `self.sync_host()` (below)
//        src/evaluation.rs:268-345  the evaluator's loop: the three call sites marked in `eval_hooks`
//  (2) new functions on those types: the `impl` blocks below;
//  (3) nothing in gpu_ops.rs: its `compute` bodies go through `DeviceIo` (device.rs) either way.
//
// Ownership rules that keep this sound:
//  * a DeviceArray is immutable once it is an op's output (clones share it); only a variable's device
//    copy is written in place, by an op that holds it through `input_device_mut`, and the evaluator's
//    order (one op at a time, src/evaluation.rs:268) is what serialises those writes, as it does for
//    `RdWrVariable` on the host;
//  * exactly one of a variable's two copies is current: `DeviceCopy::host_stale` says which;
//  * every copy and kernel is enqueued on one stream (device.rs `stream()`), so "written before read"
//    follows from enqueue order; the only waits are in `download`.
#![cfg(feature = "device_storage")]
use super::device::DeviceArray;
use crate::ndarray_ext::{NdArray, NdArrayView, RawNdArrayView};
use crate::op::{ComputeContext, OpError, OpInput, OpOutput, SmallVec};
use crate::tensor::TensorID;
use crate::variable::{VariableEnvironment, VariableID};
use crate::{Float, FxHashMap};
use std::cell::RefCell;

// ------------------------------------------------------------------------------------------------
// variables                                                        src/variable.rs:152-155, :685-703
// ------------------------------------------------------------------------------------------------
pub(crate) struct DeviceCopy<F> {
    array: DeviceArray<F>,
    /// The device copy is ahead of `array_list[vid]`: an update op has written it.
    host_stale: bool,
}
pub(crate) type DeviceCopies<F> = FxHashMap<VariableID, DeviceCopy<F>>;

impl<F: Float> VariableEnvironment<F> {
    /// The variable on the device for reading: uploaded the first time, shared afterwards (the weights
    /// of a training loop go up once and stay).
    pub(crate) fn device_view(&self, vid: VariableID) -> DeviceArray<F> {
        let mut copies = self.device.borrow_mut();
        copies
            .entry(vid)
            .or_insert_with(|| DeviceCopy { array: DeviceArray::from_host(&self.array_list[vid.0].borrow().view()), host_stale: false })
            .array
            .clone()
    }
    /// The variable on the device for an update in place: as above, and the host copy is stale from now on.
    pub(crate) fn device_view_mut(&self, vid: VariableID) -> DeviceArray<F> {
        let a = self.device_view(vid);
        self.device.borrow_mut().get_mut(&vid).unwrap().host_stale = true;
        a
    }
    /// Brings `array_list[vid]` up to date.  Called by `as_view` (src/variable.rs:685) before it borrows.
    pub(crate) fn sync_host_one(&self, vid: VariableID) {
        if let Some(c) = self.device.borrow_mut().get_mut(&vid) {
            if c.host_stale {
                self.array_list[vid.0].borrow_mut().assign(&c.array.to_host());
                c.host_stale = false;
            }
        }
    }
    /// A CPU op is about to write the variable (`as_view_mut`, src/variable.rs:695): the host copy
    /// becomes the only one.
    pub(crate) fn take_to_host(&self, vid: VariableID) {
        self.sync_host_one(vid);
        self.device.borrow_mut().remove(&vid);
    }
    /// Everything a user can reach through the environment (`save`, `iter`, `get_array_by_id`, the
    /// namespaces) sees current values: those entry points call this first.
    pub fn sync_host(&self) {
        let vids: Vec<VariableID> = self.device.borrow().keys().copied().collect();
        for vid in vids {
            self.sync_host_one(vid);
        }
    }
}

// ------------------------------------------------------------------------------------------------
// what an op sees                                                           src/op.rs:125-136, :186-305
// ------------------------------------------------------------------------------------------------
/// (node, output selector) of a stored value, or a placeholder's node: the key under which one
/// evaluation remembers the device copy of a host value, so an array that several GPU ops read (the
/// images: forward convolution and filter gradient) goes up once.
pub(crate) type InputKey = Option<(TensorID, usize)>;
pub(crate) type UploadCache<T> = RefCell<FxHashMap<(TensorID, usize), DeviceArray<T>>>;

impl<'v, T: Float> ComputeContext<'v, T> {
    /// The `i`th input on the device.  May be taken once, like `input(i)` (src/op.rs:206-217).
    pub fn input_device(&mut self, i: usize) -> DeviceArray<T> {
        let key = self.keys.get(i).cloned().flatten();
        let x = self.xs.get_mut(i).unwrap_or_else(|| panic!("Bad op impl: input index out of range."));
        let twice = || -> ! { panic!("Bad op impl: input({i})/input_mut({i}) cannot be called twice") };
        match x {
            OpInput::Device(a) => a.take().unwrap_or_else(|| twice()),
            OpInput::Variable { env, vid, taken, .. } => {
                if std::mem::replace(taken, true) {
                    twice()
                }
                env.device_view(*vid)
            }
            OpInput::NonVariable(a) | OpInput::RdOnlyVariable(a) => {
                let view = a.take().unwrap_or_else(|| twice());
                match (key, self.uploads) {
                    (Some(k), Some(cache)) => cache.borrow_mut().entry(k).or_insert_with(|| DeviceArray::from_host(&view)).clone(),
                    _ => DeviceArray::from_host(&view),
                }
            }
            OpInput::RdWrVariable(_) => panic!("Bad op impl: cannot perform mutable borrowing for input({i}). Use input_device_mut() instead."),
        }
    }

    /// The `i`th input, a variable registered with allow_mut, for an update in place
    /// (`input_mut(i)`, src/op.rs:239-262).
    pub fn input_device_mut(&mut self, i: usize) -> DeviceArray<T> {
        match self.xs.get_mut(i) {
            Some(OpInput::Variable { env, vid, allow_mut: true, taken }) => {
                if std::mem::replace(taken, true) {
                    panic!("Bad op impl: input({i})/input_mut({i}) cannot be called twice");
                }
                env.device_view_mut(*vid)
            }
            Some(_) => panic!("Bad op impl: cannot perform mutable borrowing for input({i})"),
            None => panic!("Bad op impl: {i}'s input doesn't exist."),
        }
    }

    /// Turns input `i` into the host kind `input` / `input_mut` (src/op.rs:206-262) work on.  A CPU op
    /// behind a GPU op pays one download here; the array it gets lives as long as the context.
    pub(crate) fn make_host(&mut self, i: usize) {
        let host = match self.xs.get_mut(i) {
            Some(OpInput::Device(a)) => match a.take() {
                Some(a) => {
                    self.host_copies.push(Box::new(a.to_host()));
                    // the box does not move when the vector grows, and the context outlives the view
                    let raw: RawNdArrayView<T> = self.host_copies.last().unwrap().raw_view();
                    OpInput::NonVariable(Some(unsafe { raw.deref_into_view() }))
                }
                None => return, // taken already: `input` reports it
            },
            Some(OpInput::Variable { env, vid, allow_mut, taken }) => {
                if *taken {
                    OpInput::NonVariable(None)
                } else if *allow_mut {
                    env.take_to_host(*vid);
                    OpInput::RdWrVariable(Some(env.as_view_mut(*vid)))
                } else {
                    env.sync_host_one(*vid);
                    OpInput::RdOnlyVariable(Some(env.as_view(*vid)))
                }
            }
            _ => return,
        };
        self.xs[i] = host;
    }

    /// A device array as the next output (`append_output`, src/op.rs:300-302).
    pub fn append_device_output(&mut self, y: DeviceArray<T>) {
        self.ys.push(OpOutput::Device(y));
    }
}

// ------------------------------------------------------------------------------------------------
// the evaluator                                                          src/evaluation.rs:183-365
// ------------------------------------------------------------------------------------------------
/// What `OpOutputStorage::get` (src/evaluation.rs:203-213) hands out once values can live on the device.
pub(crate) enum Stored<F: Float> {
    Host(RawNdArrayView<F>),
    Device(DeviceArray<F>),
}

/// `OpOutputStorage::get`: the two host kinds as before, the device kind by a shared handle.
pub(crate) fn storage_get<F: Float>(ys: &Result<SmallVec<OpOutput<F>>, OpError>, selector: usize) -> Result<Stored<F>, OpError> {
    match ys {
        Ok(ys) => Ok(match &ys[selector] {
            OpOutput::Owned(arr) => Stored::Host(arr.raw_view()),
            OpOutput::View(arr) => Stored::Host(arr.clone()),
            OpOutput::Device(arr) => Stored::Device(arr.clone()),
        }),
        Err(e) => Err(e.clone()),
    }
}

/// `OpOutputStorage::take` (src/evaluation.rs:215-223): a requested tensor comes down here, and only
/// here -- the values between the feeds and the requested tensors never leave the device.
pub(crate) fn storage_take<F: Float>(y: OpOutput<F>) -> NdArray<F> {
    match y {
        OpOutput::Owned(y) => y,
        OpOutput::View(y) => unsafe { y.deref_into_view() }.to_owned(),
        OpOutput::Device(y) => y.to_host(),
    }
}

/// The three places where `Graph::eval` (src/evaluation.rs:254-365) changes.
pub(crate) mod eval_hooks {
    use super::*;

    /// :292-309, the input of one incoming edge.  Variables are no longer borrowed here: whether the op
    /// wants the host or the device copy is known only when it asks, so the choice is deferred to
    /// `input` / `input_device`.
    pub(crate) fn gather<'v, F: Float>(
        placeholder: Option<NdArrayView<'v, F>>,
        variable: Option<(VariableID, bool)>, // (id, allow_mut) of incoming.get_variable_id(self)
        env: &'v VariableEnvironment<F>,
        stored: impl FnOnce() -> Result<Stored<F>, OpError>, // storage.get(incoming.id, incoming.array_selector)
    ) -> Result<OpInput<'v, F>, OpError> {
        if let Some(view) = placeholder {
            Ok(OpInput::new_non_variable(view))
        } else if let Some((vid, allow_mut)) = variable {
            Ok(OpInput::Variable { env, vid, allow_mut, taken: false })
        } else {
            stored().map(|s| match s {
                Stored::Host(raw) => OpInput::new_non_variable(unsafe { raw.deref_into_view() }),
                Stored::Device(a) => OpInput::Device(Some(a)),
            })
        }
    }

    /// :319-325, the context of one op: as `ComputeContext::new(op_inputs)` plus the evaluation's
    /// upload cache and the key of every input (`Some((incoming.id, incoming.array_selector))` for
    /// placeholders and stored values, `None` for variables, which have their own device copies).
    pub(crate) fn context<'v, F: Float>(xs: SmallVec<OpInput<'v, F>>, keys: SmallVec<InputKey>, uploads: &'v UploadCache<F>) -> ComputeContext<'v, F> {
        let mut ctx = ComputeContext::new(xs);
        ctx.keys = keys;
        ctx.uploads = Some(uploads);
        ctx
    }

    /// :344-361, the values handed back to the caller: a variable is read after `env.sync_host_one(vid)`,
    /// a normal tensor through `storage_take`.
    pub(crate) fn returned_variable<F: Float>(env: &VariableEnvironment<F>, vid: VariableID) -> NdArray<F> {
        env.sync_host_one(vid);
        env.array_list[vid.0].clone().into_inner()
    }
}

// What this changes for a training step such as examples/cnn_mnist.rs: with host storage every GPU
// node uploads its inputs and downloads its outputs -- the im2col columns, the largest arrays of the
// step, go down after the forward convolution and up again for the filter gradient; with device
// storage the step moves the fed images up once and the requested tensors down, and the arrays Adam
// updates stay where the kernels write them.
