"""ctypes front-end of libag_host.so: the host-side operator layer (graph, grad, evaluator,
variables, Adam) that mirrors rust-autograd's `op::Op` interface for the GPU path.

The names follow the reference: `VariableEnvironment` (src/variable.rs:152), `Context`
(`env.run(|ctx| ...)`, src/variable.rs:650), `Tensor` handles and the `tensor_ops` builders
(src/tensor_ops/mod.rs), `grad` (src/tensor_ops/mod.rs:94), `optimizers.Adam`
(src/optimizers/adam.rs:48).  A panic of the reference becomes `Panic`; an `OpError` returned by
`eval` becomes an `OpError` instance in the result list, as `Result::Err` does there.
"""
import ctypes as C
import os

import numpy as np

from . import capi

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB = None

_i, _f, _p, _s, _z = C.c_int, C.c_float, C.c_void_p, C.c_char_p, C.c_size_t
_ip, _fp, _lp = C.POINTER(C.c_int), C.POINTER(C.c_float), C.POINTER(C.c_int64)

PROTOTYPES = {
    "agh_last_error": (_s, []),
    "agh_env_new": (_p, []),
    "agh_env_free": (None, [_p]),
    "agh_env_set": (_i, [_p, _s, _s, _fp, _lp, _i]),
    "agh_env_find": (_i, [_p, _s, _s]),
    "agh_env_shape": (_i, [_p, _i, _lp, _i]),
    "agh_env_read": (_i, [_p, _i, _fp, _z]),
    "agh_env_write": (_i, [_p, _i, _fp, _z]),
    "agh_env_len": (_i, [_p]),
    "agh_env_save": (_i, [_p, _s]),
    "agh_env_load": (_p, [_s]),
    "agh_env_initialize": (_i, [_p, _s]),
    "agh_env_file_rewrite": (_i, [_s, _s]),
    "agh_ctx_new": (_p, [_p]),
    "agh_ctx_free": (None, [_p]),
    "agh_variable": (_i, [_p, _i]),
    "agh_placeholder": (_i, [_p, _s, _lp, _i]),
    "agh_scalar": (_i, [_p, _f]),
    "agh_conv2d": (_i, [_p, _i, _i, _i, _i, _i]),
    "agh_conv2d_with_columns": (_i, [_p, _i, _i, _i, _i, _i]),
    "agh_conv2d_transpose": (_i, [_p, _i, _i, _i, _i, _i]),
    "agh_max_pool2d": (_i, [_p, _i, _i, _i, _i]),
    "agh_matmul": (_i, [_p, _i, _i]),
    "agh_batch_matmul": (_i, [_p, _i, _i, _i, _i]),
    "agh_reduce_sum": (_i, [_p, _i, _ip, _i, _i]),
    "agh_reduce_mean": (_i, [_p, _i, _ip, _i, _i]),
    "agh_sum_all": (_i, [_p, _i]),
    "agh_relu": (_i, [_p, _i]),
    "agh_add": (_i, [_p, _i, _i]),
    "agh_mul": (_i, [_p, _i, _i]),
    "agh_add_n": (_i, [_p, _ip, _i]),
    "agh_nth_tensor": (_i, [_p, _i, _i]),
    "agh_reshape": (_i, [_p, _i, _lp, _i]),
    "agh_sparse_softmax_cross_entropy": (_i, [_p, _i, _i]),
    "agh_stop_gradient": (_i, [_p, _i]),
    "agh_grad": (_i, [_p, _ip, _i, _ip, _i, _ip]),
    "agh_grad_with_default": (_i, [_p, _ip, _ip, _i, _ip, _i, _ip]),
    "agh_grad_helper": (_i, [_p, _ip, _i, _s, _ip, _ip, _i]),
    "agh_num_nodes": (_i, [_p]),
    "agh_fused_pairs": (_i, [_p]),
    "agh_reused_copies": (C.c_longlong, []),
    "agh_set_shortcuts": (None, [_i]),
    "agh_op_name": (_s, [_p, _i]),
    "agh_topo_rank": (_i, [_p, _i]),
    "agh_num_inputs": (_i, [_p, _i]),
    "agh_adam_new": (_p, [_p, _s, _ip, _i, _f, _f, _f, _f]),
    "agh_adam_free": (None, [_p]),
    "agh_adam_update_op": (_i, [_p, _p, _ip, _ip, _i]),
    "agh_eval": (_i, [_p, _ip, _i, C.POINTER(_s), C.POINTER(_fp), C.POINTER(_lp), _ip, _i]),
    "agh_eval_nowait": (_i, [_p, _ip, _i, C.POINTER(_s), C.POINTER(_fp), C.POINTER(_lp), _ip, _i]),
    "agh_synchronize": (_i, []),
    "agh_result_status": (_i, [_p, _i]),
    "agh_result_message": (_s, [_p, _i]),
    "agh_result_shape": (_i, [_p, _i, _lp, _i]),
    "agh_result_read": (_i, [_p, _i, _fp, _z]),
}


class Panic(RuntimeError):
    """The reference would have panicked (graph misuse, missing placeholder value, ...)."""


def host_library_path():
    return os.path.join(_HERE, "libag_host.so")


def lib():
    global _LIB
    if _LIB is None:
        path = host_library_path()
        if not os.path.exists(path):
            raise RuntimeError(f"{path} is not built; run rust-autograd_amd/csrc/build.sh")
        capi.lib()  # the kernel library must be there as well; no fallback exists
        L = C.CDLL(path)
        for name, (res, args) in PROTOTYPES.items():
            fn = getattr(L, name)
            fn.restype, fn.argtypes = res, args
        _LIB = L
    return _LIB


def _check(rc):
    if rc is None or (isinstance(rc, int) and rc < 0):
        raise Panic(lib().agh_last_error().decode())
    return rc


def _ints(xs):
    xs = list(xs)
    return (C.c_int * max(len(xs), 1))(*xs), len(xs)


def _shape(shape):
    shape = list(shape)
    return (C.c_int64 * max(len(shape), 1))(*shape), len(shape)


def _f32(a):
    return np.ascontiguousarray(a, dtype=np.float32)


class PersistError(Exception):
    """A saved environment that cannot be read, written or parsed (`Err(Box<dyn Error>)` of
    `VariableEnvironment::save/load/initialize`, src/variable.rs:487-503, 549-563)."""


def _check_file(rc):
    if rc is None or (isinstance(rc, int) and rc < 0):
        raise PersistError(lib().agh_last_error().decode())
    return rc


def rewrite_saved_environment(src_path, dst_path):
    """Parses a saved environment and writes it again, in host memory only."""
    _check_file(lib().agh_env_file_rewrite(os.fsencode(src_path), os.fsencode(dst_path)))


class VariableEnvironment:
    def __init__(self, _handle=None):
        self._h = _handle if _handle is not None else _check(lib().agh_env_new())

    @classmethod
    def load(cls, path):
        """`VariableEnvironment::<f32>::load(path)` (src/variable.rs:487-490)."""
        return cls(_check_file(lib().agh_env_load(os.fsencode(path))))

    def save(self, path):
        """`env.save(path)` (src/variable.rs:549-554): the reference's JSON format."""
        _check_file(lib().agh_env_save(self._h, os.fsencode(path)))

    def initialize(self, path):
        """`env.initialize(path)` (src/variable.rs:493-503): replaces arrays and names."""
        _check_file(lib().agh_env_initialize(self._h, os.fsencode(path)))

    def __len__(self):
        return _check(lib().agh_env_len(self._h))

    def __del__(self):
        if getattr(self, "_h", None) and _LIB is not None:
            _LIB.agh_env_free(self._h)
            self._h = None

    def set(self, name, array, namespace=""):
        a = _f32(array)
        sh, rank = _shape(a.shape)
        return _check(lib().agh_env_set(self._h, namespace.encode(), name.encode(), a.ctypes.data_as(_fp), sh, rank))

    def find(self, name, namespace=""):
        vid = lib().agh_env_find(self._h, namespace.encode(), name.encode())
        return None if vid < 0 else vid

    def array(self, var_id):
        buf = (C.c_int64 * 8)()
        rank = _check(lib().agh_env_shape(self._h, var_id, buf, 8))
        out = np.empty([buf[i] for i in range(rank)], dtype=np.float32)
        _check(lib().agh_env_read(self._h, var_id, out.ctypes.data_as(_fp), out.size))
        return out

    def write(self, var_id, array):
        """Overwrites a variable in place (what `get_array_by_id(id).borrow_mut()` is used for)."""
        a = _f32(array)
        _check(lib().agh_env_write(self._h, var_id, a.ctypes.data_as(_fp), a.size))

    def context(self):
        return Context(self)


class OpError(Exception):
    KINDS = {1: "NdArrayError", 2: "IncompatibleShape", 3: "TypeUnsupported", 4: "InvalidDims", 5: "OutOfBounds",
             100: "HipError"}

    def __init__(self, kind, message):
        super().__init__(f"{self.KINDS.get(kind, kind)}: {message}")
        self.kind = self.KINDS.get(kind, str(kind))
        self.message = message


class Tensor:
    __slots__ = ("ctx", "id")

    def __init__(self, ctx, tid):
        self.ctx, self.id = ctx, _check(tid)

    def __add__(self, o):
        return self.ctx.add(self, o)

    def __mul__(self, o):
        return self.ctx.mul(self, o)

    @property
    def op_name(self):
        return lib().agh_op_name(self.ctx._h, self.id).decode()

    @property
    def topo_rank(self):
        return lib().agh_topo_rank(self.ctx._h, self.id)

    @property
    def num_inputs(self):
        return lib().agh_num_inputs(self.ctx._h, self.id)

    def eval(self, feeds=None):
        r = self.ctx.eval([self], feeds)[0]
        if isinstance(r, OpError):
            raise r
        return r


class Context:
    def __init__(self, env):
        self.env = env
        self._h = _check(lib().agh_ctx_new(env._h))

    def __del__(self):
        if getattr(self, "_h", None) and _LIB is not None:
            _LIB.agh_ctx_free(self._h)
            self._h = None

    def _t(self, tid):
        return Tensor(self, tid)

    # -- sources ------------------------------------------------------------------------------
    def variable(self, var, namespace=""):
        if isinstance(var, str):
            vid = self.env.find(var, namespace)
            if vid is None:
                raise Panic(f"variable array not found: {var}")
            var = vid
        return self._t(lib().agh_variable(self._h, var))

    def placeholder(self, name, shape):
        sh, rank = _shape(shape)
        return self._t(lib().agh_placeholder(self._h, name.encode(), sh, rank))

    def scalar(self, v):
        return self._t(lib().agh_scalar(self._h, float(v)))

    # -- tensor_ops ---------------------------------------------------------------------------
    def conv2d(self, x, w, pad, stride, columns=False):
        """columns=True: materialise the im2col columns like the reference, whatever the geometry."""
        fn = lib().agh_conv2d_with_columns if columns else lib().agh_conv2d
        return self._t(fn(self._h, x.id, w.id, pad, stride, 1))

    def dilated_conv2d(self, x, w, pad, stride, dilation, columns=False):
        fn = lib().agh_conv2d_with_columns if columns else lib().agh_conv2d
        return self._t(fn(self._h, x.id, w.id, pad, stride, dilation))

    def conv2d_transpose(self, x, w, pad, stride):
        return self._t(lib().agh_conv2d_transpose(self._h, x.id, w.id, pad, stride, 1))

    def dilated_conv2d_transpose(self, x, w, pad, stride, dilation):
        return self._t(lib().agh_conv2d_transpose(self._h, x.id, w.id, pad, stride, dilation))

    def max_pool2d(self, x, pool_size, pad, stride):
        return self._t(lib().agh_max_pool2d(self._h, x.id, pool_size, pad, stride))

    def matmul(self, a, b):
        return self._t(lib().agh_matmul(self._h, a.id, b.id))

    def batch_matmul(self, a, b, trans_a=False, trans_b=False):
        return self._t(lib().agh_batch_matmul(self._h, a.id, b.id, int(trans_a), int(trans_b)))

    def reduce_sum(self, x, axes, keep_dims=False):
        ax, n = _ints(axes)
        return self._t(lib().agh_reduce_sum(self._h, x.id, ax, n, int(keep_dims)))

    def reduce_mean(self, x, axes, keep_dims=False):
        ax, n = _ints(axes)
        return self._t(lib().agh_reduce_mean(self._h, x.id, ax, n, int(keep_dims)))

    def sum_all(self, x):
        return self._t(lib().agh_sum_all(self._h, x.id))

    def relu(self, x):
        return self._t(lib().agh_relu(self._h, x.id))

    def add(self, a, b):
        return self._t(lib().agh_add(self._h, a.id, b.id))

    def mul(self, a, b):
        return self._t(lib().agh_mul(self._h, a.id, b.id))

    def add_n(self, xs):
        ids, n = _ints(t.id for t in xs)
        return self._t(lib().agh_add_n(self._h, ids, n))

    def nth_tensor(self, x, n):
        return self._t(lib().agh_nth_tensor(self._h, x.id, n))

    def reshape(self, x, shape):
        sh, rank = _shape(shape)
        return self._t(lib().agh_reshape(self._h, x.id, sh, rank))

    def sparse_softmax_cross_entropy(self, logits, labels):
        return self._t(lib().agh_sparse_softmax_cross_entropy(self._h, logits.id, labels.id))

    def stop_gradient(self, x):
        return self._t(lib().agh_stop_gradient(self._h, x.id))

    def grad(self, ys, xs):
        yi, ny = _ints(t.id for t in ys)
        xi, nx = _ints(t.id for t in xs)
        out = (C.c_int * max(nx, 1))()
        _check(lib().agh_grad(self._h, yi, ny, xi, nx, out))
        return [self._t(out[i]) for i in range(nx)]

    def grad_with_default(self, ys, xs, ys_grads):
        yi, ny = _ints(t.id for t in ys)
        gi, _ = _ints(t.id for t in ys_grads)
        xi, nx = _ints(t.id for t in xs)
        out = (C.c_int * max(nx, 1))()
        _check(lib().agh_grad_with_default(self._h, yi, gi, ny, xi, nx, out))
        return [self._t(out[i]) for i in range(nx)]

    def grad_helper(self, losses, namespace=""):
        li, n = _ints(t.id for t in losses)
        cap = 4096
        vs, gs = (C.c_int * cap)(), (C.c_int * cap)()
        cnt = _check(lib().agh_grad_helper(self._h, li, n, namespace.encode(), vs, gs, cap))
        return [self._t(vs[i]) for i in range(cnt)], [self._t(gs[i]) for i in range(cnt)]

    @property
    def num_nodes(self):
        return lib().agh_num_nodes(self._h)

    @property
    def fused_pairs(self):
        return lib().agh_fused_pairs(self._h)

    # -- evaluation ---------------------------------------------------------------------------
    def _evaluate(self, entry, tensors, feeds):
        feeds = feeds or {}
        ids, n = _ints(t.id for t in tensors)
        arrays = [_f32(a) for a in feeds.values()]
        nf = len(arrays)
        names = (_s * max(nf, 1))(*[k.encode() for k in feeds])
        data = (_fp * max(nf, 1))(*[a.ctypes.data_as(_fp) for a in arrays])
        shapes_keep = [_shape(a.shape)[0] for a in arrays]
        shapes = (_lp * max(nf, 1))(*[C.cast(s, _lp) for s in shapes_keep])
        ranks, _ = _ints(a.ndim for a in arrays)
        _check(entry(self._h, ids, n, names, data, shapes, ranks, nf))
        return n

    def eval(self, tensors, feeds=None):
        n = self._evaluate(lib().agh_eval, tensors, feeds)
        out = []
        buf = (C.c_int64 * 8)()
        for i in range(n):
            st = lib().agh_result_status(self._h, i)
            if st != 0:
                out.append(OpError(st, lib().agh_result_message(self._h, i).decode()))
                continue
            rank = _check(lib().agh_result_shape(self._h, i, buf, 8))
            a = np.empty([buf[k] for k in range(rank)], dtype=np.float32)
            _check(lib().agh_result_read(self._h, i, a.ctypes.data_as(_fp), a.size))
            out.append(a)
        return out

    def run(self, tensors, feeds=None):
        """Evaluates `tensors` for their effects (optimizer updates) without waiting for the device and without
        reading anything back: returns None per tensor, or its OpError.  The next graph can be built while the
        device works; reading a variable (or any eval) waits as needed."""
        n = self._evaluate(lib().agh_eval_nowait, tensors, feeds)
        out = []
        for i in range(n):
            st = lib().agh_result_status(self._h, i)
            out.append(OpError(st, lib().agh_result_message(self._h, i).decode()) if st != 0 else None)
        return out


def reused_copies():
    """How often an op of this thread found a rearranged copy it needed already made by an earlier op."""
    return lib().agh_reused_copies()


def set_shortcuts(on):
    """Evaluation-time shortcuts (fused pairs, reused copies) on or off, process-wide; same results either way."""
    lib().agh_set_shortcuts(int(bool(on)))


def synchronize():
    """Waits until the device has finished everything enqueued so far."""
    _check(lib().agh_synchronize())


class Adam:
    """optimizers::Adam::new(alpha, eps, b1, b2, var_ids, env, namespace) (src/optimizers/adam.rs:60-91)."""

    def __init__(self, env, var_ids, alpha=0.001, eps=1e-08, b1=0.9, b2=0.999, namespace="adam"):
        ids, n = _ints(var_ids)
        self.env = env
        self._h = lib().agh_adam_new(env._h, namespace.encode(), ids, n, alpha, eps, b1, b2)
        if not self._h:
            raise Panic(lib().agh_last_error().decode())

    def __del__(self):
        if getattr(self, "_h", None) and _LIB is not None:
            _LIB.agh_adam_free(self._h)
            self._h = None

    def get_update_op(self, params, grads, ctx):
        pi, n = _ints(t.id for t in params)
        gi, _ = _ints(t.id for t in grads)
        return ctx._t(lib().agh_adam_update_op(self._h, ctx._h, pi, gi, n))

    def update(self, params, grads, ctx, feeds=None):
        """Optimizer::update (optimizers/mod.rs:63-81): runs the updates; the call does not wait for the device."""
        r = ctx.run([self.get_update_op(params, grads, ctx)], feeds)[0]
        if isinstance(r, OpError):
            raise r
