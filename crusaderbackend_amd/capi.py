"""ctypes binding of the C ABI declared in include/crusader_hip.h.

This module is plumbing for tests and the benchmark: it loads the in-tree
``lib/libcrusader_hip.so`` and passes raw device pointers (``tensor.data_ptr()``) and sizes
straight through. There is no CPU fallback: if the shared library is missing, loading raises.
"""
import ctypes
import os

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "lib", "libcrusader_hip.so")

CRB_OK = 0
CRB_EINVAL_SHAPE = -1
CRB_ENULL = -2
CRB_EHIP = -3
CRB_EWORKSPACE = -4
CRB_FLAG_RELU = 1

_u32 = ctypes.c_uint32
_ptr = ctypes.c_void_p


class ConvGeom(ctypes.Structure):
    """Mirror of ``crb_conv_geom``."""

    _fields_ = [(n, _u32) for n in ("N", "IC", "IH", "IW", "OC", "FH", "FW", "OH", "OW", "sH", "sW", "pH", "pW")]

    @classmethod
    def make(cls, N, IC, IH, IW, OC, FH, FW, sH=1, sW=1, pH=0, pW=0, OH=None, OW=None):
        if OH is None:
            OH = (IH - FH + 2 * pH) // sH + 1
        if OW is None:
            OW = (IW - FW + 2 * pW) // sW + 1
        return cls(N, IC, IH, IW, OC, FH, FW, OH, OW, sH, sW, pH, pW)


# name -> (restype, argtypes); every symbol include/crusader_hip.h declares
SIGNATURES = {
    "crb_abi_version": (ctypes.c_int, []),
    "crb_last_error_string": (ctypes.c_char_p, []),
    "crb_release_workspace": (None, []),
    "crb_bind_workspace": (ctypes.c_int, [_ptr, ctypes.c_size_t, _ptr]),
    "crb_gemm_workspace_bytes": (ctypes.c_size_t, [_u32, _u32, _u32, _u32]),
    "crb_conv_fwd_workspace_bytes": (ctypes.c_size_t, [ctypes.POINTER(ConvGeom), ctypes.c_int]),
    "crb_conv_dgrad_workspace_bytes": (ctypes.c_size_t, [ctypes.POINTER(ConvGeom), ctypes.c_int]),
    "crb_conv_bias_grad_workspace_bytes": (ctypes.c_size_t, [_u32, _u32, _u32]),
    "crb_conv_wgrad_noalloc": (ctypes.c_int, [_ptr, _ptr, _ptr, ctypes.POINTER(ConvGeom), _ptr]),
    "crb_sgemm_nn": (ctypes.c_int, [_ptr, _ptr, _ptr, _u32, _u32, _u32, _u32, _ptr]),
    "crb_sgemm_tn": (ctypes.c_int, [_ptr, _ptr, _ptr, _u32, _u32, _u32, _u32, _ptr]),
    "crb_sgemm_nt": (ctypes.c_int, [_ptr, _ptr, _ptr, _u32, _u32, _u32, _ptr]),
    "crb_sgemm_nta": (ctypes.c_int, [_ptr, _ptr, _ptr, _u32, _u32, _u32, _u32, _ptr]),
    "crb_linear_fwd": (ctypes.c_int, [_ptr, _ptr, _ptr, _ptr, _u32, _u32, _u32, _u32, _ptr]),
    "crb_linear_dgrad": (ctypes.c_int, [_ptr, _ptr, _ptr, _u32, _u32, _u32, _ptr]),
    "crb_linear_wgrad": (ctypes.c_int, [_ptr, _ptr, _ptr, _ptr, _u32, _u32, _u32, _ptr]),
    "crb_conv_fwd": (ctypes.c_int, [_ptr, _ptr, _ptr, _ptr, ctypes.POINTER(ConvGeom), _u32, _ptr]),
    "crb_conv_dgrad": (ctypes.c_int, [_ptr, _ptr, _ptr, ctypes.POINTER(ConvGeom), _ptr]),
    "crb_conv_wgrad_workspace_bytes": (ctypes.c_size_t, [ctypes.POINTER(ConvGeom)]),
    "crb_conv_wgrad": (ctypes.c_int, [_ptr, _ptr, _ptr, ctypes.POINTER(ConvGeom), _ptr, ctypes.c_size_t, _ptr]),
    "crb_conv_bwd": (ctypes.c_int, [_ptr, _ptr, _ptr, _ptr, _ptr, ctypes.POINTER(ConvGeom), _ptr, ctypes.c_size_t, _ptr]),
    "crb_conv_bwd_slices": (_u32, [ctypes.POINTER(ConvGeom)]),
    "crb_conv_bwd_sliced": (ctypes.c_int, [_ptr, _ptr, _ptr, _ptr, ctypes.POINTER(ConvGeom), _ptr, ctypes.c_size_t, _ptr]),
    "crb_sum_slices_multi": (ctypes.c_int, [_ptr, _u32, _ptr]),
    "crb_conv_bias": (ctypes.c_int, [_ptr, _ptr, _u32, _u32, _u32, _ptr]),
    "crb_conv_bias_grad": (ctypes.c_int, [_ptr, _ptr, _u32, _u32, _u32, _ptr]),
    "crb_tensor_add_inplace": (ctypes.c_int, [_ptr, _ptr, _u32, _ptr]),
    "crb_tensor_fill": (ctypes.c_int, [_ptr, ctypes.c_float, _u32, _ptr]),
    "crb_tensor_sub_inplace": (ctypes.c_int, [_ptr, _ptr, _u32, _ptr]),
    "crb_tensor_copy": (ctypes.c_int, [_ptr, _ptr, _u32, _ptr]),
    "crb_tensor_add_clear": (ctypes.c_int, [_ptr, _ptr, _u32, _ptr]),
    "crb_tensor_add": (ctypes.c_int, [_ptr, _ptr, _ptr, _u32, _ptr]),
    "crb_tensor_add_clear_copy": (ctypes.c_int, [_ptr, _ptr, _ptr, _u32, _ptr]),
    "crb_tensor_copy2": (ctypes.c_int, [_ptr, _ptr, _ptr, _u32, _ptr]),
    "crb_tensor_scale_inplace": (ctypes.c_int, [_ptr, ctypes.c_float, _u32, _ptr]),
    "crb_relu_fwd": (ctypes.c_int, [_ptr, _ptr, _u32, _ptr]),
    "crb_relu_bwd": (ctypes.c_int, [_ptr, _ptr, _ptr, _u32, _ptr]),
    "crb_maxpool_fwd": (ctypes.c_int, [_ptr, _ptr, _ptr, _u32, _u32, _u32, _u32, _u32, _u32, _u32, _ptr]),
    "crb_maxpool_bwd": (ctypes.c_int, [_ptr, _ptr, _ptr, _u32, _u32, _u32, _u32, _u32, _u32, _u32, _ptr]),
    "crb_softmax": (ctypes.c_int, [_ptr, _ptr, _u32, _u32, _ptr]),
    "crb_cross_entropy_grad": (ctypes.c_int, [_ptr, _ptr, _ptr, _u32, _ptr]),
    "crb_cross_entropy_scratch_floats": (_u32, [_u32]),
    "crb_cross_entropy_loss": (ctypes.c_int, [_ptr, _ptr, _ptr, _u32, _ptr, _u32, _ptr]),
    "crb_momentum_apply_multi": (ctypes.c_int, [_ptr, _u32, _u32, _ptr]),
    "crb_batchnorm_fwd": (ctypes.c_int, [_ptr, _ptr, _ptr, _ptr, _ptr, _ptr, _ptr, _u32, _u32, _ptr]),
    "crb_batchnorm_bwd": (ctypes.c_int, [_ptr, _ptr, _ptr, _ptr, _ptr, _ptr, _u32, _u32, _ptr]),
    "crb_batchnorm_param_grads": (ctypes.c_int, [_ptr, _ptr, _ptr, _ptr, _u32, _u32, _ptr]),
    "crb_batchnorm_relu_fwd": (ctypes.c_int, [_ptr, _ptr, _ptr, _ptr, _ptr, _ptr, _ptr, _ptr, _ptr, _u32, _u32, _ptr]),
    "crb_batchnorm_relu_bwd": (ctypes.c_int, [_ptr, _ptr, _ptr, _ptr, _ptr, _ptr, _ptr, _ptr, _ptr, _u32, _u32, _ptr]),
    "crb_tensor_add_relu": (ctypes.c_int, [_ptr, _ptr, _ptr, _u32, _ptr]),
    "crb_tensor_relu_grad_copy2": (ctypes.c_int, [_ptr, _ptr, _ptr, _ptr, _ptr, _u32, _ptr]),
    "crb_momentum_apply": (ctypes.c_int, [_ptr, _ptr, _ptr, _u32, ctypes.c_float, ctypes.c_float, ctypes.c_float, _ptr]),
    "crb_images_from_bytes": (ctypes.c_int, [_ptr, _ptr, _u32, _u32, _u32, _u32, ctypes.c_int, ctypes.c_float, ctypes.c_float,
                                             _ptr, _ptr]),
}

_lib = None


def load():
    """Load the HIP library (once) and attach signatures. Raises OSError if it has not been built."""
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            raise OSError(f"{LIB_PATH} not found: build it with `make -C crusaderbackend_amd/csrc`")
        lib = ctypes.CDLL(LIB_PATH)
        for name, (res, args) in SIGNATURES.items():
            fn = getattr(lib, name)
            fn.restype = res
            fn.argtypes = args
        _lib = lib
    return _lib


class CrbError(RuntimeError):
    def __init__(self, status, message):
        super().__init__(f"crb status {status}: {message}")
        self.status = status


def check(status):
    if status != CRB_OK:
        raise CrbError(status, load().crb_last_error_string().decode())


def _p(t):
    return None if t is None else t.data_ptr()


def _stream(stream):
    return None if stream is None else stream.cuda_stream


def prepared(name, *args):
    """A zero-argument callable that issues entry point `name` with `args` converted once (tensors to their device
    addresses, a ConvGeom to a reference to it, the rest as given, in the order of the C declaration). A timing loop over
    the plain wrappers spends 3.5-4.5 us per call in argument conversion, which hides every kernel shorter than that; a
    prepared call costs about a microsecond. The tensors and the geometry must outlive the callable."""
    fn = getattr(load(), name)
    conv, keep = [], []
    for a in args:
        if a is None or isinstance(a, int):
            conv.append(a)
        elif isinstance(a, ConvGeom):
            keep.append(a)
            conv.append(ctypes.byref(a))
        elif hasattr(a, "data_ptr"):
            keep.append(a)
            conv.append(ctypes.c_void_p(a.data_ptr()))
        elif hasattr(a, "cuda_stream"):
            conv.append(ctypes.c_void_p(a.cuda_stream))
        else:
            conv.append(a)
    conv = tuple(conv)

    def call(_keep=keep):
        st = fn(*conv)
        if st != CRB_OK:
            check(st)

    return call


class _Recorder:
    """Stands in for the library while `frozen` runs a wrapper once: passes every call through and notes the launching
    ones (those that return a status) with their converted arguments."""

    def __init__(self, lib):
        self._lib, self.calls = lib, []

    def __getattr__(self, name):
        fn = getattr(self._lib, name)
        if fn.restype is not ctypes.c_int or name == "crb_abi_version":
            return fn  # size queries, error text: needed by the wrapper now, not part of the replay

        def passthrough(*args):
            self.calls.append((fn, args))
            return fn(*args)

        return passthrough


def frozen(fn):
    """Runs `fn` (any composition of the wrappers below) once and returns a zero-argument callable that re-issues the
    same entry points with the same already-converted arguments. For timing loops over short kernels, like `prepared`,
    without spelling the C argument list out. Every tensor `fn` touches must outlive the callable; host-side decisions
    `fn` makes (workspace sizes, branches) are frozen with it."""
    global _lib
    real = load()
    rec = _Recorder(real)
    _lib = rec
    try:
        fn()
    finally:
        _lib = real
    calls = tuple(rec.calls)
    if not calls:  # `fn` does not go through the wrappers (already prepared calls): nothing to freeze
        return fn
    if len(calls) == 1:
        f, a = calls[0]

        def call():
            st = f(*a)
            if st != CRB_OK:
                check(st)
    else:
        def call():
            for f, a in calls:
                st = f(*a)
                if st != CRB_OK:
                    check(st)
    call.keep = fn  # the closure of `fn` holds the tensors
    return call


# Thin helpers over torch CUDA tensors (device memory + streams only; no torch math).
def sgemm_nn(A, B, C, M, N, K, batch=1, stream=None):
    check(load().crb_sgemm_nn(_p(A), _p(B), _p(C), M, N, K, batch, _stream(stream)))


def sgemm_tn(A, B, C, M, N, K, batch=1, stream=None):
    check(load().crb_sgemm_tn(_p(A), _p(B), _p(C), M, N, K, batch, _stream(stream)))


def sgemm_nt(A, B, C, M, N, K, stream=None):
    check(load().crb_sgemm_nt(_p(A), _p(B), _p(C), M, N, K, _stream(stream)))


def sgemm_nta(A, B, C, M, N, K, batch=1, stream=None):
    check(load().crb_sgemm_nta(_p(A), _p(B), _p(C), M, N, K, batch, _stream(stream)))


def linear_fwd(X, W, bias, Y, batch, IN, OUT, flags=0, stream=None):
    check(load().crb_linear_fwd(_p(X), _p(W), _p(bias), _p(Y), batch, IN, OUT, flags, _stream(stream)))


def linear_dgrad(dY, W, dX, batch, IN, OUT, stream=None):
    check(load().crb_linear_dgrad(_p(dY), _p(W), _p(dX), batch, IN, OUT, _stream(stream)))


def linear_wgrad(dY, X, dW, dB, batch, IN, OUT, stream=None):
    check(load().crb_linear_wgrad(_p(dY), _p(X), _p(dW), _p(dB), batch, IN, OUT, _stream(stream)))


def conv_fwd(W, X, Y, bias, geom, flags=0, stream=None):
    check(load().crb_conv_fwd(_p(W), _p(X), _p(Y), _p(bias), ctypes.byref(geom), flags, _stream(stream)))


def conv_dgrad(W, dY, dX, geom, stream=None):
    check(load().crb_conv_dgrad(_p(W), _p(dY), _p(dX), ctypes.byref(geom), _stream(stream)))


def conv_wgrad_workspace_bytes(geom):
    return load().crb_conv_wgrad_workspace_bytes(ctypes.byref(geom))


def conv_wgrad(dY, X, dW, geom, workspace=None, stream=None):
    nbytes = 0 if workspace is None else workspace.numel() * workspace.element_size()
    check(load().crb_conv_wgrad(_p(dY), _p(X), _p(dW), ctypes.byref(geom), _p(workspace), nbytes, _stream(stream)))


def conv_wgrad_noalloc(dY, X, dW, geom, stream=None):
    """conv_wgrad on the library's built-in scratch buffer: the call allocates nothing."""
    check(load().crb_conv_wgrad_noalloc(_p(dY), _p(X), _p(dW), ctypes.byref(geom), _stream(stream)))


NOALLOC_SCRATCH_BYTES = 8 << 20  # CRB_NOALLOC_SCRATCH_BYTES


def bind_workspace(workspace, stream=None):
    """Bind `workspace` (a torch tensor, or None to unbind) as the split scratch of calls on `stream`."""
    nbytes = 0 if workspace is None else workspace.numel() * workspace.element_size()
    check(load().crb_bind_workspace(_p(workspace), nbytes, _stream(stream)))


def gemm_workspace_bytes(M, N, K, batch=1):
    return load().crb_gemm_workspace_bytes(M, N, K, batch)


def conv_fwd_workspace_bytes(geom, aligned16=True):
    return load().crb_conv_fwd_workspace_bytes(ctypes.byref(geom), int(aligned16))


def conv_dgrad_workspace_bytes(geom, aligned16=True):
    return load().crb_conv_dgrad_workspace_bytes(ctypes.byref(geom), int(aligned16))


def conv_bias_grad_workspace_bytes(N, C, HW):
    return load().crb_conv_bias_grad_workspace_bytes(N, C, HW)


def conv_bwd(W, dY, X, dX, dW, geom, workspace=None, stream=None):
    """Data gradient and weight gradient of one layer in one call (one launch for the residual-network layer shapes)."""
    nbytes = 0 if workspace is None else workspace.numel() * workspace.element_size()
    check(load().crb_conv_bwd(_p(W), _p(dY), _p(X), _p(dX), _p(dW), ctypes.byref(geom), _p(workspace), nbytes, _stream(stream)))


def conv_bwd_slices(geom):
    return load().crb_conv_bwd_slices(ctypes.byref(geom))


def conv_bwd_sliced(W, dY, X, dX, geom, workspace, stream=None):
    """dX now; the weight gradient stays as conv_bwd_slices(geom) partial sums in `workspace` until sum_slices_multi."""
    nbytes = workspace.numel() * workspace.element_size()
    check(load().crb_conv_bwd_sliced(_p(W), _p(dY), _p(X), _p(dX), ctypes.byref(geom), _p(workspace), nbytes, _stream(stream)))


class SliceSumItem(ctypes.Structure):
    """Mirror of ``crb_slice_sum_item``."""

    _fields_ = [("slices", ctypes.c_void_p), ("dst", ctypes.c_void_p), ("count", _u32), ("n_slices", _u32)]


def slice_sum_table(entries):
    """entries: (workspace tensor, dW tensor, number of slices) -> host array for sum_slices_multi (keep the tensors alive)."""
    arr = (SliceSumItem * len(entries))()
    for i, (ws, dW, n) in enumerate(entries):
        arr[i] = SliceSumItem(ws.data_ptr(), dW.data_ptr(), dW.numel(), n)
    return arr


def sum_slices_multi(table, stream=None):
    check(load().crb_sum_slices_multi(ctypes.cast(table, ctypes.c_void_p), len(table), _stream(stream)))


def conv_bias(Y, bias, N, C, HW, stream=None):
    check(load().crb_conv_bias(_p(Y), _p(bias), N, C, HW, _stream(stream)))


def conv_bias_grad(dY, dB, N, C, HW, stream=None):
    check(load().crb_conv_bias_grad(_p(dY), _p(dB), N, C, HW, _stream(stream)))


def tensor_add_inplace(a, b, count, stream=None):
    check(load().crb_tensor_add_inplace(_p(a), _p(b), count, _stream(stream)))


def tensor_fill(a, value, count, stream=None):
    check(load().crb_tensor_fill(_p(a), value, count, _stream(stream)))


def tensor_sub_inplace(a, b, count, stream=None):
    check(load().crb_tensor_sub_inplace(_p(a), _p(b), count, _stream(stream)))


def tensor_scale_inplace(a, factor, count, stream=None):
    check(load().crb_tensor_scale_inplace(_p(a), factor, count, _stream(stream)))


def relu_fwd(X, Y, count, stream=None):
    check(load().crb_relu_fwd(_p(X), _p(Y), count, _stream(stream)))


def relu_bwd(X, dY, dX, count, stream=None):
    check(load().crb_relu_bwd(_p(X), _p(dY), _p(dX), count, _stream(stream)))


def maxpool_fwd(X, Y, record, planes, IH, IW, sH, sW, rH, rW, stream=None):
    check(load().crb_maxpool_fwd(_p(X), _p(Y), _p(record), planes, IH, IW, sH, sW, rH, rW, _stream(stream)))


def maxpool_bwd(dX, dY, record, planes, IH, IW, sH, sW, rH, rW, stream=None):
    check(load().crb_maxpool_bwd(_p(dX), _p(dY), _p(record), planes, IH, IW, sH, sW, rH, rW, _stream(stream)))


def softmax(A, out, rows, step, stream=None):
    check(load().crb_softmax(_p(A), _p(out), rows, step, _stream(stream)))


def cross_entropy_grad(Y, labels, dY, count, stream=None):
    check(load().crb_cross_entropy_grad(_p(Y), _p(labels), _p(dY), count, _stream(stream)))


def cross_entropy_scratch_floats(count):
    return int(load().crb_cross_entropy_scratch_floats(count))


def cross_entropy_loss(Y, labels, scratch, loss_out, count, stream=None):
    """`loss_out`: one-element device tensor; `scratch`: device tensor of cross_entropy_scratch_floats(count) floats or None."""
    n = 0 if scratch is None else scratch.numel()
    check(load().crb_cross_entropy_loss(_p(Y), _p(labels), _p(scratch), n, _p(loss_out), count, _stream(stream)))


def momentum_apply(X, G, M, count, lr, beta, decay=1.0, stream=None):
    check(load().crb_momentum_apply(_p(X), _p(G), _p(M), count, lr, beta, decay, _stream(stream)))


def batchnorm_fwd(X, beta, gamma, mean, var, Y, xHat, N, F, stream=None):
    check(load().crb_batchnorm_fwd(_p(X), _p(beta), _p(gamma), _p(mean), _p(var), _p(Y), _p(xHat), N, F, _stream(stream)))


def batchnorm_bwd(dY, gamma, X, dX, N, F, dGamma=None, dBeta=None, stream=None):
    check(load().crb_batchnorm_bwd(_p(dY), _p(gamma), _p(X), _p(dX), _p(dGamma), _p(dBeta), N, F, _stream(stream)))


def batchnorm_param_grads(dY, xHat, dGamma, dBeta, N, F, stream=None):
    check(load().crb_batchnorm_param_grads(_p(dY), _p(xHat), _p(dGamma), _p(dBeta), N, F, _stream(stream)))


def tensor_copy(dst, src, count, stream=None):
    check(load().crb_tensor_copy(_p(dst), _p(src), count, _stream(stream)))


def tensor_add_clear(a, b, count, stream=None):
    check(load().crb_tensor_add_clear(_p(a), _p(b), count, _stream(stream)))


class MomentumItem(ctypes.Structure):
    """Mirror of ``crb_momentum_item``."""

    _fields_ = [("X", ctypes.c_void_p), ("G", ctypes.c_void_p), ("M", ctypes.c_void_p), ("count", _u32),
                ("lr", ctypes.c_float), ("beta", ctypes.c_float), ("decay", ctypes.c_float)]


def momentum_table(torch, dev, entries):
    """entries: (X, G, M, lr, beta, decay) tuples of device tensors / floats -> (device byte tensor holding the table, n,
    largest count). The tensors must stay alive as long as the table is used."""
    arr = (MomentumItem * len(entries))()
    for i, (X, G, M, lr, beta, decay) in enumerate(entries):
        arr[i] = MomentumItem(X.data_ptr(), G.data_ptr(), M.data_ptr(), X.numel(), lr, beta, decay)
    raw = torch.frombuffer(bytearray(bytes(arr)), dtype=torch.uint8).to(dev)
    return raw, len(entries), max(e[0].numel() for e in entries)


def momentum_apply_multi(table, n_items, max_count, stream=None):
    check(load().crb_momentum_apply_multi(_p(table), n_items, max_count, _stream(stream)))


def tensor_add(dst, a, b, count, stream=None):
    check(load().crb_tensor_add(_p(dst), _p(a), _p(b), count, _stream(stream)))


def tensor_add_clear_copy(dst, a, b, count, stream=None):
    check(load().crb_tensor_add_clear_copy(_p(dst), _p(a), _p(b), count, _stream(stream)))


def tensor_copy2(dst1, dst2, src, count, stream=None):
    check(load().crb_tensor_copy2(_p(dst1), _p(dst2), _p(src), count, _stream(stream)))


NORM_NONE, NORM_UNIFORM, NORM_DISTRIBUTION = 0, 1, 2
AUG_MIRROR, AUG_SHIFT = 1, 2


class ImageAug(ctypes.Structure):
    """Mirror of ``crb_image_aug``."""

    _fields_ = [("dh", ctypes.c_int32), ("dw", ctypes.c_int32), ("flags", _u32)]


def image_aug_table(torch, dev, entries):
    """entries: (dh, dw, flags) per image -> device byte tensor holding the records."""
    arr = (ImageAug * len(entries))()
    for i, (dh, dw, flags) in enumerate(entries):
        arr[i] = ImageAug(dh, dw, flags)
    return torch.frombuffer(bytearray(bytes(arr)), dtype=torch.uint8).to(dev)


def images_from_bytes(src, dst, images, channels, H, W, norm=NORM_NONE, p0=0.0, p1=1.0, aug=None, stream=None):
    check(load().crb_images_from_bytes(_p(src), _p(dst), images, channels, H, W, norm, p0, p1, _p(aug), _stream(stream)))


def batchnorm_relu_fwd(X, beta, gamma, mean, var, reluOut, N, F, Y=None, xHat=None, addend=None, stream=None):
    check(load().crb_batchnorm_relu_fwd(_p(X), _p(beta), _p(gamma), _p(mean), _p(var), _p(Y), _p(xHat), _p(addend), _p(reluOut), N, F,
                                        _stream(stream)))


def batchnorm_relu_bwd(dY, reluOut, gamma, X, dX, N, F, dGamma=None, dBeta=None, dY2=None, dYmasked=None, stream=None):
    check(load().crb_batchnorm_relu_bwd(_p(dY), _p(dY2), _p(reluOut), _p(gamma), _p(X), _p(dX), _p(dGamma), _p(dBeta), _p(dYmasked), N, F,
                                        _stream(stream)))


def tensor_add_relu(dst, a, b, count, stream=None):
    check(load().crb_tensor_add_relu(_p(dst), _p(a), _p(b), count, _stream(stream)))


def tensor_relu_grad_copy2(dst1, dst2, relu_out, dY, count, dY2=None, stream=None):
    check(load().crb_tensor_relu_grad_copy2(_p(dst1), _p(dst2), _p(relu_out), _p(dY), _p(dY2), count, _stream(stream)))
