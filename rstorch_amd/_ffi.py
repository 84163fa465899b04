"""ctypes binding of ``librstorch_hip.so`` (declared in ``include/rstorch_hip.h``).

There is no CPU fallback: if the library is missing or no GPU can be opened, the calls raise.
"""
import ctypes
import os

from . import _build

c_double_p = ctypes.POINTER(ctypes.c_double)
c_size_p = ctypes.POINTER(ctypes.c_size_t)
c_void_pp = ctypes.POINTER(ctypes.c_void_p)

RST_OK = 0
RST_ERR_INVALID_ARGUMENT = 1
RST_ERR_SHAPE = 2
RST_ERR_STATE = 3
RST_ERR_HIP = 4
RST_ERR_NAN = 5
RST_ERR_OUT_OF_MEMORY = 6
RST_ERR_UNSUPPORTED = 7

LAYER_IDENTITY, LAYER_LINEAR, LAYER_RELU = 0, 1, 2

KERNEL_NAMES = {
    0: "linear_forward", 1: "grad_weight", 2: "grad_bias", 3: "grad_input", 4: "relu_forward",
    5: "relu_backward", 6: "cross_entropy", 7: "loss_reduce", 8: "sgd", 9: "grad_pair",
}


class RstorchError(RuntimeError):
    """A failed call into the backend; the reference would have panicked."""

    def __init__(self, status, message):
        super().__init__("rstorch backend error %d: %s" % (status, message))
        self.status = status
        self.message = message


class ShapeError(RstorchError):
    pass


class StateError(RstorchError):
    pass


class NanError(RstorchError):
    pass


class KernelRecord(ctypes.Structure):
    _fields_ = [("kind", ctypes.c_int), ("layer", ctypes.c_int), ("ms", ctypes.c_double),
                ("flops", ctypes.c_double), ("bytes", ctypes.c_double)]


# name -> (argtypes); every function returns int status unless listed in _SPECIAL
_vp, _sz, _dbl, _i32, _u64 = (ctypes.c_void_p, ctypes.c_size_t, ctypes.c_double, ctypes.c_int,
                              ctypes.c_uint64)
_dp = ctypes.c_void_p  # device pointers travel as integers

SIGNATURES = {
    "rst_engine_create": [_i32, c_void_pp],
    "rst_engine_destroy": [_vp],
    "rst_engine_synchronize": [_vp],
    "rst_engine_trim": [_vp],
    "rst_engine_device_info": [_vp, ctypes.c_char_p, _sz, ctypes.POINTER(_i32), c_size_p],
    "rst_malloc": [_vp, _sz, c_void_pp],
    "rst_free": [_vp, _dp],
    "rst_upload": [_vp, _dp, c_double_p, _sz],
    "rst_download": [_vp, c_double_p, _dp, _sz],
    "rst_copy": [_vp, _dp, _dp, _sz],
    "rst_fill": [_vp, _dp, _sz, _dbl],
    "rst_event_create": [_vp, c_void_pp],
    "rst_event_destroy": [_vp],
    "rst_event_record": [_vp],
    "rst_event_wait": [_vp, _vp],
    "rst_event_elapsed_ms": [_vp, _vp, c_double_p],
    "rst_linear_forward": [_vp, _dp, _dp, _dp, _dp, _sz, _sz, _sz, _i32],
    "rst_linear_backward": [_vp, _dp, _dp, _dp, _dp, _dp, _dp, _dp, _sz, _sz, _sz],
    "rst_relu_forward": [_vp, _dp, _dp, _sz],
    "rst_relu_backward": [_vp, _dp, _dp, _dp, _sz],
    "rst_softmax_rows": [_vp, _dp, _dp, _sz, _sz],
    "rst_softmax_forward": [_vp, _dp, _dp, _sz, _sz, _i32],
    "rst_softmax_backward": [_vp, _dp, _dp, _dp, _sz, _sz],
    "rst_cross_entropy": [_vp, _dp, _dp, _dp, _dp, _sz, _sz, c_double_p],
    "rst_cross_entropy_accuracy": [_vp, _dp, _dp, _dp, _sz, _sz, c_double_p, c_double_p],
    "rst_cross_entropy_static": [_vp, _dp, _dp, _dp, _sz, _sz, c_double_p],
    "rst_loss_value": [_vp, c_double_p],
    "rst_sgd_step": [_vp, c_void_pp, c_void_pp, c_size_p, _sz, _dbl],
    "rst_sgd_step_flat": [_vp, _dp, _dp, _sz, _dbl],
    "rst_accuracy": [_vp, _dp, _dp, _sz, _sz, c_double_p],
    "rst_fill_uniform": [_vp, _dp, _sz, _u64, _u64, _dbl, _dbl],
    "rst_fill_normal": [_vp, _dp, _sz, _u64, _u64, _dbl, _dbl],
    "rst_fill_one_hot": [_vp, _dp, _sz, _sz, _u64, _u64],
    "rst_model_create": [_vp, ctypes.POINTER(_i32), c_size_p, c_size_p, _sz, c_void_pp],
    "rst_model_destroy": [_vp],
    "rst_model_parameter_count": [_vp, c_size_p, c_size_p],
    "rst_model_parameter": [_vp, _sz, c_void_pp, c_void_pp, c_size_p, c_size_p],
    "rst_model_init_kaiming": [_vp, _u64, _u64],
    "rst_model_export_parameters": [_vp, c_double_p, _sz],
    "rst_model_import_parameters": [_vp, c_double_p, _sz],
    "rst_stager_create": [_vp, _sz, _sz, _sz, _i32, c_void_pp],
    "rst_stager_destroy": [_vp],
    "rst_stager_submit_labels": [_vp, c_double_p, ctypes.POINTER(ctypes.c_uint32), _sz],
    "rst_stager_submit_dense": [_vp, c_double_p, c_double_p, _sz],
    "rst_stager_next": [_vp, c_void_pp, c_void_pp, c_size_p],
    "rst_stager_acquire_host": [_vp, ctypes.POINTER(c_double_p), ctypes.POINTER(ctypes.POINTER(ctypes.c_uint32))],
    "rst_stager_commit_labels": [_vp, _sz],
    "rst_model_forward": [_vp, _dp, _sz, c_void_pp],
    "rst_model_loss": [_vp, _dp, c_double_p],
    "rst_model_backward": [_vp, _dp, _i32, c_void_pp],
    "rst_model_forward_to": [_vp, _dp, _sz, _dp],
    "rst_model_backward_to": [_vp, _dp, _dp, _i32, _dbl],
    "rst_model_loss_accuracy_to": [_vp, _dp, _dp, _dp, _i32, _dp, _dp],
    "rst_model_discard_inputs": [_vp],
    "rst_model_sgd_step": [_vp, _dbl],
    "rst_model_train_step": [_vp, _dp, _dp, _sz, _dbl, c_double_p],
    "rst_model_profile_enable": [_vp, _i32],
    "rst_model_graph_enable": [_vp, _i32],
    "rst_model_graph_active": [_vp, ctypes.POINTER(ctypes.c_int)],
    "rst_model_fuse_sgd": [_vp, _i32],
    "rst_model_fuse_head": [_vp, _i32],
    "rst_model_pair_gradients": [_vp, _i32],
    "rst_model_profile_read": [_vp, ctypes.POINTER(KernelRecord), _sz, c_size_p],
}
_SPECIAL = {
    "rst_last_error": (ctypes.c_char_p, []),
    "rst_last_hip_error": (_i32, []),
    "rst_status_string": (ctypes.c_char_p, [_i32]),
    "rst_engine_stream": (_vp, [_vp]),
}

EXPORTED_SYMBOLS = sorted(list(SIGNATURES) + list(_SPECIAL))

_lib = None


def library_path():
    return _build.LIB_PATH


def load():
    """Loads the shared library (building it first only if it has never been built)."""
    global _lib
    if _lib is not None:
        return _lib
    path = library_path()
    if not os.path.exists(path):
        _build.build_library()
    lib = ctypes.CDLL(path)
    for name, args in SIGNATURES.items():
        fn = getattr(lib, name)
        fn.restype = ctypes.c_int
        fn.argtypes = args
    for name, (res, args) in _SPECIAL.items():
        fn = getattr(lib, name)
        fn.restype = res
        fn.argtypes = args
    _lib = lib
    return lib


def check(status):
    if status == RST_OK:
        return
    msg = load().rst_last_error().decode("utf-8", "replace")
    cls = {RST_ERR_SHAPE: ShapeError, RST_ERR_STATE: StateError, RST_ERR_NAN: NanError}.get(
        status, RstorchError)
    raise cls(status, msg)
