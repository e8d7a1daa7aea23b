"""ctypes binding of ``libpet_hip.so`` (the C ABI declared in ``include/pet_hip.h``).

Plumbing only: torch supplies device memory and the current stream, every
compute call goes through the shared library. There is no CPU fallback: if the
library is missing or a call fails, a ``PetHipError`` is raised.
"""
import ctypes
import os

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "lib", "libpet_hip.so")

ACT = {"none": 0, "relu": 1, "sigmoid": 2, "tanh": 3, "gelu": 4, None: 0}
ELT = {"add": 0, "sub": 1, "mul": 2, "div": 3}
# pet_hip_call_flags
Y_INITIALISED, DEFER_RELU, X_RELU, RES_RELU, A_SHARED, BIAS_PER_BATCH = 1, 2, 4, 8, 16, 32


class Fill(ctypes.Structure):
    """pet_hip_fill"""
    _fields_ = [("y", ctypes.c_void_p), ("bias", ctypes.c_void_p), ("outer", ctypes.c_size_t),
                ("ch", ctypes.c_size_t), ("inner", ctypes.c_size_t)]

class ConvView(ctypes.Structure):
    """pet_hip_conv_view: strides, in floats, of a 2-D convolution operand; the batch index is
    taken apart innermost first into n_extent[0], n_extent[1] and the rest."""
    _fields_ = [("c_stride", ctypes.c_longlong), ("h_stride", ctypes.c_longlong),
                ("w_stride", ctypes.c_longlong), ("n_extent", ctypes.c_int * 2),
                ("n_stride", ctypes.c_longlong * 3)]


_c_int_p = ctypes.POINTER(ctypes.c_int)
_vp = ctypes.c_void_p
_i = ctypes.c_int
_sz = ctypes.c_size_t

# name -> argtypes, exactly the declarations of include/pet_hip.h
SIGNATURES = {
    "pet_hip_init": [_i],
    "pet_hip_shutdown": [],
    "pet_hip_device_info": [ctypes.c_char_p, _sz, _c_int_p],
    "pet_hip_set_deterministic": [ctypes.c_int],
    "pet_hip_get_deterministic": [_c_int_p],
    "pet_hip_malloc": [ctypes.POINTER(_vp), _sz],
    "pet_hip_free": [_vp],
    "pet_hip_memcpy_h2d": [_vp, _vp, _sz, _vp],
    "pet_hip_memcpy_d2h": [_vp, _vp, _sz, _vp],
    "pet_hip_memcpy_d2d": [_vp, _vp, _sz, _vp],
    "pet_hip_fill_f32": [_vp, ctypes.c_float, _sz, _vp],
    "pet_hip_rand_uniform_f32": [_vp, _sz, ctypes.c_uint64, ctypes.c_float, ctypes.c_float, _vp],
    "pet_hip_stream_create": [ctypes.POINTER(_vp)],
    "pet_hip_stream_destroy": [_vp],
    "pet_hip_stream_sync": [_vp],
    "pet_hip_event_create": [ctypes.POINTER(_vp)],
    "pet_hip_event_destroy": [_vp],
    "pet_hip_event_record": [_vp, _vp],
    "pet_hip_event_sync": [_vp],
    "pet_hip_event_elapsed_ms": [ctypes.POINTER(ctypes.c_float), _vp, _vp],
    "pet_hip_graph_begin_capture": [_vp],
    "pet_hip_graph_end_capture": [_vp, ctypes.POINTER(_vp)],
    "pet_hip_graph_launch": [_vp, _vp],
    "pet_hip_graph_destroy": [_vp],
    "pet_hip_conv_out_dim": [_i] * 5,
    "pet_hip_conv2d_f32": [_vp] * 4 + [_i] * 15 + [_vp],
    "pet_hip_conv2d_static_f32": [_vp] * 4 + [_i] * 15 + [_vp],
    "pet_hip_conv3d_f32": [_vp] * 4 + [_i] * 20 + [_vp],
    "pet_hip_conv2d_res_f32": [_vp] * 5 + [_i] * 15 + [_vp],
    "pet_hip_conv3d_res_f32": [_vp, _vp, _i, _vp, _vp, _vp] + [_i] * 20 + [_vp],
    "pet_hip_bmm_res_f32": [_i] * 6 + [_vp] * 5 + [_i, _vp],
    "pet_hip_conv2d_ex_f32": [_vp] * 5 + [_i] * 15 + [ctypes.c_uint, _vp],
    "pet_hip_conv3d_ex_f32": [_vp, _vp, _i, _vp, _vp, _vp] + [_i] * 20 + [ctypes.c_uint, _vp],
    "pet_hip_bmm_ex_f32": [_i] * 6 + [_vp] * 5 + [_i, ctypes.c_uint, _vp],
    "pet_hip_conv2d_view_f32": [_vp] * 7 + [_i] * 15 + [ctypes.c_uint, _vp],
    "pet_hip_conv2d_view_supported": [_i] * 14 + [_c_int_p],
    "pet_hip_conv2d_accumulates": [_i] * 14 + [_c_int_p],
    "pet_hip_conv3d_accumulates": [_i] * 20 + [_c_int_p],
    "pet_hip_bmm_accumulates": [_i] * 6 + [_c_int_p],
    "pet_hip_bias_fill_batch": [_vp, _i, _vp],
    "pet_hip_conv3d_pack_filters": [_vp, _vp] + [_i] * 5 + [_vp],
    "pet_hip_conv3d_packed_f32": [_vp] * 4 + [_i] * 20 + [_vp],
    "pet_hip_bmm_f32": [_i] * 6 + [_vp] * 4 + [_i, _vp],
    "pet_hip_conv_trans_out_dim": [_i] * 6,
    "pet_hip_conv_trans_f32": [_vp] * 4 + [_i] * 16 + [_vp],
    "pet_hip_g2bmm_f32": [_vp] * 3 + [_i] * 5 + [_vp],
    "pet_hip_gbmml_f32": [_vp] * 3 + [_i] * 5 + [_vp],
    "pet_hip_attention_f32": [_vp] * 4 + [_i] * 8 + [ctypes.c_longlong] * 4 + [ctypes.c_float, _vp, _vp],
    "pet_hip_expr_program_create": [_c_int_p, _i, ctypes.POINTER(_vp)],
    "pet_hip_expr_f32": [_c_int_p, _i, _vp, ctypes.POINTER(_vp), _i, _vp, _vp],
    "pet_hip_transpose": [_vp, _vp, _c_int_p, _c_int_p, _i, _vp],
    "pet_hip_trans_chain": [_vp, _vp, _c_int_p, _i, _c_int_p, _i, _c_int_p, _c_int_p, _c_int_p, _vp],
    "pet_hip_split": [_vp, ctypes.POINTER(_vp), _i, _c_int_p, _i, _i, _c_int_p, _vp],
    "pet_hip_concat": [ctypes.POINTER(_vp), _i, _vp, _c_int_p, _i, _i, _c_int_p, _vp],
    "pet_hip_pad": [_vp, _vp, _c_int_p, _c_int_p, _c_int_p, _i, _vp],
    "pet_hip_slice": [_vp, _vp, _c_int_p, _c_int_p, _c_int_p, _i, _vp],
    "pet_hip_extend": [_vp, _vp, _c_int_p, _i, _i, _i, _vp],
    "pet_hip_eltwise": [_i, ctypes.POINTER(_vp), ctypes.POINTER(_sz), _i, _vp, _sz, _vp],
    "pet_hip_activation": [_vp, _vp, _sz, _i, _vp],
    "pet_hip_pow": [_vp, _vp, _sz, _i, _vp],
    "pet_hip_gather": [_vp, _vp, _i, _vp, _sz, _sz, _sz, _sz, _vp],
    "pet_hip_reduce_mean": [_vp, _vp, _sz, _sz, _sz, _vp],
    "pet_hip_batchnorm": [_vp] * 6 + [_sz, _sz, _sz, ctypes.c_float, _vp],
    "pet_hip_bias_act": [_vp, _vp, _vp, _sz, _sz, _sz, _i, _vp],
    "pet_hip_pool2d": [_vp, _vp] + [_i] * 13 + [_vp],
    "pet_hip_pool2d_ex": [_vp, _vp] + [_i] * 13 + [ctypes.c_uint, _vp],
    "pet_hip_softmax": [_vp, _vp, _sz, _sz, _vp],
    "pet_hip_layernorm": [_vp, _vp, _vp, _vp, _sz, _sz, ctypes.c_float, _vp],
}


class PetHipError(RuntimeError):
    def __init__(self, status, message):
        super().__init__("pet_hip status %d: %s" % (status, message))
        self.status = status


_lib = None
_initialised = False


def load():
    """Load the shared library and set prototypes. Raises if it is not built."""
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            raise PetHipError(-1, "%s is missing: build it with "
                              "`make -C pet_amd/csrc` (or __graft_entry__.build())" % LIB_PATH)
        lib = ctypes.CDLL(LIB_PATH)
        for name, argtypes in SIGNATURES.items():
            fn = getattr(lib, name)
            fn.argtypes = argtypes
            fn.restype = ctypes.c_int
        lib.pet_hip_last_error.argtypes = []
        lib.pet_hip_last_error.restype = ctypes.c_char_p
        _lib = lib
    return _lib


def last_error():
    return load().pet_hip_last_error().decode("utf-8", "replace")


def call(name, *args):
    """Invoke an entry point, raising PetHipError on a non-zero status."""
    rc = getattr(load(), name)(*args)
    if rc != 0:
        raise PetHipError(rc, last_error())
    return rc


def status(name, *args):
    """Invoke an entry point and return its raw status (for error-path tests)."""
    return getattr(load(), name)(*args)


def init(device=0):
    global _initialised
    if not _initialised:
        call("pet_hip_init", device)
        _initialised = True


def ints(values):
    values = [int(v) for v in values]
    return (ctypes.c_int * max(1, len(values)))(*values)
