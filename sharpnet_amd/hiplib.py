"""ctypes binding of libsharpnet_hip.so - the Python twin of the P/Invoke shim a
SharpNet maintainer would write in place of Prod/GPU/CublasWrapper.cs:221-250.

Nothing here computes: every function forwards raw device addresses to the C
ABI declared in include/sharpnet_hip.h.  There is no CPU fallback; if the
library is missing, ``load_library`` raises.
"""
import ctypes
import enum
import os

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB = None


class CublasStatus(enum.IntEnum):
    """Status numbering shared with cublasStatus_t (Prod/GPU/CublasWrapper.cs:8-20)."""
    CUBLAS_STATUS_SUCCESS = 0
    CUBLAS_STATUS_NOT_INITIALIZED = 1
    CUBLAS_STATUS_ALLOC_FAILED = 3
    CUBLAS_STATUS_INVALID_VALUE = 7
    CUBLAS_STATUS_ARCH_MISMATCH = 8
    CUBLAS_STATUS_MAPPING_ERROR = 11
    CUBLAS_STATUS_EXECUTION_FAILED = 13
    CUBLAS_STATUS_INTERNAL_ERROR = 14
    CUBLAS_STATUS_NOT_SUPPORTED = 15


class SharpNetHipError(Exception):
    """Raised for any non-zero status, like GPUWrapper.CheckStatus (Prod/GPU/GPUWrapper.cs:662-668)."""

    def __init__(self, status, where=""):
        try:
            name = CublasStatus(status).name
        except ValueError:
            name = "status %d" % status
        super().__init__(name + (" in " + where if where else ""))
        self.status = status


def check_status(status, where=""):
    if status != 0:
        raise SharpNetHipError(status, where)


def library_path():
    return os.environ.get("SHARPNET_HIP_LIB", os.path.join(_HERE, "libsharpnet_hip.so"))


_c_int_p = ctypes.POINTER(ctypes.c_int)
_c_float_p = ctypes.POINTER(ctypes.c_float)
_vp = ctypes.c_void_p
_vpp = ctypes.POINTER(ctypes.c_void_p)
_i = ctypes.c_int
_ll = ctypes.c_longlong
_f = ctypes.c_float
_sz = ctypes.c_size_t



class GemmDesc(ctypes.Structure):
    """snhip_gemm_desc of include/sharpnet_hip.h (field for field)."""
    _fields_ = [
        ("struct_size", _i), ("transA", _i), ("transB", _i), ("M", _i), ("N", _i), ("K", _i),
        ("alpha", _f), ("beta", _f), ("A", _vp), ("B", _vp), ("C", _vp), ("lda", _i), ("ldb", _i), ("ldc", _i),
        ("batch", _i), ("batch_inner", _i), ("strideA", _ll), ("strideB", _ll), ("strideC", _ll),
        ("strideA_outer", _ll), ("strideB_outer", _ll), ("strideC_outer", _ll), ("bias", _vp), ("D", _vp),
        ("ldd", _i), ("strideD", _ll), ("strideD_outer", _ll), ("gamma", _f), ("activation", _i),
        ("activation_param", _f), ("colsum", _vp), ("math", _i),
    ]

    def __init__(self, **kw):
        super().__init__()
        self.struct_size = ctypes.sizeof(GemmDesc)
        self.alpha, self.batch, self.math = 1.0, 1, -1
        for k, v in kw.items():
            if k not in dict(self._fields_):
                raise TypeError("snhip_gemm_desc has no field %r" % k)
            setattr(self, k, v)


class AttentionDesc(ctypes.Structure):
    """snhip_attention_desc of include/sharpnet_hip.h (field for field)."""
    _fields_ = [
        ("struct_size", _i), ("batch", _i), ("batch_inner", _i), ("Tq", _i), ("Tk", _i), ("dk", _i), ("dv", _i),
        ("scale", _f), ("causal", _i), ("Q", _vp), ("K", _vp), ("V", _vp), ("O", _vp), ("weights", _vp),
        ("ldq", _i), ("ldk", _i), ("ldv", _i), ("ldo", _i), ("strideQ", _ll), ("strideK", _ll), ("strideV", _ll),
        ("strideO", _ll), ("strideQ_outer", _ll), ("strideK_outer", _ll), ("strideV_outer", _ll), ("strideO_outer", _ll),
    ]

    def __init__(self, **kw):
        super().__init__()
        self.struct_size = ctypes.sizeof(AttentionDesc)
        self.scale = 1.0
        for k, v in kw.items():
            if k not in dict(self._fields_):
                raise TypeError("snhip_attention_desc has no field %r" % k)
            setattr(self, k, v)


class AttentionBwdDesc(ctypes.Structure):
    """snhip_attention_bwd_desc of include/sharpnet_hip.h (field for field)."""
    _fields_ = [
        ("struct_size", _i), ("batch", _i), ("batch_inner", _i), ("Tq", _i), ("Tk", _i), ("dk", _i), ("dv", _i),
        ("scale", _f), ("Q", _vp), ("K", _vp), ("V", _vp), ("dO", _vp), ("weights", _vp), ("scores_gradients", _vp),
        ("dQ", _vp), ("dK", _vp), ("dV", _vp), ("ldq", _i), ("ldk", _i), ("ldv", _i), ("ldo", _i),
        ("strideQ", _ll), ("strideK", _ll), ("strideV", _ll), ("strideO", _ll), ("strideQ_outer", _ll),
        ("strideK_outer", _ll), ("strideV_outer", _ll), ("strideO_outer", _ll), ("causal", _i),
    ]

    def __init__(self, **kw):
        super().__init__()
        self.struct_size = ctypes.sizeof(AttentionBwdDesc)
        self.scale = 1.0
        for k, v in kw.items():
            if k not in dict(self._fields_):
                raise TypeError("snhip_attention_bwd_desc has no field %r" % k)
            setattr(self, k, v)


class RnnDesc(ctypes.Structure):
    """snhip_rnn_desc of include/sharpnet_hip.h (field for field)."""
    _fields_ = [("struct_size", _i), ("cell_mode", _i), ("bias_mode", _i), ("bidirectional", _i), ("num_layers", _i),
                ("input_size", _i), ("hidden_size", _i), ("dropout", _f)]

    def __init__(self, **kw):
        super().__init__()
        self.struct_size = ctypes.sizeof(RnnDesc)
        self.num_layers = 1
        for k, v in kw.items():
            if k not in dict(self._fields_):
                raise TypeError("snhip_rnn_desc has no field %r" % k)
            setattr(self, k, float(v) if k == "dropout" else int(v))


# SNHIP_ACT_* and the reference's cudnnActivationMode_t names for them (Prod/GPU/CudnnWrapper.cs:267-281)
ACT_NONE, ACT_RELU, ACT_LEAKY_RELU, ACT_SIGMOID, ACT_TANH = range(5)
ACTIVATIONS = {
    None: ACT_NONE, "CUDNN_ACTIVATION_IDENTITY": ACT_NONE, "CUDNN_ACTIVATION_RELU": ACT_RELU,
    "CUDNN_ACTIVATION_LEAKY_RELU": ACT_LEAKY_RELU, "CUDNN_ACTIVATION_SIGMOID": ACT_SIGMOID,
    "CUDNN_ACTIVATION_TANH": ACT_TANH,
}


def activation_code(mode):
    """SNHIP_ACT_* for a cudnnActivationMode_t name (or an SNHIP_ACT_* integer, passed through)."""
    if isinstance(mode, int):
        return mode
    if mode not in ACTIVATIONS:
        raise SharpNetHipError(CublasStatus.CUBLAS_STATUS_NOT_SUPPORTED, "activation %r" % (mode,))
    return ACTIVATIONS[mode]


# name -> argtypes; every function returns int.  Must list every symbol of include/sharpnet_hip.h.
SIGNATURES = {
    "snhip_create": [_vpp],
    "snhip_destroy": [_vp],
    "snhip_set_stream": [_vp, _vp],
    "snhip_reserve_workspace": [_vp, _sz],
    "snhip_get_workspace_size": [_vp, ctypes.POINTER(_sz)],
    "snhip_get_version": [_vp, _c_int_p],
    "snhip_sgemm": [_vp, _i, _i, _i, _i, _i, _c_float_p, _vp, _i, _vp, _i, _c_float_p, _vp, _i],
    "snhip_sgemm_strided_batched": [_vp, _i, _i, _i, _i, _i, _c_float_p, _vp, _i, _ll, _vp, _i, _ll, _c_float_p, _vp,
                                    _i, _ll, _i],
    "snhip_dot": [_vp, _vp, _i, _i, _i, _vp, _i, _i, _i, _vp, _f, _f],
    "snhip_dot_noalloc": [_vp, _vp, _i, _i, _i, _vp, _i, _i, _i, _vp, _f, _f],
    "snhip_static_scratch_bytes": [],
    "snhip_get_last_error_message": [_vp, ctypes.c_char_p, _i],
    "snhip_dot_bias": [_vp, _vp, _i, _i, _i, _vp, _i, _i, _i, _vp, _f, _f, _vp],
    "snhip_bmm": [_vp, _vp, _i, _i, _i, _ll, _vp, _i, _i, _i, _ll, _vp, _ll, _i, _f, _f],
    "snhip_gemm_rm": [_vp, _i, _i, _i, _i, _i, _f, _vp, _i, _ll, _vp, _i, _ll, _f, _vp, _i, _ll, _i, _vp],
    "snhip_set_math_mode": [_vp, _i],
    "snhip_dot_bf16": [_vp, _vp, _i, _i, _i, _vp, _i, _i, _i, _vp, _f, _f, _vp],
    "snhip_bmm_bf16": [_vp, _vp, _i, _i, _i, _ll, _vp, _i, _i, _i, _ll, _vp, _ll, _i, _f, _f],
    "snhip_dot_bf16_stored": [_vp, _vp, _i, _i, _i, _vp, _i, _i, _i, _vp, _f, _f, _vp],
    "snhip_bmm_bf16_stored": [_vp, _vp, _i, _i, _i, _ll, _vp, _i, _i, _i, _ll, _vp, _ll, _i, _f, _f, _vp],
    "snhip_convert_f32_to_bf16": [_vp, _vp, _vp, _ll],
    "snhip_convert_f32_to_bf16_2d": [_vp, _vp, _i, _i, _ll, _i, _vp, _ll],
    "snhip_gemm_ex": [_vp, ctypes.POINTER(GemmDesc)],
    "snhip_sizeof_gemm_desc": [],
    "snhip_operand_element_bytes": [_i],
    "snhip_attention_forward": [_vp, ctypes.POINTER(AttentionDesc)],
    "snhip_sizeof_attention_desc": [],
    "snhip_attention_backward": [_vp, ctypes.POINTER(AttentionBwdDesc)],
    "snhip_sizeof_attention_bwd_desc": [],
    "snhip_sizeof_rnn_desc": [],
    "snhip_rnn_weight_space_size": [ctypes.POINTER(RnnDesc), ctypes.POINTER(_sz)],
    "snhip_rnn_weight_params": [ctypes.POINTER(RnnDesc), _i, _i, ctypes.POINTER(_ll), _c_int_p, _c_int_p,
                                ctypes.POINTER(_ll)],
    "snhip_rnn_temp_space_sizes": [ctypes.POINTER(RnnDesc), _i, _i, _i, ctypes.POINTER(_sz), ctypes.POINTER(_sz)],
    "snhip_rnn_forward": [_vp, ctypes.POINTER(RnnDesc), _i, _i, _i, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _sz, _vp, _sz],
    "snhip_rnn_set_step_mode": [_vp, _i],
    "snhip_rnn_set_dropout_seed": [_vp, ctypes.c_ulonglong],
    "snhip_rnn_get_dropout_calls": [_vp, ctypes.POINTER(ctypes.c_ulonglong)],
    "snhip_rnn_dropout_mask": [_vp, ctypes.POINTER(RnnDesc), _i, _i, ctypes.c_ulonglong, _i, _vp],
    "snhip_rnn_backward_data": [_vp, ctypes.POINTER(RnnDesc), _i, _i, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _vp,
                                _vp, _sz, _vp, _sz],
    "snhip_rnn_backward_weights": [_vp, ctypes.POINTER(RnnDesc), _i, _i, _vp, _vp, _vp, _vp, _vp, _sz, _vp, _sz],
    "snhip_dense_forward": [_vp, _vp, _vp, _vp, _vp, _i, _i, _i, _i, _f],
    "snhip_dense_backward": [_vp, _vp, _vp, _vp, _vp, _vp, _vp, _i, _i, _i, _f, _f],
    "snhip_dense_backward_ex": [_vp, _vp, _vp, _vp, _vp, _vp, _vp, _i, _i, _i, _f, _f, _vp, _f],
    "snhip_activation_forward": [_vp, _i, _f, _vp, _vp, _ll],
    "snhip_activation_backward": [_vp, _i, _f, _vp, _vp, _vp, _ll],
    "snhip_sgeam": [_vp, _i, _i, _i, _i, _c_float_p, _vp, _i, _c_float_p, _vp, _i, _vp, _i],
    "snhip_sdgmm": [_vp, _i, _i, _i, _vp, _i, _vp, _i, _vp, _i],
    "snhip_bias_gradient": [_vp, _vp, _i, _i, _vp],
    "snhip_transpose_second_and_third_dimension": [_vp, _vp, _vp, _i, _i, _i, _i],
    "snhip_broadcast_add_vector": [_vp, _vp, _vp, _i, _i],
    "snhip_axpy": [_vp, _ll, _f, _vp, _vp],
    "snhip_softmax_last_dim": [_vp, _vp, _vp, _ll, _i],
    "snhip_softmax_last_dim_backward": [_vp, _vp, _vp, _vp, _ll, _i],
    "snhip_set_above_main_diagonal": [_vp, _vp, _i, _i, _i, _f],
    "snhip_malloc": [_vpp, _sz],
    "snhip_free": [_vp],
    "snhip_memset32": [_vp, _vp, ctypes.c_uint, _sz],
    "snhip_memcpy_htod_async": [_vp, _vp, _vp, _sz],
    "snhip_memcpy_dtoh": [_vp, _vp, _vp, _sz],
    "snhip_memcpy_dtod_async": [_vp, _vp, _vp, _sz],
    "snhip_stream_synchronize": [_vp],
    "snhip_stream_create": [_vpp],
    "snhip_stream_destroy": [_vp],
    "snhip_event_create": [_vpp],
    "snhip_event_destroy": [_vp],
    "snhip_event_record": [_vp, _vp],
    "snhip_event_elapsed_ms": [_vp, _vp, _c_float_p],
    "snhip_copy_f32": [_vp, _vp, _vp, _ll],
    "snhip_device_info": [_vp, _c_int_p],
    "snhip_set_tuning": [_vp, _i, _i],
    "snhip_get_last_tuning": [_vp, _c_int_p, _c_int_p],
    "snhip_set_splitk_mode": [_vp, _i],
    "snhip_query_tuning": [_vp, _i, _i, _i, _i, _i, _c_int_p, _c_int_p],
    "snhip_config_count": [],
    "snhip_config_desc": [_i, _c_int_p],
}


def load_library(path=None):
    """dlopen libsharpnet_hip.so and attach the prototypes.  Raises if it is absent."""
    global _LIB
    if _LIB is not None and path is None:
        return _LIB
    path = path or library_path()
    if not os.path.exists(path):
        raise FileNotFoundError(
            "%s not found: build it with `python -m sharpnet_amd.build` (hipcc, gfx950). "
            "There is no CPU fallback for this path." % path)
    lib = ctypes.CDLL(path)
    for name, argtypes in SIGNATURES.items():
        fn = getattr(lib, name)  # AttributeError if the symbol is not exported
        fn.argtypes = argtypes
        fn.restype = ctypes.c_int
    _LIB = lib
    return lib
