"""ctypes binding of libdopthip.so (the C ABI declared in include/dopt_hip.h).

This module only loads the library and declares prototypes.  There is no CPU fallback: if the
library is missing or a call fails, an exception is raised.
"""
import ctypes as C
import os

HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(HERE, "libdopthip.so")

F32, I32 = 0, 1


class HipError(RuntimeError):
    """Raised with the library's last_error text, as the D wrappers would `enforce`."""

    def __init__(self, code, message):
        super().__init__("dopt_hip error %d: %s" % (code, message))
        self.code = code


class TinyNode(C.Structure):
    """dopt_hip_tiny_node of include/dopt_hip.h."""
    _fields_ = [(n, C.c_int) for n in ("kind", "op", "dst", "a", "b", "a_kind", "b_kind", "n", "dst_offset", "a_offset",
                                       "b_offset")] + [("dims", C.c_int * 4), ("reps", C.c_int * 4)]


class ConvDesc(C.Structure):
    _fields_ = [(n, C.c_size_t) for n in
                ("N", "C", "H", "W", "K", "R", "S", "padH", "padW", "strideH", "strideW")]


class SplitSum(C.Structure):
    """dopt_hip_split_sum: a convolution result left as partial copies for its reader to add."""
    _fields_ = [("partial", C.c_void_p), ("splits", C.c_int), ("elems", C.c_size_t), ("C", C.c_size_t),
                ("inner", C.c_size_t), ("bias", C.c_void_p), ("value", C.c_void_p), ("lanes", C.c_int)]


class TensorRef(C.Structure):
    _fields_ = [("w", C.c_void_p), ("g", C.c_void_p), ("m", C.c_void_p), ("v", C.c_void_p),
                ("vhat", C.c_void_p), ("n", C.c_size_t), ("skip_w", C.c_int)]


_sz, _vp, _i, _f, _d = C.c_size_t, C.c_void_p, C.c_int, C.c_float, C.c_double
_szp = C.POINTER(C.c_size_t)

# name -> argtypes (every function returns int unless listed in _SPECIAL)
PROTOTYPES = {
    "dopt_hip_init": [_i],
    "dopt_hip_shutdown": [],
    "dopt_hip_malloc": [C.POINTER(_vp), _sz],
    "dopt_hip_free": [_vp],
    "dopt_hip_pool_trim": [],
    "dopt_hip_pool_stats": [_szp, _szp, _szp],
    "dopt_hip_memset": [_vp, _i, _sz],
    "dopt_hip_copy_h2d": [_vp, _vp, _sz],
    "dopt_hip_copy_d2h": [_vp, _vp, _sz],
    "dopt_hip_copy_d2d": [_vp, _vp, _sz],
    "dopt_hip_host_alloc": [C.POINTER(_vp), _sz],
    "dopt_hip_host_free": [_vp],
    "dopt_hip_copy_h2d_async": [_vp, _vp, _sz],
    "dopt_hip_copy_d2d_batch": [C.c_int, C.POINTER(_vp), C.POINTER(_vp), C.POINTER(_sz)],
    "dopt_hip_sync": [],
    "dopt_hip_event_create": [C.POINTER(_vp)],
    "dopt_hip_event_record": [_vp],
    "dopt_hip_event_elapsed_ms": [_vp, _vp, C.POINTER(_f)],
    "dopt_hip_event_sync": [_vp],
    "dopt_hip_event_destroy": [_vp],
    "dopt_hip_pointwise": [C.c_char_p, _i, _sz, _vp, _vp, _vp],
    "dopt_hip_pointwise_chain": [_i, _sz, _sz, _i, C.POINTER(_vp), C.POINTER(C.c_ubyte), _i, C.POINTER(C.c_char_p),
                                 C.POINTER(_i), C.POINTER(_i), _vp],
    "dopt_hip_pointwise_chain_compile_only": [_i, _i, C.POINTER(C.c_ubyte), _i, C.POINTER(C.c_char_p), C.POINTER(_i),
                                              C.POINTER(_i), C.c_char_p],
    "dopt_hip_pointwise_index": [C.c_char_p],
    "dopt_hip_tiny_graph": [_i, C.POINTER(_vp), _i, C.POINTER(TinyNode)],
    "dopt_hip_pointwise_arity": [C.c_char_p],
    "dopt_hip_reduce": [C.c_char_p, _i, _szp, _i, _szp, _i, _vp, _vp],
    "dopt_hip_reduce_squares": [_szp, _i, _szp, _i, _vp, _vp],
    "dopt_hip_copy_h2d_beside": [_vp, _vp, _sz],
    "dopt_hip_upload_join": [],
    "dopt_hip_argmin": [_i, _szp, _i, _sz, _vp, _vp],
    "dopt_hip_rtc_compile_only": [C.c_char_p, _i, C.c_char_p],
    "dopt_hip_slice": [_i, _szp, _szp, _szp, _vp, _vp],
    "dopt_hip_pad": [_i, _szp, _szp, _szp, _vp, _vp],
    "dopt_hip_repeat": [_i, _szp, _szp, _vp, _vp],
    "dopt_hip_transpose2d": [_sz, _sz, _vp, _vp],
    "dopt_hip_sgemm": [_sz, _sz, _sz, _vp, _vp, _vp],
    "dopt_hip_sgemm_t": [C.c_int, C.c_int, _sz, _sz, _sz, _vp, _vp, _vp],
    "dopt_hip_sgemm_batch": [_i, C.POINTER(C.c_int), C.POINTER(C.c_int), _szp, _szp, _szp, C.POINTER(_vp), C.POINTER(_vp), C.POINTER(_vp)],
    "dopt_hip_sgemm_rank1": [_i, _i, _sz, _sz, _sz, _vp, _vp, _vp, _vp, _i, _vp],
    "dopt_hip_sgemm_relu_grad": [_i, _i, _sz, _sz, _sz, _vp, _vp, _vp, _vp],
    "dopt_hip_conv_fwd": [C.POINTER(ConvDesc), _vp, _vp, _vp],
    "dopt_hip_conv_fwd_bias": [C.POINTER(ConvDesc), _vp, _vp, _vp, _vp],
    "dopt_hip_conv_bwd_data": [C.POINTER(ConvDesc), _vp, _vp, _vp],
    "dopt_hip_conv_packed_layout": [C.POINTER(ConvDesc), _i],
    "dopt_hip_conv_pack_batch": [_i, C.POINTER(ConvDesc), C.POINTER(_i), C.POINTER(_vp), C.POINTER(_vp)],
    "dopt_hip_conv_fwd_bias_packed": [C.POINTER(ConvDesc), _vp, _vp, _vp, _vp],
    "dopt_hip_conv_bwd_data_packed": [C.POINTER(ConvDesc), _vp, _vp, _vp],
    "dopt_hip_conv_fwd_bias_packed_open": [C.POINTER(ConvDesc), _vp, _vp, _vp, _vp, C.POINTER(SplitSum)],
    "dopt_hip_conv_bwd_data_packed_open": [C.POINTER(ConvDesc), _vp, _vp, _vp, C.POINTER(SplitSum)],
    "dopt_hip_conv_pair_probe": [_i],
    "dopt_hip_conv_pair_probe_read": [C.POINTER(_i), C.POINTER(_d), C.POINTER(_d), C.POINTER(_d)],
    "dopt_hip_conv_bwd_pair_packed_open": [C.POINTER(ConvDesc), _vp, _vp, _vp, _vp, _vp, C.POINTER(SplitSum), C.POINTER(SplitSum)],
    "dopt_hip_split_sum_close": [C.POINTER(SplitSum)],
    "dopt_hip_conv_bwd_filter": [C.POINTER(ConvDesc), _vp, _vp, _vp],
    "dopt_hip_conv_bwd_filter_batch": [_i, C.POINTER(ConvDesc), C.POINTER(_vp), C.POINTER(_vp), C.POINTER(_vp)],
    "dopt_hip_maxpool_fwd": [_sz, _sz, _sz, _sz, _sz, _sz, _vp, _vp],
    "dopt_hip_maxpool_bwd": [_sz, _sz, _sz, _sz, _sz, _sz, _vp, _vp, _vp],
    "dopt_hip_softmax_fwd": [_sz, _sz, _sz, _vp, _vp],
    "dopt_hip_softmax_bwd": [_sz, _sz, _sz, _vp, _vp, _vp],
    "dopt_hip_relu_fwd": [_sz, _vp, _vp],
    "dopt_hip_relu_bwd": [_sz, _vp, _vp, _vp],
    "dopt_hip_bias_fwd": [_sz, _sz, _sz, _vp, _vp, _vp],
    "dopt_hip_bias_bwd": [_sz, _sz, _sz, _vp, _vp],
    "dopt_hip_bias_bwd_noalloc": [_sz, _sz, _sz, _vp, _vp],
    "dopt_hip_uniform": [C.c_uint64, C.c_uint64, _sz, _vp],
    "dopt_hip_philox_raw": [C.c_uint64, C.c_uint64, _sz, _vp],
    "dopt_hip_image_transform": [_sz, _sz, _sz, _sz, _sz, _sz, _vp, _vp, _vp],
    "dopt_hip_bn_train": [_sz, _sz, _sz, _d, _vp, _vp, _vp, _vp, _vp, _vp],
    "dopt_hip_bn_train_relu": [_sz, _sz, _sz, _d, _vp, _vp, _vp, _vp, _vp, _vp],
    "dopt_hip_bn_grad": [_sz, _sz, _sz, _vp, _vp, _vp, _vp],
    "dopt_hip_bn_grad_relu": [_sz, _sz, _sz, _vp, _vp, _vp, _vp, _vp],
    "dopt_hip_bn_grad_fused": [_sz, _sz, _sz, _vp, _vp, _vp, _vp, _vp, _vp],
    "dopt_hip_bn_train_pool": [_sz, _sz, _sz, _sz, _d, _vp, C.POINTER(SplitSum), _vp, _vp, _vp, _vp, _vp, _i, _vp],
    "dopt_hip_bn_grad_pool": [_sz, _sz, _sz, _sz, _vp, _vp, _vp, _vp, _vp, _vp],
    "dopt_hip_bn_train_open": [_sz, _sz, _sz, _d, C.POINTER(SplitSum), _vp, _vp, _vp, _vp, _vp, _i],
    "dopt_hip_bn_grad_open": [_sz, _sz, _sz, C.POINTER(SplitSum), _i, _vp, _vp, _vp, _vp, _vp],
    "dopt_hip_bn_grad_side": [_sz, _sz, _sz, _sz, _vp, C.POINTER(SplitSum), _i, _vp, C.POINTER(SplitSum), _vp, _vp, _vp, _vp, _vp,
                              C.POINTER(SplitSum)],
    "dopt_hip_bn_wait_limit": [C.c_uint],
    "dopt_hip_bn_infer": [_sz, _sz, _sz, _vp, _vp, _vp, _vp, _vp, _vp],
    "dopt_hip_optim_create": [_i, C.POINTER(TensorRef), C.POINTER(_vp)],
    "dopt_hip_optim_destroy": [_vp],
    "dopt_hip_sgd_step": [_vp, _f, _f, _i],
    "dopt_hip_adam_step": [_vp, _f, _f, _f, _f, C.POINTER(_f), C.POINTER(_f)],
    "dopt_hip_amsgrad_step": [_vp, _f, _f, _f, _f, C.POINTER(_f), C.POINTER(_f)],
}
_SPECIAL = {
    "dopt_hip_last_error": ([], C.c_char_p),
    "dopt_hip_stream": ([], _vp),
    "dopt_hip_conv_packed_bytes": ([C.POINTER(ConvDesc), _i], _sz),
    "dopt_hip_sgemm_order": ([C.c_int, C.c_int, _sz, _sz, _sz], C.c_uint64),
}

_lib = None


def load():
    """Loads the built library; raises if it has not been built (python -m dopt_amd.build)."""
    global _lib
    if _lib is not None:
        return _lib
    if not os.path.exists(LIB_PATH):
        raise ImportError("%s is missing: build it with `python -m dopt_amd.build` "
                          "(there is no CPU fallback)" % LIB_PATH)
    lib = C.CDLL(LIB_PATH)
    for name, argtypes in PROTOTYPES.items():
        fn = getattr(lib, name)
        fn.argtypes = argtypes
        fn.restype = C.c_int
    for name, (argtypes, restype) in _SPECIAL.items():
        fn = getattr(lib, name)
        fn.argtypes = argtypes
        fn.restype = restype
    _lib = lib
    return lib


def exported_symbols():
    return sorted(list(PROTOTYPES) + list(_SPECIAL))


def check(rc):
    if rc != 0:
        msg = load().dopt_hip_last_error()
        raise HipError(rc, msg.decode(errors="replace") if msg else "")


def sizes(seq):
    seq = [int(s) for s in seq]
    return (C.c_size_t * max(len(seq), 1))(*seq)
