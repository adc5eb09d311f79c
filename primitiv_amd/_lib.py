"""ctypes binding of libphip.so, the C ABI declared in include/phip.h.

There is no fallback: if the library is missing the import of any compute
entry fails with an Error that says how to build it.
"""
import ctypes
import os

HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(HERE, "libphip.so")

PHIP_OK = 0
PHIP_ERR_INVALID_ARGUMENT = -1
PHIP_ERR_RUNTIME = -2
PHIP_ERR_OUT_OF_MEMORY = -3
PHIP_ERR_UNSUPPORTED = -4


class Error(RuntimeError):
    """Counterpart of primitiv::Error (primitiv/core/error.h:14-32)."""

    def __init__(self, message, code=None):
        super().__init__(message)
        self.code = code


class DeviceInfo(ctypes.Structure):
    _fields_ = [
        ("name", ctypes.c_char * 256),
        ("arch", ctypes.c_char * 64),
        ("device_id", ctypes.c_int32),
        ("compute_units", ctypes.c_int32),
        ("clock_mhz", ctypes.c_int32),
        ("memory_clock_mhz", ctypes.c_int32),
        ("memory_bus_bits", ctypes.c_int32),
        ("wavefront_size", ctypes.c_int32),
        ("lds_bytes_per_workgroup", ctypes.c_int32),
        ("l2_bytes", ctypes.c_int32),
        ("global_memory_bytes", ctypes.c_uint64),
    ]


_vp = ctypes.c_void_p
_u32 = ctypes.c_uint32
_u64 = ctypes.c_uint64
_sz = ctypes.c_size_t
_f = ctypes.c_float
_int = ctypes.c_int
_pp = ctypes.POINTER(ctypes.c_void_p)
_ids = ctypes.POINTER(ctypes.c_uint32)   # host array of indices / extents

# name -> argument types; every function returns int unless listed in _RESTYPES
SIGNATURES = {
    "phip_last_error": [],
    "phip_device_count": [ctypes.POINTER(_int)],
    "phip_check_support": [_int],
    "phip_ctx_create": [_int, _pp],
    "phip_ctx_destroy": [_vp],
    "phip_ctx_id": [_vp],
    "phip_set_deterministic": [_vp, _int],
    "phip_set_overlap": [_vp, _int],
    "phip_device_info_get": [_vp, ctypes.POINTER(DeviceInfo)],
    "phip_describe": [_vp, ctypes.c_char_p, _sz],
    "phip_sync": [_vp],
    "phip_malloc": [_vp, _sz, _pp],
    "phip_free": [_vp, _vp],
    "phip_pool_alloc": [_vp, _sz, _pp, ctypes.POINTER(_sz)],
    "phip_pool_free": [_vp, _vp],
    "phip_pool_free_by_id": [_u64, _vp],
    "phip_pool_release_reserved": [_vp],
    "phip_pool_stats": [_vp, ctypes.POINTER(_u64), ctypes.POINTER(_u64)],
    "phip_memcpy_h2d": [_vp, _vp, _vp, _sz],
    "phip_memcpy_d2h": [_vp, _vp, _vp, _sz],
    "phip_memcpy_d2d": [_vp, _vp, _vp, _sz],
    "phip_fill_f32": [_vp, _vp, _f, _sz],
    "phip_fill_f16": [_vp, _vp, _f, _sz],
    "phip_fill_bf16": [_vp, _vp, _f, _sz],
    "phip_cvt_f32_to_f16": [_vp, _vp, _vp, _sz],
    "phip_cvt_f16_to_f32": [_vp, _vp, _vp, _sz],
    "phip_cvt_f32_to_bf16": [_vp, _vp, _vp, _sz],
    "phip_cvt_bf16_to_f32": [_vp, _vp, _vp, _sz],
    "phip_inplace_add_f32": [_vp, _vp, _vp, _u32, _u32, _u32],
    "phip_inplace_add_f16": [_vp, _vp, _vp, _u32, _u32, _u32],
    "phip_inplace_add_bf16": [_vp, _vp, _vp, _u32, _u32, _u32],
    "phip_batch_sum_f32": [_vp, _vp, _vp, _u32, _u32],
    "phip_batch_sum_f16": [_vp, _vp, _vp, _u32, _u32],
    "phip_batch_sum_bf16": [_vp, _vp, _vp, _u32, _u32],
    "phip_unary_fw_f32": [_vp, _int, _vp, _vp, _sz],
    "phip_unary_bw_f32": [_vp, _int, _vp, _vp, _vp, _vp, _sz],
    "phip_const_fw_f32": [_vp, _int, _vp, _f, _vp, _sz],
    "phip_const_bw_f32": [_vp, _int, _vp, _vp, _vp, _f, _vp, _sz],
    "phip_pown_fw_f32": [_vp, _vp, ctypes.c_int32, _vp, _sz],
    "phip_pown_bw_f32": [_vp, _vp, _vp, _vp, ctypes.c_int32, _vp, _sz],
    "phip_binary_fw_f32": [_vp, _int, _vp, _vp, _vp, _u32, _u32, _u32],
    "phip_binary_bw_f32": [_vp, _int, _vp, _vp, _vp, _vp, _vp, _vp, _u32, _u32, _u32],
    "phip_scalar_fw_f32": [_vp, _int, _int, _vp, _vp, _vp, _u32, _u32, _u32],
    "phip_inplace_subtract_f32": [_vp, _vp, _vp, _u32, _u32, _u32],
    "phip_inplace_multiply_const_f32": [_vp, _f, _vp, _sz],
    "phip_identity_f32": [_vp, _vp, _u32],
    "phip_unary_fw_f16": [_vp, _int, _vp, _vp, _sz],
    "phip_unary_bw_f16": [_vp, _int, _vp, _vp, _vp, _vp, _sz],
    "phip_const_fw_f16": [_vp, _int, _vp, _f, _vp, _sz],
    "phip_const_bw_f16": [_vp, _int, _vp, _vp, _vp, _f, _vp, _sz],
    "phip_pown_fw_f16": [_vp, _vp, ctypes.c_int32, _vp, _sz],
    "phip_pown_bw_f16": [_vp, _vp, _vp, _vp, ctypes.c_int32, _vp, _sz],
    "phip_binary_fw_f16": [_vp, _int, _vp, _vp, _vp, _u32, _u32, _u32],
    "phip_binary_bw_f16": [_vp, _int, _vp, _vp, _vp, _vp, _vp, _vp, _u32, _u32, _u32],
    "phip_scalar_fw_f16": [_vp, _int, _int, _vp, _vp, _vp, _u32, _u32, _u32],
    "phip_inplace_subtract_f16": [_vp, _vp, _vp, _u32, _u32, _u32],
    "phip_inplace_multiply_const_f16": [_vp, _f, _vp, _sz],
    "phip_identity_f16": [_vp, _vp, _u32],
    "phip_unary_fw_bf16": [_vp, _int, _vp, _vp, _sz],
    "phip_unary_bw_bf16": [_vp, _int, _vp, _vp, _vp, _vp, _sz],
    "phip_const_fw_bf16": [_vp, _int, _vp, _f, _vp, _sz],
    "phip_const_bw_bf16": [_vp, _int, _vp, _vp, _vp, _f, _vp, _sz],
    "phip_pown_fw_bf16": [_vp, _vp, ctypes.c_int32, _vp, _sz],
    "phip_pown_bw_bf16": [_vp, _vp, _vp, _vp, ctypes.c_int32, _vp, _sz],
    "phip_binary_fw_bf16": [_vp, _int, _vp, _vp, _vp, _u32, _u32, _u32],
    "phip_binary_bw_bf16": [_vp, _int, _vp, _vp, _vp, _vp, _vp, _vp, _u32, _u32, _u32],
    "phip_scalar_fw_bf16": [_vp, _int, _int, _vp, _vp, _vp, _u32, _u32, _u32],
    "phip_inplace_subtract_bf16": [_vp, _vp, _vp, _u32, _u32, _u32],
    "phip_inplace_multiply_const_bf16": [_vp, _f, _vp, _sz],
    "phip_identity_bf16": [_vp, _vp, _u32],
    "phip_copy_rows_f32": [_vp, _vp, _vp, _u32, _u32, _u64, _u64, _u32, _u64, _u64, _int],
    "phip_pick_fw_f32": [_vp, _vp, _ids, _u32, _vp, _u32, _u32, _u32, _u32, _u32],
    "phip_pick_bw_f32": [_vp, _vp, _ids, _u32, _vp, _u32, _u32, _u32, _u32, _u32],
    "phip_batch_pick_fw_f32": [_vp, _vp, _ids, _u32, _vp, _u32, _u32],
    "phip_batch_pick_bw_f32": [_vp, _vp, _ids, _u32, _vp, _u32, _u32],
    "phip_transpose_fw_f32": [_vp, _vp, _vp, _u32, _u32, _u32],
    "phip_transpose_bw_f32": [_vp, _vp, _vp, _u32, _u32, _u32],
    "phip_permute_dims_fw_f32": [_vp, _vp, _vp, _u32, _ids, _ids, _u32],
    "phip_permute_dims_bw_f32": [_vp, _vp, _vp, _u32, _ids, _ids, _u32],
    "phip_flip_fw_f32": [_vp, _vp, _vp, _u32, _u32, _u32],
    "phip_flip_bw_f32": [_vp, _vp, _vp, _u32, _u32, _u32],
    "phip_broadcast_fw_f32": [_vp, _vp, _vp, _u32, _u32, _u32],
    "phip_reduce_fw_f32": [_vp, _int, _vp, _vp, _u32, _u32, _u32],
    "phip_extremum_bw_f32": [_vp, _int, _vp, _vp, _vp, _vp, _u32, _u32, _u32],
    "phip_arg_extremum_f32": [_vp, _int, _vp, _ids, _u32, _u32, _u32],
    "phip_copy_rows_f16": [_vp, _vp, _vp, _u32, _u32, _u64, _u64, _u32, _u64, _u64, _int],
    "phip_pick_fw_f16": [_vp, _vp, _ids, _u32, _vp, _u32, _u32, _u32, _u32, _u32],
    "phip_pick_bw_f16": [_vp, _vp, _ids, _u32, _vp, _u32, _u32, _u32, _u32, _u32],
    "phip_batch_pick_fw_f16": [_vp, _vp, _ids, _u32, _vp, _u32, _u32],
    "phip_batch_pick_bw_f16": [_vp, _vp, _ids, _u32, _vp, _u32, _u32],
    "phip_transpose_fw_f16": [_vp, _vp, _vp, _u32, _u32, _u32],
    "phip_transpose_bw_f16": [_vp, _vp, _vp, _u32, _u32, _u32],
    "phip_permute_dims_fw_f16": [_vp, _vp, _vp, _u32, _ids, _ids, _u32],
    "phip_permute_dims_bw_f16": [_vp, _vp, _vp, _u32, _ids, _ids, _u32],
    "phip_flip_fw_f16": [_vp, _vp, _vp, _u32, _u32, _u32],
    "phip_flip_bw_f16": [_vp, _vp, _vp, _u32, _u32, _u32],
    "phip_broadcast_fw_f16": [_vp, _vp, _vp, _u32, _u32, _u32],
    "phip_reduce_fw_f16": [_vp, _int, _vp, _vp, _u32, _u32, _u32],
    "phip_extremum_bw_f16": [_vp, _int, _vp, _vp, _vp, _vp, _u32, _u32, _u32],
    "phip_arg_extremum_f16": [_vp, _int, _vp, _ids, _u32, _u32, _u32],
    "phip_copy_rows_bf16": [_vp, _vp, _vp, _u32, _u32, _u64, _u64, _u32, _u64, _u64, _int],
    "phip_pick_fw_bf16": [_vp, _vp, _ids, _u32, _vp, _u32, _u32, _u32, _u32, _u32],
    "phip_pick_bw_bf16": [_vp, _vp, _ids, _u32, _vp, _u32, _u32, _u32, _u32, _u32],
    "phip_batch_pick_fw_bf16": [_vp, _vp, _ids, _u32, _vp, _u32, _u32],
    "phip_batch_pick_bw_bf16": [_vp, _vp, _ids, _u32, _vp, _u32, _u32],
    "phip_transpose_fw_bf16": [_vp, _vp, _vp, _u32, _u32, _u32],
    "phip_transpose_bw_bf16": [_vp, _vp, _vp, _u32, _u32, _u32],
    "phip_permute_dims_fw_bf16": [_vp, _vp, _vp, _u32, _ids, _ids, _u32],
    "phip_permute_dims_bw_bf16": [_vp, _vp, _vp, _u32, _ids, _ids, _u32],
    "phip_flip_fw_bf16": [_vp, _vp, _vp, _u32, _u32, _u32],
    "phip_flip_bw_bf16": [_vp, _vp, _vp, _u32, _u32, _u32],
    "phip_broadcast_fw_bf16": [_vp, _vp, _vp, _u32, _u32, _u32],
    "phip_reduce_fw_bf16": [_vp, _int, _vp, _vp, _u32, _u32, _u32],
    "phip_extremum_bw_bf16": [_vp, _int, _vp, _vp, _vp, _vp, _u32, _u32, _u32],
    "phip_arg_extremum_bf16": [_vp, _int, _vp, _ids, _u32, _u32, _u32],
    "phip_random_uniform_f32": [_vp, _u64, _u64, _f, _f, _vp, _sz],
    "phip_random_bernoulli_f32": [_vp, _u64, _u64, _f, _vp, _sz],
    "phip_random_normal_f32": [_vp, _u64, _u64, _f, _f, _vp, _sz],
    "phip_random_log_normal_f32": [_vp, _u64, _u64, _f, _f, _vp, _sz],
    "phip_random_uniform_f16": [_vp, _u64, _u64, _f, _f, _vp, _sz],
    "phip_random_bernoulli_f16": [_vp, _u64, _u64, _f, _vp, _sz],
    "phip_random_normal_f16": [_vp, _u64, _u64, _f, _f, _vp, _sz],
    "phip_random_log_normal_f16": [_vp, _u64, _u64, _f, _f, _vp, _sz],
    "phip_random_uniform_bf16": [_vp, _u64, _u64, _f, _f, _vp, _sz],
    "phip_random_bernoulli_bf16": [_vp, _u64, _u64, _f, _vp, _sz],
    "phip_random_normal_bf16": [_vp, _u64, _u64, _f, _f, _vp, _sz],
    "phip_random_log_normal_bf16": [_vp, _u64, _u64, _f, _f, _vp, _sz],
    "phip_matmul_fw_f32": [_vp, _vp, _vp, _vp, _u32, _u32, _u32, _u32, _u32],
    "phip_matmul_fw_f32_noalloc": [_vp, _vp, _vp, _vp, _u32, _u32, _u32, _u32, _u32],
    "phip_gemm_trace": [_vp, ctypes.c_int, ctypes.c_char_p, _sz],
    "phip_set_deferred_zero_fill": [_vp, ctypes.c_int],
    "phip_matmul_fw_f16": [_vp, _vp, _vp, _vp, _u32, _u32, _u32, _u32, _u32],
    "phip_matmul_fw_bf16": [_vp, _vp, _vp, _vp, _u32, _u32, _u32, _u32, _u32],
    "phip_matmul_bw_f32": [_vp, _vp, _vp, _vp, _vp, _vp, _u32, _u32, _u32, _u32, _u32],
    "phip_matmul_bw_f16": [_vp, _vp, _vp, _vp, _vp, _vp, _u32, _u32, _u32, _u32, _u32],
    "phip_matmul_bw_bf16": [_vp, _vp, _vp, _vp, _vp, _vp, _u32, _u32, _u32, _u32, _u32],
    "phip_conv2d_fw_f32": [_vp, _vp, _vp, _vp] + [_u32] * 14,
    "phip_conv2d_bw_f32": [_vp, _vp, _vp, _vp, _vp, _vp] + [_u32] * 14,
    "phip_max_pool2d_fw_f32": [_vp, _vp, _vp] + [_u32] * 9,
    "phip_max_pool2d_bw_f32": [_vp, _vp, _vp, _vp, _vp] + [_u32] * 9,
    "phip_conv2d_fw_f16": [_vp, _vp, _vp, _vp] + [_u32] * 14,
    "phip_conv2d_bw_f16": [_vp, _vp, _vp, _vp, _vp, _vp] + [_u32] * 14,
    "phip_max_pool2d_fw_f16": [_vp, _vp, _vp] + [_u32] * 9,
    "phip_max_pool2d_bw_f16": [_vp, _vp, _vp, _vp, _vp] + [_u32] * 9,
    "phip_conv2d_fw_bf16": [_vp, _vp, _vp, _vp] + [_u32] * 14,
    "phip_conv2d_bw_bf16": [_vp, _vp, _vp, _vp, _vp, _vp] + [_u32] * 14,
    "phip_max_pool2d_fw_bf16": [_vp, _vp, _vp] + [_u32] * 9,
    "phip_max_pool2d_bw_bf16": [_vp, _vp, _vp, _vp, _vp] + [_u32] * 9,
    "phip_event_create": [_vp, _pp],
    "phip_event_destroy": [_vp],
    "phip_event_record": [_vp, _vp],
    "phip_event_elapsed_ms": [_vp, _vp, ctypes.POINTER(_f)],
    "phip_randomizer_create": [_u32, _pp],
    "phip_randomizer_destroy": [_vp],
    "phip_randomizer_fill_uniform": [_vp, _f, _f, _sz, _vp],
    "phip_randomizer_fill_normal": [_vp, _f, _f, _sz, _vp],
}
_RESTYPES = {"phip_last_error": ctypes.c_char_p, "phip_ctx_id": _u64}

_lib = None


def lib():
    """Loads libphip.so once; raises Error when it has not been built."""
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            raise Error(
                "libphip.so is not built (%s missing); run `python -m primitiv_amd.build`. "
                "There is no CPU fallback." % LIB_PATH)
        l = ctypes.CDLL(LIB_PATH)
        for name, argtypes in SIGNATURES.items():
            fn = getattr(l, name)
            fn.argtypes = argtypes
            fn.restype = _RESTYPES.get(name, _int)
        _lib = l
    return _lib


def check(rc):
    """Turns a non-zero status into Error carrying the library's message."""
    if rc != PHIP_OK:
        msg = lib().phip_last_error()
        raise Error(msg.decode("utf-8", "replace") if msg else "libphip error %d" % rc, rc)


def call(name, *args):
    check(getattr(lib(), name)(*args))
