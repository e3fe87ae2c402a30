"""ctypes binding of libsliced_hip.so (the C ABI declared in include/sliced_hip.h).

There is no fallback: if the library has not been built, or no gfx950 device is visible,
loading / init raises.  Nothing here computes on the CPU.
"""
import ctypes as C
import os

HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(HERE, "libsliced_hip.so")

c_f = C.POINTER(C.c_float)
c_sz = C.c_size_t
c_i32 = C.c_int32
c_vp = C.c_void_p

# name -> argument types (return type is int32 status unless listed in _RESTYPE)
PROTOTYPES = {
    "slhip_init": [c_i32, C.POINTER(c_vp)],
    "slhip_init_on_stream": [c_i32, c_vp, C.POINTER(c_vp)],
    "slhip_destroy": [c_vp],
    "slhip_last_error_string": [],
    "slhip_device_name": [c_vp, C.c_char_p, c_sz],
    "slhip_stream": [c_vp, C.POINTER(c_vp)],
    "slhip_workspace_bytes": [c_vp],
    "slhip_workspace": [c_vp, C.POINTER(c_vp)],
    "slhip_malloc": [c_vp, c_sz, C.POINTER(c_vp)],
    "slhip_free": [c_vp, c_vp],
    "slhip_memcpy_h2d": [c_vp, c_vp, c_vp, c_sz],
    "slhip_memcpy_d2h": [c_vp, c_vp, c_vp, c_sz],
    "slhip_memcpy_d2d": [c_vp, c_vp, c_vp, c_sz],
    "slhip_memset": [c_vp, c_vp, c_i32, c_sz],
    "slhip_fill": [c_vp, c_sz, C.c_float, c_vp],
    "slhip_sync": [c_vp],
    "slhip_event_create": [c_vp, C.POINTER(c_vp)],
    "slhip_event_record": [c_vp, c_vp],
    "slhip_event_elapsed_ms": [c_vp, c_vp, C.POINTER(C.c_float)],
    "slhip_event_destroy": [c_vp],
    "slhip_graph_begin": [c_vp],
    "slhip_graph_end": [c_vp, C.POINTER(c_vp)],
    "slhip_graph_launch": [c_vp, c_vp],
    "slhip_graph_node_count": [c_vp, C.POINTER(c_sz)],
    "slhip_graph_destroy": [c_vp],
    "slhip_rand_uniform": [c_vp, C.c_uint64, C.c_uint64, C.c_float, C.c_float, c_sz, c_vp],
    "slhip_sgemm": [c_vp, c_i32, c_i32, c_sz, c_sz, c_sz, c_vp, c_vp, c_vp, C.c_float],
    "slhip_gemm_tail_policy": [c_vp, c_i32],
    "slhip_gemm_tile_policy": [c_vp, c_i32],
    "slhip_gemm_plan_describe": [c_vp, C.c_char_p, c_sz],
    "slhip_sgemm_relu_mask": [c_vp, c_i32, c_i32, c_sz, c_sz, c_sz, c_vp, c_vp, c_vp, c_vp, C.c_float],
    "slhip_gemm": [c_vp, c_sz, c_sz, c_sz, c_vp, c_vp, c_vp],
    "slhip_gemm_grad": [c_vp, c_sz, c_sz, c_sz, c_vp, c_vp, c_vp, c_vp, c_vp, C.c_float],
    "slhip_linear_fwd": [c_vp, c_sz, c_sz, c_sz, c_vp, c_vp, c_vp, c_i32, c_vp, c_vp],
    "slhip_linear_grad": [c_vp, c_sz, c_sz, c_sz, c_vp, c_vp, c_vp, c_vp, c_vp, c_vp, c_vp, C.c_float],
    "slhip_linear_fwd_bits": [c_vp, c_sz, c_sz, c_sz, c_vp, c_vp, c_vp, c_vp, c_vp],
    "slhip_sgemm_relu_bits": [c_vp, c_i32, c_i32, c_sz, c_sz, c_sz, c_vp, c_vp, c_vp, c_vp, C.c_float],
    "slhip_relu_grad_bits": [c_vp, c_sz, c_sz, c_vp, c_vp, c_vp],
    "slhip_sum_rows": [c_vp, c_sz, c_sz, c_vp, c_vp],
    "slhip_sum_rows_static": [c_vp, c_sz, c_sz, c_vp, c_vp],
    "slhip_sum_cols": [c_vp, c_sz, c_sz, c_vp, c_vp],
    "slhip_max_rows": [c_vp, c_sz, c_sz, c_vp, c_vp],
    "slhip_max_cols": [c_vp, c_sz, c_sz, c_vp, c_vp],
    "slhip_mean_rows": [c_vp, c_sz, c_sz, c_vp, c_vp],
    "slhip_mean_cols": [c_vp, c_sz, c_sz, c_vp, c_vp],
    "slhip_sum": [c_vp, c_sz, c_vp, c_vp],
    "slhip_max": [c_vp, c_sz, c_vp, c_vp],
    "slhip_mean": [c_vp, c_sz, c_vp, c_vp],
    "slhip_sum_rows_grad": [c_vp, c_sz, c_sz, c_vp, c_vp],
    "slhip_sum_cols_grad": [c_vp, c_sz, c_sz, c_vp, c_vp],
    "slhip_max_rows_grad": [c_vp, c_sz, c_sz, c_vp, c_vp, c_vp, c_vp],
    "slhip_max_cols_grad": [c_vp, c_sz, c_sz, c_vp, c_vp, c_vp, c_vp],
    "slhip_mean_rows_grad": [c_vp, c_sz, c_sz, c_vp, c_vp],
    "slhip_mean_cols_grad": [c_vp, c_sz, c_sz, c_vp, c_vp],
    "slhip_softmax": [c_vp, c_sz, c_sz, c_vp, c_vp],
    "slhip_softmax_grad": [c_vp, c_sz, c_sz, c_vp, c_vp, c_vp, C.c_float],
    "slhip_transpose": [c_vp, c_sz, c_sz, c_vp, c_vp, C.c_float],
    "slhip_add_row": [c_vp, c_sz, c_sz, c_vp, c_vp, c_vp],
    "slhip_add_row_grad": [c_vp, c_sz, c_sz, c_vp, c_vp, c_vp],
    "slhip_add_row_mut_grad": [c_vp, c_sz, c_sz, c_vp, c_vp],
    "slhip_ew_binary": [c_vp, c_i32, c_sz, c_vp, c_vp, c_vp],
    "slhip_ew_binary_grad": [c_vp, c_i32, c_sz, c_vp, c_vp, c_vp, c_vp, c_vp],
    "slhip_ew_unary": [c_vp, c_i32, C.c_float, C.c_float, c_sz, c_vp, c_vp],
    "slhip_ew_unary_grad": [c_vp, c_i32, C.c_float, c_sz, c_vp, c_vp, c_vp],
    "slhip_ew_chain": [c_vp, c_sz, c_vp, c_vp, c_vp, c_vp, c_vp],
    "slhip_ew_program": [c_vp, c_sz, c_sz, c_vp, c_sz, c_vp, c_vp],
    "slhip_ew_program_grad": [c_vp, c_sz, c_sz, c_vp, c_vp, c_sz, c_vp, c_vp],
    "slhip_sgd_step": [c_vp, c_sz, c_vp, c_vp, C.c_float],
    "slhip_row_op": [c_vp, c_i32, c_sz, c_sz, c_vp, c_vp, c_vp],
    "slhip_row_op_grad": [c_vp, c_i32, c_sz, c_sz, c_vp, c_vp, c_vp, c_vp, c_vp],
    "slhip_col_op": [c_vp, c_i32, c_sz, c_sz, c_vp, c_vp, c_vp],
    "slhip_col_op_grad": [c_vp, c_i32, c_sz, c_sz, c_vp, c_vp, c_vp, c_vp, c_vp],
    "slhip_diagflat": [c_vp, c_sz, c_vp, c_vp],
    "slhip_diagflat_grad": [c_vp, c_sz, c_vp, c_vp],
    "slhip_onehot_grad": [c_vp, c_sz, c_sz, c_vp, c_vp, c_vp],
    "slhip_mse": [c_vp, c_sz, c_vp, c_vp, c_vp],
    "slhip_mse_grad": [c_vp, c_sz, c_vp, c_vp, c_vp, c_vp],
    "slhip_softmax_cce": [c_vp, c_sz, c_sz, c_vp, c_vp, c_vp, c_vp],
    "slhip_softmax_cce_grad": [c_vp, c_sz, c_sz, c_vp, c_vp, c_vp, C.c_float, c_vp],
    "slhip_mlp3_mse_step": [c_vp, c_sz, c_sz, c_sz, c_sz, c_vp, c_vp, c_vp, c_vp, c_vp, c_vp, c_vp, c_vp, c_vp, C.c_float, c_vp],
    "slhip_sgd_step_multi": [c_vp, c_sz, c_vp, c_vp, c_vp, C.c_float],
    "slhip_cce": [c_vp, c_sz, c_sz, c_vp, c_vp, c_vp],
    "slhip_cce_grad": [c_vp, c_sz, c_sz, c_vp, c_vp, c_vp],
    "slhip_onehot": [c_vp, c_sz, c_sz, c_vp, c_vp],
}
_RESTYPE = {"slhip_last_error_string": C.c_char_p, "slhip_workspace_bytes": c_sz}

_lib = None


class SlicedHipError(RuntimeError):
    pass


def load():
    """Load libsliced_hip.so and attach prototypes.  Raises if it is missing."""
    global _lib
    if _lib is not None:
        return _lib
    if not os.path.exists(LIB_PATH):
        raise SlicedHipError(
            "%s not found: build it first (python -m sliced_amd.build); there is no CPU fallback" % LIB_PATH)
    lib = C.CDLL(LIB_PATH)
    for name, argtypes in PROTOTYPES.items():
        fn = getattr(lib, name)          # AttributeError if the symbol is not exported
        fn.argtypes = argtypes
        fn.restype = _RESTYPE.get(name, c_i32)
    _lib = lib
    return lib


def check(rc, what=""):
    if rc != 0:
        msg = load().slhip_last_error_string()
        raise SlicedHipError("%s failed with status %d: %s" % (what, rc, msg.decode() if msg else "?"))
