"""ctypes binding of libgnnhip.so.  Loading fails loudly: there is no CPU fallback."""
import ctypes
import os
from ctypes import POINTER, c_char_p, c_float, c_int, c_size_t, c_void_p

_HERE = os.path.dirname(os.path.abspath(__file__))
# GNNHIP_LIBRARY overrides the in-tree location (e.g. an instrumented build of the same ABI)
_LIB_PATH = os.environ.get("GNNHIP_LIBRARY") or os.path.join(_HERE, "lib", "libgnnhip.so")
_lib = None


class GnnHipError(RuntimeError):
    def __init__(self, code, text):
        super().__init__("gnnhip error %d: %s" % (code, text))
        self.code = code


def library_path():
    return _LIB_PATH


_P = c_void_p
_I, _F, _Z = c_int, c_float, c_size_t

# name -> argtypes; every entry returns int unless listed in _RESTYPES
SIGNATURES = {
    "gnnhip_init": [_I],
    "gnnhip_shutdown": [],
    "gnnhip_malloc": [POINTER(c_void_p), _Z],
    "gnnhip_recycle": [_P],
    "gnnhip_free": [_P],
    "gnnhip_pool_stats": [POINTER(c_size_t), POINTER(c_size_t), POINTER(c_size_t)],
    "gnnhip_memcpy_h2d": [_P, _P, _Z, _P],
    "gnnhip_memcpy_h2d_sparse32": [_P, _P, _Z, _P],
    "gnnhip_memcpy_d2h": [_P, _P, _Z, _P],
    "gnnhip_memcpy_d2d": [_P, _P, _Z, _P],
    "gnnhip_memcpy_d2h_batch": [_I, _P, _P, _P, _P],
    "gnnhip_memcpy_h2d_batch": [_I, _P, _P, _P, _P],
    "gnnhip_memset0": [_P, _Z, _P],
    "gnnhip_memset0_batch": [_I, _P, _P, _P],
    "gnnhip_stream_sync": [_P],
    "gnnhip_spmm_csr_f32": [_I, _I, _I, _I, _F, _P, _P, _P, _P, _I, _F, _P, _I, _P],
    "gnnhip_csr_plan_create": [_I, _I, _P, _P, _P, _P, POINTER(_P)],
    "gnnhip_csr_plan_destroy": [_P],
    "gnnhip_csr_plan_bytes": [_P, POINTER(c_size_t)],
    "gnnhip_spmm_csr_planned_f32": [_P, _I, _F, _P, _I, _F, _P, _I, _P],
    "gnnhip_s2v_level_planned_f32": [_P, _I, _P, _P, _P, _P, _P, _P],
    "gnnhip_release_scratch": [_P],
    "gnnhip_csr_group_i32": [_I, _I, _P, _I, _P, _I, _I, _P, _P, _P, _P],
    "gnnhip_csr_group_both_i32": [_I, _I, _P, _I, _P, _I, _P, _P, _P, _P, _P, _P, _P],
    "gnnhip_csr_consecutive_rows_f32": [_I, _P, _I, _P, _P, _P],
    "gnnhip_csr_consecutive_rows_host_f32": [_I, _P, _I, _P, _P, _P, _P],
    "gnnhip_csr_transpose_f32": [_I, _I, _I, _P, _P, _P, _P, _P, _P, _P],
    "gnnhip_gemm_f32": [_I, _I, _I, _I, _I, _F, _P, _I, _P, _I, _F, _P, _I, _P],
    "gnnhip_gemm_tn_batch_f32": [_I, _P, _P, _P, _P, _P, _P, _P, _F, _F, _P, _P, _P],
    "gnnhip_s2v_level_f32": [_I, _I, _I, _P, _P, _P, _P, _P, _P, _P, _P, _P],
    "gnnhip_s2v_input_f32": [_I, _I, _I, _P, _P, _P, _P, _P],
    "gnnhip_s2v_readout_f32": [_I, _I, _I, _I, _I, _P, _P, _P, _P, _P, _P, _P, _P, _P, _P, _P, _P],
    "gnnhip_s2v_forward_f32": [_I] * 8 + [_P] * 11 + [_P] * 8 + [POINTER(c_int), _P],
    "gnnhip_s2v_forward_planned_f32": [_P] + [_I] * 6 + [_P] * 8 + [_P] * 8 + [POINTER(c_int), _P],
    "gnnhip_s2v_forward_batched_f32": [_I] * 8 + [_P] * 11 + [_P] * 7 + [_P, _P],
    "gnnhip_s2v_forward_batched_train_f32": [_I] * 8 + [_P] * 11 + [_P] * 7 + [_P, _P],
    "gnnhip_s2v_forward_batched_labels_f32": [_I] * 8 + [_P] * 11 + [_P] * 7 + [_P, _P],
    "gnnhip_s2v_input_labels_f32": [_I, _I, _I, _P, _P, _P, _P, _P, _P],
    "gnnhip_unary_f32": [_I, _P, _Z, _F, _F, _P],
    "gnnhip_relu_f32": [_P, _P, _Z, _P],
    "gnnhip_axpy_f32": [_Z, _F, _P, _P, _P],
    "gnnhip_axpby_f32": [_Z, _F, _P, _F, _P, _P],
    "gnnhip_add_f32": [_Z, _P, _P, _P, _P],
    "gnnhip_row_softmax_f32": [_P, _I, _I, _P],
    "gnnhip_jagged_softmax_f32": [_P, _P, _I, _P],
    "gnnhip_jagged_softmax_static_f32": [_P, _P, _I, _P],
    "gnnhip_jagged_softmax_deriv_f32": [_P, _P, _P, _P, _I, _P],
    "gnnhip_row_softmax_deriv_f32": [_P, _P, _P, _I, _I, _P],
    "gnnhip_reduce_f32": [_I, _P, _Z, _P, _P],
    "gnnhip_row_argmax_f32": [_P, _I, _I, _P, _P],
    "gnnhip_csr_row_argmax_f32": [_P, _P, _P, _I, _P, _P],
    "gnnhip_cross_entropy_f32": [_P, _I, _I, _P, _P, _P, _P, _P],
    "gnnhip_in_top_k_f32": [_P, _P, _I, _I, _I, _P, _P],
    "gnnhip_cast_i32_f32": [_P, _P, _Z, _P],
    "gnnhip_spmm_csr_t_f32": [_I, _I, _I, _F, _P, _P, _P, _P, _I, _F, _P, _I, _P],
    "gnnhip_csr_axpy_f32": [_I, _I, _F, _P, _P, _P, _P, _P],
    "gnnhip_relu_deriv_f32": [_Z, _P, _P, _P, _P],
    "gnnhip_mul_f32": [_Z, _P, _P, _P],
    "gnnhip_row_scale_f32": [_I, _I, _P, _P, _P],
    "gnnhip_s2v_loss_acc_f32": [_I, _I, _P, _P, _P, _P, _P, _P, _P, _P, _P, _P],
    "gnnhip_s2v_readout_backward_f32": [_I] * 5 + [_P] * 7 + [_F] + [_P] * 6 + [_P],
    "gnnhip_s2v_level_backward_f32": [_I, _I, _I, _P, _P, _P, _P, _P, _P, _P, _P, _P, _P],
    "gnnhip_s2v_grad_gate_f32": [_Z, _P, _P, _P, _P, _I, _P],
    "gnnhip_momentum_sgd_batch_f32": [_I, _P, _P, _P, _P, _F, _F, _F, _P],
    "gnnhip_adam_batch_f32": [_I, _P, _P, _P, _P, _P, _F, _F, _F, _F, _F, _F, _F, _F, _P],
    "gnnhip_last_error": [],
    "gnnhip_version": [],
}
_RESTYPES = {"gnnhip_last_error": c_char_p, "gnnhip_version": c_char_p}


def load_library():
    """Load libgnnhip.so and declare every entry point.  Raises if the library is missing."""
    global _lib
    if _lib is not None:
        return _lib
    if not os.path.exists(_LIB_PATH):
        raise RuntimeError(
            "libgnnhip.so is not built (%s). Run `python -m graphnn_amd.build`; "
            "there is no CPU fallback for the HIP kernels." % _LIB_PATH)
    lib = ctypes.CDLL(_LIB_PATH)
    for name, argtypes in SIGNATURES.items():
        fn = getattr(lib, name)          # AttributeError if the symbol is not exported
        fn.argtypes = argtypes
        fn.restype = _RESTYPES.get(name, c_int)
    _lib = lib
    return lib


def check(rc):
    if rc != 0:
        text = load_library().gnnhip_last_error()
        raise GnnHipError(rc, text.decode() if text else "")
    return rc
