"""ctypes binding of liblantern_hip.so (the C ABI declared in include/lantern_hip.h).

The library is loaded from lantern_amd/csrc/ (built in-tree).  There is no CPU fallback:
if the shared object is missing or a symbol does not resolve, loading raises.
"""
import ctypes as C
import os

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "csrc", "liblantern_hip.so")

P, I, F, L, Z, U64 = C.c_void_p, C.c_int, C.c_float, C.c_int64, C.c_size_t, C.c_uint64

# name -> (restype, argtypes); one line per declaration in include/lantern_hip.h
SIGNATURES = {
    "lh_setup": (None, [Z]),
    "lh_cleanup": (None, []),
    "lh_set_error_mode": (None, [I]),
    "lh_last_error": (C.c_char_p, []),
    "lh_clear_error": (None, []),
    "lh_sync": (None, []),
    "lh_malloc": (P, [Z]),
    "lh_malloc_uninit": (P, [Z]),
    "lh_free_top": (None, [Z]),
    "lh_mark": (Z, []),
    "lh_rewind": (None, [Z]),
    "lh_heap_used": (Z, []),
    "lh_heap_peak": (Z, []),
    "lh_h2d": (None, [P, P, Z]),
    "lh_d2h": (None, [P, P, Z]),
    "lh_host_alloc": (P, [Z]),
    "lh_host_free": (None, [P]),
    "lh_h2d_async": (None, [P, P, Z]),
    "lh_copy_join": (None, []),
    "lh_d2h_async": (None, [P, P, Z]),
    "lh_d2d": (None, [P, P, Z]),
    "lh_event_create": (P, []),
    "lh_event_record": (None, [P]),
    "lh_event_elapsed_ms": (F, [P, P]),
    "lh_event_destroy": (None, [P]),
    "lh_prof_enable": (None, [C.c_uint]),
    "lh_set_tuning": (None, [I]),
    "lh_tune_counters": (None, [P, P]),
    "lh_set_deterministic": (None, [I]),
    "lh_get_deterministic": (I, []),
    "lh_side_begin": (None, []),
    "lh_side_end": (None, []),
    "lh_side_join": (None, []),
    "lh_set_side_stream": (None, [I]),
    "lh_side_forks": (L, []),
    "lh_capture_begin": (None, []),
    "lh_capture_end": (I, []),
    "lh_graph_launch": (None, [I]),
    "lh_graph_destroy": (None, [I]),
    "lh_cmdlist_begin": (None, []),
    "lh_cmdlist_end": (None, []),
    "lh_cmdlist_inject_timeout": (None, []),
    "lh_cmdlist_stats": (None, [C.POINTER(C.c_int64), C.POINTER(C.c_int64)]),
    "lh_prof_collect": (None, [P, P, I]),
    "lh_set_fusion": (None, [I]),
    "lh_get_fusion": (I, []),
    "lh_flush_deferred": (None, []),
    "lh_fusion_stats": (None, [P, I]),
    "lh_work_collect": (None, [P, I]),
    "lh_fill": (None, [P, F, L]),
    "lh_fill_with_bias": (None, [P, P, L, L, L]),
    "lh_clip": (None, [P, F, L]),
    "lh_mask4d": (None, [P, P, I, I, I, I]),
    "lh_cifar_decode": (None, [P, P, P, I, I]),
    "lh_repeat0": (None, [P, P, I, I, L]),
    "lh_repeat0_grad": (None, [P, P, I, I, L]),
    "lh_unary": (None, [I, P, P, L, F, F]),
    "lh_unary_grad": (None, [I, P, P, P, P, L, I, F, F]),
    "lh_scalar_op": (None, [I, P, P, F, L]),
    "lh_bcast_op": (None, [I, P, P, P, P, P, P, I]),
    "lh_bcast_op_grad": (None, [I, P, P, P, I, P, P, P, I, P, P, I]),
    "lh_bcast_update": (None, [I, P, P, P, P, I]),
    "lh_geam": (None, [P, F, P, F, P, L]),
    "lh_trans": (None, [P, P, I, I]),
    "lh_trans_grad": (None, [P, P, I, I]),
    "lh_permute": (None, [P, P, P, P, I]),
    "lh_permute_grad": (None, [P, P, P, P, I]),
    "lh_sum_all": (None, [P, P, L]),
    "lh_mean_all": (None, [P, P, L]),
    "lh_add_scalar_from": (None, [P, P, F, L]),
    "lh_sum_dim": (None, [P, P, I, I, I]),
    "lh_sum_dim_grad": (None, [P, P, I, I, I]),
    "lh_softmax": (None, [I, P, P, I, I, I]),
    "lh_softmax_grad": (None, [I, P, P, P, I, I, I]),
    "lh_nll": (None, [P, P, P, I, I]),
    "lh_nll_grad": (None, [P, P, P, I, I]),
    "lh_sgemm": (None, [I, I, I, I, I, F, P, I, P, I, F, P, I]),
    "lh_sgemv": (None, [I, I, I, F, P, I, P, F, P]),
    "lh_ger": (None, [I, I, P, P, P]),
    "lh_dot_vv": (None, [P, P, P, I]),
    "lh_axpy_dev": (None, [P, P, P, L]),
    "lh_conv2d_fwd": (None, [P, P, P, P] + [I] * 11),
    "lh_conv2d_bwd_data": (None, [P, P, P, F] + [I] * 11),
    "lh_conv2d_bwd_filter": (None, [P, P, P, P, F] + [I] * 11),
    "lh_maxpool_fwd": (None, [P, P, P] + [I] * 9),
    "lh_maxpool_bwd": (None, [P, P, P, L]),
    "lh_avgpool_fwd": (None, [P, P] + [I] * 8),
    "lh_avgpool_bwd": (None, [P, P] + [I] * 8),
    "lh_avgpool_pad_fwd": (None, [P, P] + [I] * 10),
    "lh_avgpool_pad_bwd": (None, [P, P] + [I] * 10),
    "lh_bn_infer": (None, [P, P, P, P, P, P, I, I, I, F]),
    "lh_bn_train_fwd": (None, [P, P, P, P, P, P, P, P, I, I, I, F, F]),
    "lh_bn_bwd": (None, [P, P, P, P, P, P, F, P, P, I, I, I]),
    "lh_bn_train_fwd_relu": (None, [P, P, P, P, P, P, P, P, I, I, I, F, F]),
    "lh_bn_bwd_relu": (None, [P, P, P, P, P, P, P, P, F, P, P, I, I, I]),
    "lh_conv2d_fwd_bnstats": (None, [P, P, P, P] + [I] * 11 + [P, P, P, P, F, F]),
    "lh_conv2d_fwd_bn_apply": (None, [P, P, P, P] + [I] * 11 + [P, P, P, P, P, P, F, F, P, P, I]),
    "lh_bn_stats": (None, [P, P, P, P, P, I, I, I, F, F]),
    "lh_bn_apply": (None, [P, P, P, P, P, P, I, I, I, I]),
    "lh_bn_apply_add_relu": (None, [P, P, P, P, P, P, P, I, I, I]),
    "lh_bn_bwd_add_relu": (None, [P, P, P, P, P, P, P, F, P, F, P, P, I, I, I]),
    "lh_rnn_fwd": (None, [I, P, P, P, I, I, I, I, I]),
    "lh_rnn_bwd": (None, [I, P, P, P, P, P, F, P, I, I, I, I, I]),
    "lh_rnn_gated_reserve_floats": (L, [I, I, I, I, I]),
    "lh_rnn_gated_fwd": (None, [I, P, P, P, P, I, I, I, I, I]),
    "lh_rnn_gated_bwd": (None, [I, P, P, P, P, P, P, F, P, I, I, I, I, I]),
    "lh_rnn_fwd_init": (None, [I, P, P, P, P, I, I, I, I, I]),
    "lh_rnn_bwd_init": (None, [I, P, P, P, P, P, P, F, P, I, I, I, I, I]),
    "lh_rnn_gated_fwd_init": (None, [I, P, P, P, P, P, P, I, I, I, I, I]),
    "lh_rnn_gated_bwd_init": (None, [I, P, P, P, P, P, P, P, P, F, P, I, I, I, I, I]),
    "lh_ctc_loss": (None, [P, P, P, P, P, P, I, I, I]),
    "lh_maxpool_bwd_dense": (None, [P, P, P, F, I, I, I, I, I, I, I, I, I]),
    "lh_add_relu": (None, [P, P, P, L]),
    "lh_add_relu_grad": (None, [P, P, P, F, P, F, L]),
    "lh_dropout_fwd": (None, [P, P, P, L, F, U64, U64]),
    "lh_dropout_bwd": (None, [P, P, P, L]),
    "lh_concat": (None, [I, P, P, P, I, I]),
    "lh_concat_grad": (None, [I, P, P, P, I, I]),
    "lh_concat_grad_beta": (None, [I, P, P, P, P, I, I]),
    "lh_sgd": (None, [P, P, F, L]),
    "lh_momentum": (None, [P, P, P, F, F, F, I, L]),
    "lh_adagrad": (None, [P, P, P, F, F, L]),
    "lh_multi_momentum": (None, [I, P, P, P, P, F, F, F, I]),
    "lh_multi_sgd": (None, [I, P, P, P, F]),
    "lh_multi_momentum_static": (None, [I, P, P, P, P, F, F, F, I]),
}

_lib = None


class LanternHipError(RuntimeError):
    """Raised when an entry point of liblantern_hip reports an error (error mode 1)."""


def load():
    """Load the shared library once and bind every declared symbol; raises if it is absent."""
    global _lib
    if _lib is not None:
        return _lib
    if not os.path.exists(LIB_PATH):
        raise ImportError(
            "%s not found: build it with `python -c 'import __graft_entry__ as g; g.build()'` "
            "or `make -C lantern_amd/csrc` (there is no CPU fallback)" % LIB_PATH)
    lib = C.CDLL(LIB_PATH)
    for name, (res, args) in SIGNATURES.items():
        fn = getattr(lib, name)  # AttributeError if the symbol is missing
        fn.restype = res
        fn.argtypes = args
    # The error text lives in one static buffer: its first byte says whether an error is recorded, and reading that byte
    # costs a third of a foreign call (check() runs after every operator).
    global _err_flag
    lib.lh_last_error.restype = C.c_void_p
    _err_flag = C.c_ubyte.from_address(lib.lh_last_error())
    lib.lh_last_error.restype = C.c_char_p
    _lib = lib
    return lib


_err_flag = None


def check():
    """Raise LanternHipError if the last call recorded an error (used with error mode 1)."""
    if _err_flag.value:
        text = _lib.lh_last_error().decode()
        _lib.lh_clear_error()
        raise LanternHipError(text)
