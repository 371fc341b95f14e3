"""ctypes binding of libtorchgt_hip.so (the C ABI in include/torchgt_hip.h).

The library is loaded from the package directory.  There is no fallback: if the
shared object is missing or a call fails, an exception is raised.
"""
import ctypes
import os

HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(HERE, "libtorchgt_hip.so")

OK = 0
ERR_INVALID_ARG, ERR_INDEX_RANGE, ERR_UNSUPPORTED, ERR_HIP, ERR_WORKSPACE = -1, -2, -3, -4, -5
DTYPE_F32, DTYPE_BF16, DTYPE_F32_BF16_PRODUCTS = 0, 1, 2
BIAS_NONE, BIAS_EDGE_HEAD, BIAS_EDGE = 0, 1, 2
BIAS_PLAN_ORDER = 0x10
BIAS_BOTH_ORDERS = 0x20
(PLAN_ROWPTR_DST, PLAN_COL_DST, PLAN_EID_DST, PLAN_ROWPTR_SRC, PLAN_COL_SRC, PLAN_EID_SRC,
 PLAN_ITEMS_DST, PLAN_ITEMS_SRC, PLAN_POS_SRC) = range(9)

_c = ctypes
_vp, _i64, _i32 = _c.c_void_p, _c.c_int64, _c.c_int

# name -> (restype, argtypes); one entry per declaration in include/torchgt_hip.h
SIGNATURES = {
    "tgt_version": (_i32, []),
    "tgt_error_string": (_c.c_char_p, [_i32]),
    "tgt_last_error": (_c.c_char_p, []),
    "tgt_plan_create": (_i32, [_vp, _vp, _i64, _i64, _vp, _c.POINTER(_vp)]),
    "tgt_plan_create_remaining": (_i32, [_vp, _vp, _i64, _i64, _vp, _c.POINTER(_vp)]),
    "tgt_plan_destroy": (_i32, [_vp]),
    "tgt_set_allocator": (_i32, [_vp, _vp, _vp]),
    "tgt_edge_index_hash": (_i32, [_vp, _vp, _i64, _vp, _c.POINTER(_c.c_uint64)]),
    "tgt_plan_info": (_i32, [_vp, _c.POINTER(_i64)]),
    "tgt_plan_array_len": (_i64, [_vp, _i32]),
    "tgt_plan_export": (_i32, [_vp, _i32, _vp, _i64]),
    "tgt_plan_enable_bias_order": (_i32, [_vp, _vp]),
    "tgt_plan_edge_order": (_i32, [_vp, _vp, _vp]),
    "tgt_plan_edge_order_src": (_i32, [_vp, _vp, _vp]),
    "tgt_plan_sort_rows": (_i32, [_vp, _vp, _i32, _vp, _i32, _vp]),
    "tgt_sparse_attn_workspace_bytes": (_i64, [_vp, _i32, _i32]),
    "tgt_sparse_attn_fwd": (_i32, [_vp, _vp, _vp, _vp, _vp, _i32, _i32, _i32, _i32, _vp, _vp, _vp, _i64, _vp]),
    "tgt_sparse_attn_fwd_noalloc": (_i32, [_vp, _vp, _vp, _vp, _vp, _i32, _i32, _i32, _i32, _vp, _vp, _vp]),
    "tgt_plan_prepare": (_i32, [_vp, _i32, _i32, _vp]),
    "tgt_sparse_attn_bwd": (_i32, [_vp, _vp, _vp, _vp, _vp, _i32, _i32, _i32, _i32, _vp, _vp, _vp,
                                   _vp, _vp, _vp, _vp, _vp, _i64, _vp]),
    "tgt_dense_attn_dropout_fwd": (_i32, [_vp, _vp, _vp, _vp, _i32, _i32, _i32, _i32, _i32, _c.c_float, _c.c_uint64, _vp, _vp, _vp]),
    "tgt_dense_attn_dropout_bwd": (_i32, [_vp, _vp, _vp, _vp, _i32, _i32, _i32, _i32, _i32, _c.c_float, _c.c_uint64, _vp, _vp, _vp,
                                          _vp, _vp, _vp, _vp, _vp]),
    "tgt_dense_attn_dropout_mask": (_i32, [_i32, _i32, _i32, _c.c_float, _c.c_uint64, _vp, _vp]),
    "tgt_dense_ids_pack": (_i32, [_vp, _vp, _i32, _i32, _i32, _i32, _i32, _vp, _vp, _vp]),
    "tgt_dense_attn_ids_fwd": (_i32, [_vp, _vp, _vp, _vp, _vp, _vp, _i32, _vp, _i32, _vp, _i32, _vp, _i32, _i32, _i32, _i32, _i32,
                                      _c.c_float, _c.c_uint64, _vp, _vp, _vp]),
    "tgt_dense_attn_ids_bwd_workspace_bytes": (_i64, [_i32, _i32, _i32, _i32]),
    "tgt_dense_attn_ids_bwd": (_i32, [_vp, _vp, _vp, _vp, _vp, _vp, _i32, _vp, _i32, _vp, _i32, _vp, _i32, _i32, _i32, _i32, _i32,
                                      _c.c_float, _c.c_uint64, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _i64, _vp]),
    "tgt_dense_attn_fwd": (_i32, [_vp, _vp, _vp, _vp, _i32, _i32, _i32, _i32, _i32, _vp, _vp, _vp]),
    "tgt_dense_attn_bwd": (_i32, [_vp, _vp, _vp, _vp, _i32, _i32, _i32, _i32, _i32, _vp, _vp, _vp,
                                  _vp, _vp, _vp, _vp, _vp]),
    "tgt_tiles_create": (_i32, [_vp, _i64, _i32, _i64, _vp, _c.POINTER(_vp)]),
    "tgt_tiles_destroy": (_i32, [_vp]),
    "tgt_block_attn_workspace_bytes": (_i64, [_vp, _vp, _i32, _i32]),
    "tgt_block_attn_fwd": (_i32, [_vp, _vp, _vp, _vp, _vp, _vp, _i32, _i32, _i32, _i32, _vp, _vp, _vp, _i64, _vp]),
    "tgt_block_attn_bwd": (_i32, [_vp, _vp, _vp, _vp, _vp, _vp, _i32, _i32, _i32, _i32, _vp, _vp, _vp,
                                  _vp, _vp, _vp, _vp, _vp, _i64, _vp]),
    "tgt_reformat_num_tiles": (_i64, [_vp]),
    "tgt_reformat_num_raw_edges": (_i64, [_vp]),
    "tgt_reformat_export_tiles": (_i32, [_vp, _vp, _vp, _vp]),
    "tgt_fix_edge_index": (_i32, [_vp, _i64, _i64, _vp, _vp]),
    "tgt_sub_edge_index": (_i32, [_vp, _i64, _i64, _vp, _i64, _vp, _i64, _c.POINTER(_i64), _vp]),
    "tgt_reformat_create": (_i32, [_vp, _vp, _i64, _i64, _vp, _i32, _i32, _i32, _vp, _c.POINTER(_vp)]),
    "tgt_reformat_num_edges": (_i64, [_vp]),
    "tgt_reformat_export": (_i32, [_vp, _vp, _vp, _vp]),
    "tgt_reformat_destroy": (_i32, [_vp]),
    "tgt_np_legacy_randint": (_i32, [_c.c_uint32, _vp, _i32, _vp]),
    "tgt_linear_fwd": (_i32, [_vp, _vp, _vp, _vp, _i32, _i64, _i32, _i32, _i32, _vp]),
    "tgt_linear_bwd_workspace_bytes": (_i64, [_i32, _i32, _i32]),
    "tgt_linear_bwd": (_i32, [_vp, _vp, _vp, _i32, _i64, _i32, _i32, _i32, _vp, _vp, _vp, _vp, _i64, _vp]),
    "tgt_linear_bwd_deferred": (_i32, [_vp, _vp, _vp, _i32, _i64, _i32, _i32, _i32, _vp, _vp, _vp, _vp, _i64, _vp, _vp]),
    "tgt_reduce_partials": (_i32, [_vp, _i32, _i32, _vp]),
    "tgt_linear_act_fwd": (_i32, [_vp, _vp, _vp, _i64, _i32, _i32, _i32, _i32, _vp, _vp, _vp]),
    "tgt_linear_act_bwd": (_i32, [_vp, _vp, _vp, _vp, _i64, _i32, _i32, _i32, _i32, _vp, _vp, _vp, _vp, _i64, _vp, _vp]),
    "tgt_add_layer_norm_fwd": (_i32, [_vp, _vp, _vp, _vp, _i64, _i32, _c.c_float, _i32, _vp, _vp, _vp, _vp, _vp]),
    "tgt_layer_norm_bwd_workspace_bytes": (_i64, [_i32]),
    "tgt_layer_norm_bwd": (_i32, [_vp, _vp, _vp, _vp, _vp, _vp, _i64, _i32, _i32, _vp, _vp, _vp, _vp, _i64, _vp]),
    "tgt_layer_norm_bwd_deferred": (_i32, [_vp, _vp, _vp, _vp, _vp, _vp, _i64, _i32, _i32, _vp, _vp, _vp, _vp, _i64, _vp, _vp]),
    "tgt_gelu_fwd": (_i32, [_vp, _i64, _i32, _vp, _vp]),
    "tgt_gelu_bwd": (_i32, [_vp, _vp, _i64, _i32, _vp, _vp]),
    "tgt_relu_fwd": (_i32, [_vp, _i64, _i32, _vp, _vp]),
    "tgt_relu_bwd": (_i32, [_vp, _vp, _i64, _i32, _vp, _vp]),
    "tgt_nll_loss_workspace_bytes": (_i64, [_i64]),
    "tgt_nll_loss_fwd": (_i32, [_vp, _vp, _i64, _i32, _i32, _i64, _vp, _vp, _vp, _i64, _vp]),
    "tgt_nll_loss_bwd": (_i32, [_vp, _vp, _vp, _i64, _i32, _i32, _i64, _vp, _vp]),
    "tgt_graph_attn_bias_fwd": (_i32, [_vp, _vp, _vp, _i32, _vp, _i32, _vp, _i32, _vp, _i32, _i32, _i32, _i32, _vp, _vp]),
    "tgt_graph_attn_bias_bwd_workspace_bytes": (_i64, [_i32, _i32, _i32]),
    "tgt_graph_attn_bias_bwd": (_i32, [_vp, _vp, _vp, _i32, _i32, _i32, _i32, _i32, _i32, _i32, _vp, _vp, _vp, _vp, _i64, _vp]),
    "tgt_floyd_warshall": (_i32, [_vp, _vp, _i32, _i32, _vp, _vp, _vp]),
    "tgt_graph_attn_bias_multi_hop_fwd": (_i32, [_vp, _vp, _vp, _i32, _i32, _vp, _i32, _vp, _i32, _vp, _i32, _vp, _i32, _i32, _i32,
                                                 _i32, _i32, _vp, _vp]),
    "tgt_graph_attn_bias_multi_hop_bwd_workspace_bytes": (_i64, [_i32, _i32, _i32, _i32]),
    "tgt_graph_attn_bias_multi_hop_bwd": (_i32, [_vp, _vp, _vp, _i32, _i32, _vp, _i32, _i32, _vp, _i32, _i32, _i32, _i32, _i32, _i32,
                                                 _vp, _vp, _vp, _vp, _vp, _i64, _vp]),
    "tgt_graph_node_feature_fwd": (_i32, [_vp, _vp, _vp, _i32, _vp, _i32, _vp, _i32, _vp, _i32, _vp, _i32, _i32, _i32, _i32, _vp, _vp]),
    "tgt_graph_node_feature_bwd_workspace_bytes": (_i64, [_i32, _i32, _i32, _i32]),
    "tgt_graph_node_feature_bwd": (_i32, [_vp, _vp, _vp, _vp, _i32, _i32, _i32, _i32, _i32, _i32, _i32, _i32, _vp, _vp, _vp, _vp, _vp,
                                          _i64, _vp]),
    "tgt_embedding_sum_fwd": (_i32, [_vp, _i32, _vp, _i32, _i32, _i32, _i32, _i32, _vp, _vp]),
    "tgt_embedding_sum_bwd_workspace_bytes": (_i64, [_i32, _i32]),
    "tgt_embedding_sum_bwd": (_i32, [_vp, _vp, _i32, _i32, _i32, _i32, _i32, _i32, _vp, _vp, _i64, _vp]),
    "tgt_gen_edge_input": (_i32, [_vp, _vp, _i32, _i32, _vp, _i32, _i32, _i32, _vp, _vp]),
    "tgt_timing_enable": (_i32, [_i32]),
    "tgt_timing_reset": (_i32, []),
    "tgt_timing_slots": (_i32, []),
    "tgt_timing_read": (_i32, [_i32, _c.POINTER(_c.c_char_p), _c.POINTER(_c.c_double), _c.POINTER(_i64)]),
}


class ReduceDesc(_c.Structure):
    """tgt_reduce_desc of include/torchgt_hip.h: a sum over workgroup partials that a *_deferred call leaves to
    tgt_reduce_partials."""
    _fields_ = [("partial", _c.c_void_p), ("workers", _c.c_int32), ("n", _c.c_int32), ("n_out", _c.c_int32),
                ("out", _c.c_void_p * 6), ("begin", _c.c_int32 * 6)]


def kernel_timings():
    """{kernel name: (total ms, launches)} since the last tgt_timing_reset()."""
    L = lib()
    out = {}
    for slot in range(L.tgt_timing_slots()):
        name, ms, n = _c.c_char_p(), _c.c_double(), _i64()
        check(L.tgt_timing_read(slot, _c.byref(name), _c.byref(ms), _c.byref(n)))
        out[name.value.decode()] = (ms.value, n.value)
    return out


class TorchGTHipError(RuntimeError):
    def __init__(self, code, message):
        super().__init__(f"libtorchgt_hip error {code}: {message}")
        self.code = code


_lib = None


def lib():
    """The loaded library (loads on first use; raises if it is not built)."""
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            raise ImportError(
                f"{LIB_PATH} is not built; run `python -m torchgt_amd.build` "
                "(there is no fallback implementation)")
        handle = ctypes.CDLL(LIB_PATH)
        for name, (res, args) in SIGNATURES.items():
            fn = getattr(handle, name)
            fn.restype = res
            fn.argtypes = args
        _lib = handle
    return _lib


def check(code):
    if code != OK:
        l = lib()
        detail = l.tgt_last_error().decode() or l.tgt_error_string(code).decode()
        raise TorchGTHipError(code, detail)
