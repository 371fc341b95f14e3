"""The C-ABI library loads without a GPU and exports every symbol that
include/torchgt_hip.h declares; host-only entry points behave."""
import ctypes
import os
import re

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
HEADER = os.path.join(ROOT, "include", "torchgt_hip.h")


def declared_functions():
    text = open(HEADER).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(tgt_[a-z0-9_]+)\s*\(", text)))


def test_header_declares_expected_entry_points():
    names = declared_functions()
    for must in ("tgt_plan_create", "tgt_plan_destroy", "tgt_sparse_attn_fwd", "tgt_sparse_attn_bwd",
                 "tgt_sparse_attn_workspace_bytes", "tgt_plan_export"):
        assert must in names


def test_library_exports_every_declared_symbol():
    from torchgt_amd import _lib
    if not os.path.exists(_lib.LIB_PATH):
        pytest.fail(f"{_lib.LIB_PATH} not built (python -m torchgt_amd.build)")
    handle = ctypes.CDLL(_lib.LIB_PATH)
    for name in declared_functions():
        assert hasattr(handle, name), f"{name} declared in torchgt_hip.h but not exported"
    # the ctypes table covers the same set
    assert sorted(_lib.SIGNATURES) == declared_functions()


def test_host_only_entry_points():
    from torchgt_amd import _lib
    L = _lib.lib()
    assert L.tgt_version() >= 1
    assert L.tgt_error_string(0) == b"ok"
    assert b"range" in L.tgt_error_string(_lib.ERR_INDEX_RANGE)
    # argument validation happens before any GPU call
    out = ctypes.c_void_p()
    assert L.tgt_plan_create(None, None, -1, 10, None, ctypes.byref(out)) == _lib.ERR_INVALID_ARG
    assert L.tgt_plan_create(None, None, 5, 10, None, ctypes.byref(out)) == _lib.ERR_INVALID_ARG
    assert L.tgt_plan_create(None, None, 0, 0, None, ctypes.byref(out)) == _lib.ERR_INVALID_ARG
    assert L.tgt_last_error() != b""
    assert L.tgt_plan_destroy(None) == 0
    assert L.tgt_sparse_attn_workspace_bytes(None, 8, 8) == -1
    assert L.tgt_sparse_attn_fwd(None, None, None, None, None, 0, 8, 8, 0, None, None, None, 0, None) \
        == _lib.ERR_INVALID_ARG
    # the entry points around the path refuse bad arguments before they touch the GPU as well
    assert L.tgt_nll_loss_workspace_bytes(-1) == -1 and L.tgt_nll_loss_workspace_bytes(64000) == 8 * 250
    assert L.tgt_nll_loss_fwd(None, None, -1, 40, 0, -100, None, None, None, 0, None) == _lib.ERR_INVALID_ARG
    assert L.tgt_nll_loss_fwd(None, None, 10, 40, 7, -100, None, None, None, 0, None) == _lib.ERR_INVALID_ARG      # dtype
    assert L.tgt_nll_loss_bwd(None, None, None, 0, 40, 0, -100, None, None) == 0                                   # nothing to do
    assert L.tgt_reduce_partials(None, 0, 0, None) == 0
    assert L.tgt_reduce_partials(None, 3, 0, None) == _lib.ERR_INVALID_ARG
    empty = (_lib.ReduceDesc * 2)()
    assert L.tgt_reduce_partials(empty, 2, 0, None) == _lib.ERR_INVALID_ARG                                        # not filled in
    assert L.tgt_linear_act_fwd(None, None, None, 16, 64, 64, 0, 0, None, None, None) == _lib.ERR_INVALID_ARG       # activation
    assert L.tgt_linear_act_bwd(None, None, None, None, 16, 64, 64, 0, 1, None, None, None, None, 0, None, None) == _lib.ERR_INVALID_ARG
    assert ctypes.sizeof(_lib.ReduceDesc) == 8 + 3 * 4 + 4 + 6 * 8 + 6 * 4                                       # the C struct's layout
    key = (ctypes.c_uint64 * 2)()
    assert L.tgt_edge_index_hash(None, None, -1, None, key) == _lib.ERR_INVALID_ARG
    assert L.tgt_edge_index_hash(None, None, 4, None, key) == _lib.ERR_INVALID_ARG
    assert L.tgt_edge_index_hash(None, None, 0, None, None) == _lib.ERR_INVALID_ARG
    # an allocator is both functions or neither
    CB = ctypes.CFUNCTYPE(ctypes.c_void_p, ctypes.c_size_t, ctypes.c_void_p, ctypes.c_void_p)
    assert L.tgt_set_allocator(ctypes.cast(CB(lambda n, s, u: None), ctypes.c_void_p), None, None) == _lib.ERR_INVALID_ARG


def test_torch_extension_loads_and_registers_its_operators():
    """The PyTorch-ROCm extension (csrc/torch_binding.cpp) loads without a GPU, registers every operator the Python
    layer calls, and refuses CPU tensors instead of falling back."""
    import torch
    from torchgt_amd import _ext
    ops = _ext.ops()
    for name in ("sparse_attention", "dense_attention", "dense_attention_ids", "linear", "add_layer_norm", "add", "gelu", "relu",
                 "ffn", "nll_loss", "multi_head_attention", "encoder_layer", "dense_encoder_layer"):
        assert hasattr(ops, name), name
    assert hasattr(torch.classes.torchgt, "PlanHolder")
    with pytest.raises(RuntimeError, match="GPU"):
        ops.gelu(torch.zeros(8))
    with pytest.raises(RuntimeError, match="GPU"):
        ops.linear(torch.zeros(4, 8), [torch.zeros(8, 8)], [None])
