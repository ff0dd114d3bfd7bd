"""The C-ABI library loads and exports every symbol include/actnn_hip.h declares (CPU test:
no kernel is launched)."""
import ctypes
import os
import re

from actnn_amd import _lib

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def _declared():
    text = open(os.path.join(ROOT, "include", "actnn_hip.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(actnn_[a-z0-9_]+)\s*\(", text)))


def test_header_symbols_are_exported(lib):
    names = _declared()
    assert len(names) >= 17
    raw = ctypes.CDLL(_lib.LIB_PATH)
    for n in names:
        assert hasattr(raw, n), f"{n} declared in include/actnn_hip.h but not exported"
    assert set(names) == set(_lib.SIGNATURES), "ctypes signature table out of sync with the header"


def test_argument_errors_need_no_gpu(lib):
    # invalid sizes / dtypes are rejected on the host before anything is launched
    assert lib.actnn_minimax(None, None, None, 4, 0, 0, None) == -1
    assert lib.actnn_minimax(None, None, None, 0, 256, 0, None) == 0          # empty input
    assert lib.actnn_pack_mixed(None, None, None, None, None, None, None, None, 0, 0, 4, 4, 100, 0, None) == -1
    assert lib.actnn_pack_single(None, None, None, 3, None, None, None, 0, 0, 4, 4, 256, 0, None) == -3
    assert lib.actnn_relu_forward(None, None, None, -1, 0, None) == -1
    assert lib.actnn_relu_forward(None, None, None, 0, 7, None) == 0
    assert lib.actnn_max_pool2d_forward(None, None, None, 1, 1, 8, 8, 4, 4, 4, 4, 2, 2, 1, 1, 0, None) == -1
    # batch norm takes every dense shape; the quantiser's outputs only where its groups align
    assert lib.actnn_batch_norm_workspace_bytes(8, 64, 56 * 56, 2, 0) > 0
    assert lib.actnn_batch_norm_workspace_bytes(8, 64, 56 * 56, 2, 1) > 0
    assert lib.actnn_batch_norm_workspace_bytes(32, 10, 1, 0, 0) > 0              # [N, C] rows, C % 4 != 0: element by element
    assert lib.actnn_batch_norm_workspace_bytes(32, 512, 1, 2, 0) > 0             # [N, C] rows: the channels-last kernels
    assert lib.actnn_batch_norm_workspace_bytes(4, 3, 49, 2, 0) > 0               # C*HW not in whole 16-byte chunks
    assert lib.actnn_batch_norm_workspace_bytes(4, 12, 49, 2, 1) > 0              # channels-last: C % 8 != 0
    assert lib.actnn_batch_norm_workspace_bytes(0, 12, 49, 2, 1) == -1
    assert lib.actnn_batch_norm_groups_align(8, 64, 56 * 56, 2, 0) == 1
    assert lib.actnn_batch_norm_groups_align(32, 512, 1, 2, 0) == 1               # [N, 512]: two groups per row
    assert lib.actnn_batch_norm_groups_align(32, 100, 1, 2, 0) == 0
    assert lib.actnn_batch_norm_groups_align(4, 3, 49, 2, 0) == 0
    assert lib.actnn_batch_norm_groups_align(8, 192, 64, 2, 1) == 0               # channels-last: 256 % C and C % 256 != 0
    assert lib.actnn_batch_norm_forward(None, None, None, None, None, None, None, None, None, None, None, 0,
                                        8, 64, 3136, 0.1, 1e-5, 2, 0, None) == -1   # null pointers
    assert lib.actnn_batch_norm_backward_packed(None, None, None, None, None, None, None, None, None, None, None,
                                                None, None, 0, None, 0, 8, 64, 3136, 7, 0, None) == -2   # unknown dtype code
    assert lib.actnn_batch_norm_backward_sumsq_entries(8, 64, 3136, 2, 0) > 0
    assert lib.actnn_batch_norm_backward_sumsq_entries(4, 3, 49, 2, 0) == 0       # element-by-element kernels leave none
    assert lib.actnn_sample_sqnorm(None, None, 4, 30, 1, 2, None) == -1           # F % 8 != 0
    assert lib.actnn_max_pool2d_forward_cl(None, None, None, 1, 8, 8, 8, 4, 4, 4, 4, 2, 2, 1, 1, 0, None) == -1
    for name in ("actnn_max_pool2d_forward_nibble", "actnn_max_pool2d_forward_cl_nibble",
                 "actnn_max_pool2d_backward_nibble", "actnn_max_pool2d_backward_cl_nibble"):
        assert getattr(lib, name)(None, None, None, 1, 8, 8, 8, 4, 4, 4, 4, 2, 2, 1, 1, 0, None) == -1    # KH*KW >= 16
        assert getattr(lib, name)(None, None, None, 1, 8, 8, 8, 4, 4, 3, 3, 2, 2, 1, 1, 0, None) == -1    # null pointers
    # the entry point with the built-in scratch array refuses what the array cannot hold
    assert lib.actnn_batch_norm_workspace_bytes(64, 1 << 20, 8, 2, 1) > lib.actnn_batch_norm_forward_static_limit()
    assert lib.actnn_batch_norm_forward_static(None, None, None, None, None, None, None, None, None, None,
                                               64, 1 << 20, 8, 0.1, 1e-5, 2, 1, None) == -5
    assert lib.actnn_strerror(-3) == b"unsupported bit width"
    assert b"gfx950" in lib.actnn_version()
