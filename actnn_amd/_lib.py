"""Build and load ``libactnn_hip.so`` - the C-ABI library of gfx950 kernels (include/actnn_hip.h).

The library is compiled in-tree with hipcc and loaded with ctypes; there is no CPU fallback:
if the library is missing, ``load()`` raises.
"""
import ctypes
import os
import subprocess

_HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(_HERE, "csrc")
LIB_PATH = os.path.join(_HERE, "libactnn_hip.so")
SOURCES = ["minimax.hip", "pack_mixed.hip", "pack_single.hip", "mask_ops.hip", "maxpool.hip",
           "linear_gw.hip", "misc.hip", "calc_precision.cpp", "calc_precision_dev.hip", "batch_norm.hip"]
HIPCC_FLAGS = [
    "--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC", "-shared",
    "-ffp-contract=off",                      # bit-exact quantiser: no implicit FMA
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",   # no packed-FP32 codegen
    "-Wno-unused-command-line-argument",
]

c_i64, c_i32, c_u64, c_vp = ctypes.c_int64, ctypes.c_int, ctypes.c_uint64, ctypes.c_void_p

# name -> argtypes (restype is int unless listed in _RESTYPES); mirrors include/actnn_hip.h
SIGNATURES = {
    "actnn_strerror": [c_i32],
    "actnn_version": [],
    "actnn_minimax": [c_vp, c_vp, c_vp, c_i64, c_i64, c_i32, c_vp],
    "actnn_calc_precision_dp": [c_vp, c_vp, c_i64, c_i32, c_i32, c_i32, c_vp, c_vp],
    "actnn_calc_precision_device": [c_vp, c_vp, c_i64, c_i32, c_i64, c_vp],
    "actnn_range_sqr": [c_vp, c_vp, c_vp, c_i64, c_i64, ctypes.c_float, c_vp, c_i32, c_i32, c_vp],
    "actnn_sample_sqnorm": [c_vp, c_vp, c_i64, c_i64, c_i32, c_i32, c_vp],
    "actnn_allocate_bits_device": [c_vp, c_vp, ctypes.c_float, c_vp, c_i32, c_vp, c_vp, c_vp, c_i64, c_i64, c_i32,
                                   c_i64, c_i32, c_vp],
    "actnn_bits_prefix": [c_vp, c_vp, c_i64, c_vp],
    "actnn_pack_mixed": [c_vp, c_vp, c_vp, c_vp, c_vp, c_vp, c_vp, c_vp, c_u64, c_u64,
                         c_i64, c_i64, c_i64, c_i32, c_vp],
    "actnn_unpack_mixed": [c_vp, c_vp, c_vp, c_vp, c_vp, c_vp, c_i64, c_i64, c_i64, c_i32, c_vp],
    "actnn_pack_single": [c_vp, c_vp, c_vp, c_i32, c_vp, c_vp, c_vp, c_u64, c_u64,
                          c_i64, c_i64, c_i64, c_i32, c_vp],
    "actnn_unpack_single": [c_vp, c_i32, c_vp, c_vp, c_vp, c_i64, c_i64, c_i64, c_i32, c_vp],
    "actnn_relu_forward": [c_vp, c_vp, c_vp, c_i64, c_i32, c_vp],
    "actnn_relu_forward_minmax": [c_vp, c_vp, c_vp, c_vp, c_vp, c_i64, c_i32, c_vp],
    "actnn_relu_add_forward": [c_vp, c_vp, c_vp, c_vp, c_vp, c_vp, c_i64, c_i32, c_vp],
    "actnn_relu_backward": [c_vp, c_vp, c_vp, c_i64, c_i32, c_vp],
    "actnn_relu_backward_add": [c_vp, c_vp, c_vp, c_vp, c_i64, c_i32, c_vp],
    "actnn_dropout_forward": [c_vp, c_vp, c_vp, c_i64, ctypes.c_float, c_u64, c_u64, c_i32, c_vp],
    "actnn_dropout_backward": [c_vp, c_vp, c_vp, c_i64, ctypes.c_float, c_i32, c_vp],
    "actnn_max_pool2d_forward": [c_vp, c_vp, c_vp, c_i64, c_i64, c_i64, c_i64, c_i64, c_i64,
                                 c_i32, c_i32, c_i32, c_i32, c_i32, c_i32, c_i32, c_vp],
    "actnn_max_pool2d_backward": [c_vp, c_vp, c_vp, c_i64, c_i64, c_i64, c_i64, c_i64, c_i64,
                                  c_i32, c_i32, c_i32, c_i32, c_i32, c_i32, c_i32, c_vp],
    "actnn_max_pool2d_forward_cl": [c_vp, c_vp, c_vp, c_i64, c_i64, c_i64, c_i64, c_i64, c_i64,
                                    c_i32, c_i32, c_i32, c_i32, c_i32, c_i32, c_i32, c_vp],
    "actnn_max_pool2d_backward_cl": [c_vp, c_vp, c_vp, c_i64, c_i64, c_i64, c_i64, c_i64, c_i64,
                                     c_i32, c_i32, c_i32, c_i32, c_i32, c_i32, c_i32, c_vp],
    "actnn_max_pool2d_forward_nibble": [c_vp, c_vp, c_vp, c_i64, c_i64, c_i64, c_i64, c_i64, c_i64,
                                        c_i32, c_i32, c_i32, c_i32, c_i32, c_i32, c_i32, c_vp],
    "actnn_max_pool2d_backward_nibble": [c_vp, c_vp, c_vp, c_i64, c_i64, c_i64, c_i64, c_i64, c_i64,
                                         c_i32, c_i32, c_i32, c_i32, c_i32, c_i32, c_i32, c_vp],
    "actnn_max_pool2d_forward_cl_nibble": [c_vp, c_vp, c_vp, c_i64, c_i64, c_i64, c_i64, c_i64, c_i64,
                                           c_i32, c_i32, c_i32, c_i32, c_i32, c_i32, c_i32, c_vp],
    "actnn_max_pool2d_backward_cl_nibble": [c_vp, c_vp, c_vp, c_i64, c_i64, c_i64, c_i64, c_i64, c_i64,
                                            c_i32, c_i32, c_i32, c_i32, c_i32, c_i32, c_i32, c_vp],
    "actnn_calc_precision": [c_vp, c_vp, c_vp, c_i64, ctypes.c_double],
    "actnn_linear_grad_weight": [c_vp, c_vp, c_vp, c_vp, c_i32, c_vp, c_vp, c_vp, c_i64, c_i64, c_i64,
                                 c_i32, c_i32, c_i32, c_vp],
    "actnn_linear_grad_weight_workspace_bytes": [c_i64, c_i64, c_i64],
    "actnn_linear_grad_weight_ws": [c_vp, c_vp, c_vp, c_vp, c_i32, c_vp, c_vp, c_vp, c_i64, c_i64, c_i64,
                                    c_i32, c_i32, c_i32, c_vp, c_i64, c_vp],
    "actnn_linear_grad_weight_q2": [c_vp, c_vp, c_vp, c_vp, c_vp, c_i64, c_i64, c_i64,
                                    c_i32, c_i32, c_i32, c_vp],
    "actnn_stream_copy": [c_vp, c_vp, c_i64, c_vp],
    "actnn_matrix_pipe_probe": [c_vp, c_vp, c_i32, c_i32, c_vp],
    "actnn_batch_norm_workspace_bytes": [c_i64, c_i64, c_i64, c_i32, c_i32],
    "actnn_batch_norm_forward": [c_vp, c_vp, c_vp, c_vp, c_vp, c_vp, c_vp, c_vp, c_vp, c_vp, c_vp, c_i64,
                                 c_i64, c_i64, c_i64, ctypes.c_double, ctypes.c_double, c_i32, c_i32, c_vp],
    "actnn_batch_norm_forward_static_limit": [],
    "actnn_batch_norm_forward_static": [c_vp, c_vp, c_vp, c_vp, c_vp, c_vp, c_vp, c_vp, c_vp, c_vp, c_i64, c_i64,
                                        c_i64, ctypes.c_double, ctypes.c_double, c_i32, c_i32, c_vp],
    # x weight bias rm rv y save_mean save_invstd mn mx ws | ws_bytes | factor mult per_sample | sens bits prefix |
    # initial target | scale packed | seed offset | relu_mask relu_mn relu_mx residual | N C HW | momentum eps |
    # dtype channels_last stream
    "actnn_batch_norm_forward_quantize": [c_vp] * 11 + [c_i64, ctypes.c_float, c_vp, c_i32, c_vp, c_vp, c_vp,
                                          c_i32, c_i64, c_vp, c_vp, c_u64, c_u64, c_vp, c_vp, c_vp, c_vp, c_i64, c_i64,
                                          c_i64, ctypes.c_double, ctypes.c_double, c_i32, c_i32, c_vp],
    "actnn_batch_norm_forward_apply_relu": [c_vp, c_vp, c_vp, c_i64, c_vp, c_vp, c_vp, c_vp, c_vp, c_vp, c_u64,
                                            c_u64, c_vp, c_vp, c_vp, c_vp, c_i64, c_i64, c_i64, c_i32, c_i32, c_vp],
    "actnn_quantize_activation": [c_vp, c_vp, c_vp, c_i32, ctypes.c_float, c_vp, c_i32, c_vp, c_vp, c_vp, c_i32,
                                  c_i64, c_vp, c_vp, c_u64, c_u64, c_i64, c_i64, c_i32, c_vp],
    "actnn_batch_norm_forward_stats": [c_vp, c_vp, c_vp, c_vp, c_vp, c_vp, c_vp, c_vp, c_vp, c_vp, c_i64,
                                       c_i64, c_i64, c_i64, ctypes.c_double, ctypes.c_double, c_i32, c_i32, c_vp],
    "actnn_batch_norm_forward_apply": [c_vp, c_vp, c_vp, c_i64, c_vp, c_vp, c_vp, c_vp, c_vp, c_vp, c_u64, c_u64,
                                       c_i64, c_i64, c_i64, c_i32, c_i32, c_vp],
    "actnn_batch_norm_backward_packed": [c_vp, c_vp, c_vp, c_vp, c_vp, c_vp, c_vp, c_vp, c_vp, c_vp, c_vp,
                                         c_vp, c_vp, c_i64, c_vp, c_i64, c_i64, c_i64, c_i64, c_i32, c_i32, c_vp],
    "actnn_batch_norm_backward_packed_relu": [c_vp] * 14 + [c_i64, c_vp, c_i64, c_i64, c_i64, c_i64, c_i32, c_i32,
                                              c_vp],
    "actnn_batch_norm_backward": [c_vp, c_vp, c_vp, c_vp, c_vp, c_vp, c_vp, c_vp, c_vp, c_i64, c_vp, c_i64,
                                  c_i64, c_i64, c_i64, c_i32, c_i32, c_vp],
    "actnn_batch_norm_backward_sumsq_entries": [c_i64, c_i64, c_i64, c_i32, c_i32],
    "actnn_batch_norm_groups_align": [c_i64, c_i64, c_i64, c_i32, c_i32],
    "actnn_batch_norm_forward_eval": [c_vp, c_vp, c_vp, c_vp, c_vp, c_vp, c_vp, c_vp, c_vp, c_i64, c_i64, c_i64,
                                      c_i64, ctypes.c_double, c_i32, c_i32, c_vp],
    "actnn_batch_norm_backward_eval": [c_vp, c_vp, c_vp, c_vp, c_vp, c_vp, c_vp, c_vp, c_vp, c_i64, c_i64, c_i64,
                                       c_i64, c_i32, c_i32, c_vp],
}
_RESTYPES = {"actnn_strerror": ctypes.c_char_p, "actnn_version": ctypes.c_char_p,
             "actnn_linear_grad_weight_workspace_bytes": ctypes.c_int64,
             "actnn_batch_norm_workspace_bytes": ctypes.c_int64,
             "actnn_batch_norm_forward_static_limit": ctypes.c_int64,
             "actnn_batch_norm_backward_sumsq_entries": ctypes.c_int64}

_lib = None


def build(verbose=False):
    """Compile every source under csrc/ into libactnn_hip.so (always recompiles)."""
    srcs = [os.path.join(CSRC, s) for s in SOURCES]
    tmp = LIB_PATH + ".tmp"
    cmd = ["hipcc", *HIPCC_FLAGS, *srcs, "-o", tmp]
    if verbose:
        print(" ".join(cmd), flush=True)
    proc = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    # the host pass does not know the device-only target feature and says so once per file
    noise = "'-packed-fp32-ops' is not a recognized feature for this target"
    out = "\n".join(l for l in proc.stdout.splitlines() if noise not in l)
    if out.strip():
        print(out, flush=True)
    if proc.returncode != 0:
        raise RuntimeError(f"hipcc failed with exit code {proc.returncode}")
    os.replace(tmp, LIB_PATH)
    global _lib
    _lib = None
    return LIB_PATH


def load():
    """Load the library (once) and attach argument types.  Raises if it has not been built."""
    global _lib
    if _lib is not None:
        return _lib
    if not os.path.exists(LIB_PATH):
        raise RuntimeError(
            f"{LIB_PATH} is missing: the HIP kernels are not built. Run "
            "`python -c 'import __graft_entry__ as g; g.build()'` (needs hipcc). "
            "There is no CPU fallback.")
    lib = ctypes.CDLL(LIB_PATH)
    for name, argtypes in SIGNATURES.items():
        fn = getattr(lib, name)            # AttributeError if the header and library disagree
        fn.argtypes = argtypes
        fn.restype = _RESTYPES.get(name, ctypes.c_int)
    _lib = lib
    return lib


def check(rc, what):
    """Turn a non-zero return code into RuntimeError (the reference raises c10::Error ->
    RuntimeError from TORCH_CHECK, ext_common.h)."""
    if rc != 0:
        msg = load().actnn_strerror(int(rc)).decode()
        raise RuntimeError(f"{what} failed: {msg} (code {rc})")
