"""ctypes binding of liboptimus_mi355x.so, the C-ABI library of HIP kernels.

This is the only place that touches the library.  Tensors are passed as raw device pointers
(`tensor.data_ptr()`), the stream is PyTorch's current HIP stream.  There is no fallback: if
the library is missing or a call returns an error code, an exception is raised.
"""
import ctypes
import os

import torch

_PKG_ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
LIB_PATH = os.path.join(_PKG_ROOT, "lib", "liboptimus_mi355x.so")

OM_F32, OM_BF16 = 0, 1
OM_I32, OM_I64 = 0, 1

c_void_p = ctypes.c_void_p
c_int = ctypes.c_int
c_i64 = ctypes.c_int64
c_double = ctypes.c_double

# name -> (restype, argtypes); mirrors include/optimus_mi355x.h one to one
SIGNATURES = {
    "om_version": (c_int, []),
    "om_arch": (ctypes.c_char_p, []),
    "om_strerror": (ctypes.c_char_p, [c_int]),
    "om_adamw_step": (c_int, [c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_i64, c_double,
                              c_double, c_double, c_double, c_double, c_i64, c_int, c_void_p]),
    "om_adamw_traffic_probe": (c_int, [c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_i64, c_void_p]),
    "om_grad_sumsq": (c_int, [c_void_p, c_int, c_void_p, c_i64, c_void_p, c_void_p]),
    "om_grad_norm_clip_coef": (c_int, [c_void_p, c_void_p, c_i64, c_int, c_double, c_void_p, c_void_p,
                                       c_void_p, c_void_p]),
    "om_grad_scale": (c_int, [c_void_p, c_i64, c_int, c_void_p, c_void_p]),
    "om_shard_clip_multiplier": (c_int, [c_void_p, c_int, c_int, c_double, c_void_p, c_void_p, c_void_p]),
    "om_adamw_step_clipped": (c_int, [c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_i64,
                                      c_double, c_double, c_double, c_double, c_double, c_i64, c_int,
                                      c_void_p, c_int, c_void_p]),
    "om_route_softmax_topk": (c_int, [c_void_p, c_int, c_i64, c_int, c_int, c_int, c_void_p, c_int,
                                      c_void_p, c_void_p]),
    "om_route_softmax_topk_bwd": (c_int, [c_void_p, c_int, c_void_p, c_void_p, c_int, c_i64, c_int,
                                          c_int, c_int, c_void_p, c_void_p]),
    "om_router_gate_softmax_topk": (c_int, [c_void_p, c_void_p, c_i64, c_int, c_int, c_int, c_int,
                                            c_void_p, c_void_p, c_int, c_void_p, c_void_p]),
    "om_router_gate_logits": (c_int, [c_void_p, c_void_p, c_i64, c_int, c_int, c_void_p, c_void_p]),
    "om_router_gate_logits_split_workspace_bytes": (c_i64, [c_i64, c_int, c_int]),
    "om_router_gate_logits_split": (c_int, [c_void_p, c_void_p, c_i64, c_int, c_int, c_void_p, c_void_p,
                                            c_i64, c_void_p]),
    "om_router_gate_wgrad_workspace_bytes": (c_i64, [c_i64, c_int, c_int]),
    "om_router_gate_wgrad": (c_int, [c_void_p, c_void_p, c_i64, c_int, c_int, c_void_p, c_int, c_void_p,
                                     c_i64, c_void_p]),
    "om_router_gate_dgrad": (c_int, [c_void_p, c_void_p, c_void_p, c_void_p, c_i64, c_int, c_int, c_void_p]),
    "om_router_gate_logits_f32": (c_int, [c_void_p, c_void_p, c_i64, c_int, c_int, c_void_p, c_void_p]),
    "om_router_gate_dgrad_f32": (c_int, [c_void_p, c_void_p, c_i64, c_int, c_int, c_void_p, c_void_p]),
    "om_router_gate_wgrad_f32": (c_int, [c_void_p, c_void_p, c_i64, c_int, c_int, c_void_p, c_void_p]),
    "om_router_balance_workspace_bytes": (c_i64, [c_i64, c_int]),
    "om_router_balance_stats": (c_int, [c_void_p, c_int, c_i64, c_int, c_int, c_void_p, c_void_p,
                                        c_void_p, c_i64, c_void_p]),
    "om_router_balance_stats_masked": (c_int, [c_void_p, c_int, c_void_p, c_i64, c_int, c_int, c_void_p, c_void_p,
                                               c_void_p, c_i64, c_void_p]),
    "om_router_balance_bwd_masked": (c_int, [c_void_p, c_int, c_void_p, c_void_p, c_i64, c_int, c_void_p, c_void_p]),
    "om_router_balance_bwd": (c_int, [c_void_p, c_int, c_void_p, c_i64, c_int, c_void_p, c_void_p]),
    "om_rmsnorm_fwd": (c_int, [c_void_p, c_void_p, c_void_p, c_double, c_void_p, c_void_p, c_void_p,
                               c_i64, c_i64, c_int, c_void_p]),
    "om_rmsnorm_bwd_workspace_bytes": (c_i64, [c_i64, c_i64]),
    "om_rmsnorm_bwd": (c_int, [c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p,
                               c_i64, c_i64, c_i64, c_int, c_void_p]),
    "om_route_sigmoid_group_topk": (c_int, [c_void_p, c_void_p, c_i64, c_int, c_int, c_int, c_int,
                                            c_int, c_double, c_void_p, c_void_p, c_void_p]),
    "om_route_sigmoid_topk_bwd": (c_int, [c_void_p, c_void_p, c_void_p, c_i64, c_int, c_int, c_int,
                                          c_double, c_void_p, c_void_p]),
    "om_moe_sort_workspace_bytes": (c_i64, [c_i64, c_int, c_int]),
    "om_moe_sort": (c_int, [c_void_p, c_int, c_i64, c_int, c_int, c_int, c_void_p, c_void_p,
                            c_void_p, c_void_p, c_void_p, c_void_p, c_i64, c_void_p]),
    "om_moe_sort_static_capacity_bytes": (c_i64, []),
    "om_moe_sort_static": (c_int, [c_void_p, c_int, c_i64, c_int, c_int, c_int, c_void_p, c_void_p,
                                   c_void_p, c_void_p, c_void_p, c_void_p]),
    "om_compute_partial_token_counts": (c_int, [c_void_p, c_int, c_void_p, c_void_p, c_int, c_int,
                                                c_i64, c_int, c_i64, c_void_p]),
    "om_compute_input_and_output_indices": (c_int, [c_void_p, c_int, c_void_p, c_void_p, c_void_p,
                                                    c_void_p, c_void_p, c_void_p, c_int, c_int,
                                                    c_i64, c_int, c_i64, c_void_p]),
    "om_index_add": (c_int, [c_void_p, c_void_p, c_void_p, c_i64, c_i64, c_int, c_void_p]),
    "om_index_gather": (c_int, [c_void_p, c_void_p, c_void_p, c_i64, c_i64, c_int, c_void_p]),
    "om_shuffle_sub_matrix_reduce": (c_int, [c_void_p, c_void_p, c_void_p, c_void_p, c_i64, c_i64,
                                             c_int, c_void_p]),
    "om_reduce_ggemm_output": (c_int, [c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p,
                                       c_i64, c_int, c_i64, c_int, c_int, c_int, c_void_p]),
    "om_reduce_ggemm_output_residual": (c_int, [c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p,
                                                c_void_p, c_i64, c_int, c_i64, c_int, c_int, c_void_p]),
    "om_reduce_ggemm_output_backward": (c_int, [c_void_p, c_void_p, c_void_p, c_void_p, c_void_p,
                                                c_void_p, c_void_p, c_void_p, c_i64, c_int, c_i64,
                                                c_int, c_int, c_void_p]),
    "om_grouped_gemm_fwd": (c_int, [c_void_p, c_void_p, c_void_p, c_void_p, c_i64, c_int, c_int,
                                    c_int, c_i64, c_void_p]),
    "om_grouped_gemm_dgrad": (c_int, [c_void_p, c_void_p, c_void_p, c_void_p, c_i64, c_int, c_int,
                                      c_int, c_i64, c_void_p]),
    "om_grouped_gemm_wgrad": (c_int, [c_void_p, c_void_p, c_void_p, c_void_p, c_i64, c_int, c_int,
                                      c_int, c_i64, c_void_p]),
    "om_grouped_gemm_fwd_f32": (c_int, [c_void_p, c_void_p, c_void_p, c_void_p, c_i64, c_int, c_int,
                                        c_int, c_i64, c_void_p]),
    "om_grouped_gemm_dgrad_f32": (c_int, [c_void_p, c_void_p, c_void_p, c_void_p, c_i64, c_int, c_int,
                                          c_int, c_i64, c_void_p]),
    "om_grouped_gemm_wgrad_f32": (c_int, [c_void_p, c_void_p, c_void_p, c_void_p, c_i64, c_int, c_int,
                                          c_int, c_i64, c_void_p]),
    "om_merged_mlp_gate_up_fwd": (c_int, [c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p,
                                          c_void_p, c_i64, c_int, c_int, c_int, c_i64, c_void_p]),
    "om_merged_mlp_gate_up_fwd_gathered": (c_int, [c_void_p, c_void_p, c_i64, c_void_p, c_void_p, c_void_p,
                                                   c_void_p, c_void_p, c_void_p, c_i64, c_int, c_int,
                                                   c_int, c_i64, c_void_p]),
    "om_grouped_gemm_wgrad_gathered": (c_int, [c_void_p, c_void_p, c_void_p, c_i64, c_void_p, c_void_p,
                                               c_i64, c_int, c_int, c_int, c_i64, c_void_p]),
    "om_grouped_gemm_wgrad_accumulate": (c_int, [c_void_p, c_void_p, c_void_p, c_void_p, c_i64, c_int, c_int,
                                                 c_int, c_i64, c_void_p]),
    "om_grouped_gemm_wgrad_f32_accumulate": (c_int, [c_void_p, c_void_p, c_void_p, c_void_p, c_i64, c_int,
                                                     c_int, c_int, c_i64, c_void_p]),
    "om_grouped_gemm_wgrad_gathered_accumulate": (c_int, [c_void_p, c_void_p, c_void_p, c_i64, c_void_p,
                                                          c_void_p, c_i64, c_int, c_int, c_int, c_i64,
                                                          c_void_p]),
    "om_grouped_gemm_wgrad_gathered_out_accumulate": (c_int, [c_void_p, c_void_p, c_i64, c_void_p, c_void_p,
                                                              c_void_p, c_i64, c_int, c_int, c_int, c_i64,
                                                              c_void_p]),
    "om_moe_row_weights": (c_int, [c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_i64, c_int, c_int,
                                   c_void_p]),
    "om_merged_mlp_gate_up_fwd_weighted": (c_int, [c_void_p, c_void_p, c_i64, c_void_p, c_void_p, c_void_p,
                                                   c_void_p, c_void_p, c_void_p, c_void_p, c_i64, c_int,
                                                   c_int, c_int, c_i64, c_void_p]),
    "om_sum_ggemm_output": (c_int, [c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_i64, c_i64, c_int,
                                    c_void_p]),
    "om_grouped_gemm_wgrad_gathered_out": (c_int, [c_void_p, c_void_p, c_i64, c_void_p, c_void_p, c_void_p,
                                                   c_i64, c_int, c_int, c_int, c_i64, c_void_p]),
    "om_merged_mlp_row_dot_parts": (c_int, [c_int]),
    "om_merged_mlp_down_dgrad_weighted": (c_int, [c_void_p, c_void_p, c_i64, c_void_p, c_void_p, c_void_p,
                                                  c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_i64,
                                                  c_int, c_int, c_int, c_i64, c_void_p]),
    "om_moe_row_weights_grad": (c_int, [c_void_p, c_int, c_void_p, c_void_p, c_void_p, c_void_p, c_i64,
                                        c_int, c_int, c_void_p]),
    "om_merged_mlp_down_dgrad": (c_int, [c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p,
                                         c_void_p, c_i64, c_int, c_int, c_int, c_i64, c_void_p]),
    "om_merged_mlp_gate_up_dgrad": (c_int, [c_void_p, c_void_p, c_void_p, c_void_p, c_void_p,
                                            c_void_p, c_i64, c_int, c_int, c_int, c_i64, c_void_p]),
    "om_swiglu_fwd": (c_int, [c_void_p, c_void_p, c_void_p, c_i64, c_int, c_void_p]),
    "om_swiglu_bwd": (c_int, [c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_i64, c_int,
                              c_void_p]),
}

_lib = None

# Optional per-launch timing: when set to a list, every call of a kernel-launching entry point
# appends (name, start_event, end_event) recorded on the current stream.  Used by bench.py to get
# kernel durations from HIP events inside the timed region; None (the default) costs one test.
launch_log = None
launch_filter = None   # optional set of entry-point names: only these are timed while launch_log is set
_UNTIMED = {"om_version", "om_arch", "om_strerror", "om_moe_sort_workspace_bytes",
            "om_moe_sort_static_capacity_bytes",
            "om_router_balance_workspace_bytes", "om_rmsnorm_bwd_workspace_bytes",
            "om_router_gate_wgrad_workspace_bytes", "om_router_gate_logits_split_workspace_bytes",
            "om_merged_mlp_row_dot_parts"}


class NativeLibraryError(RuntimeError):
    pass


class _Library:
    """The loaded C-ABI functions as attributes (om_adamw_step, ...)."""

    def __init__(self, handle):
        for name, (res, args) in SIGNATURES.items():
            fn = getattr(handle, name)
            fn.restype = res
            fn.argtypes = args
            setattr(self, name, fn if name in _UNTIMED else self._maybe_timed(name, fn))

    @staticmethod
    def _maybe_timed(name, fn):
        def call(*args):
            if launch_log is None or (launch_filter is not None and name not in launch_filter):
                return fn(*args)
            a = torch.cuda.Event(enable_timing=True)
            b = torch.cuda.Event(enable_timing=True)
            a.record()
            rc = fn(*args)
            b.record()
            launch_log.append((name, a, b))
            return rc
        return call


def lib():
    """Load the library (once).  Raises if it has not been built."""
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            raise NativeLibraryError(
                f"{LIB_PATH} not found: build it with `python optimus-lm_amd/build.py` "
                "(there is no non-HIP fallback)")
        _lib = _Library(ctypes.CDLL(LIB_PATH))
    return _lib


def check(code, what):
    if code != 0:
        msg = lib().om_strerror(code).decode()
        raise NativeLibraryError(f"{what} failed with code {code}: {msg}")


def dtype_code(t):
    if t.dtype == torch.float32:
        return OM_F32
    if t.dtype == torch.bfloat16:
        return OM_BF16
    raise TypeError(f"unsupported dtype {t.dtype}: the HIP kernels take float32 or bfloat16")


def index_code(t):
    if t.dtype == torch.int64:
        return OM_I64
    if t.dtype == torch.int32:
        return OM_I32
    raise TypeError(f"expert indices must be int64 or int32, got {t.dtype}")


def ptr(t):
    return None if t is None else t.data_ptr()


def stream():
    return torch.cuda.current_stream().cuda_stream


def require_cuda_contiguous(*tensors):
    for t in tensors:
        if t is None:
            continue
        if not t.is_cuda:
            raise NativeLibraryError("the HIP kernels need device tensors (got a CPU tensor); "
                                     "there is no CPU fallback")
        if not t.is_contiguous():
            raise NativeLibraryError("the HIP kernels need contiguous row-major tensors")
