"""ctypes binding of ``libsswin3d.so`` (declarations in ``include/sswin3d.h``).

The library is the only compute path of this package.  If it is missing, loading raises:
there is no CPU or PyTorch fallback.
"""
from __future__ import annotations

import ctypes as C
import os

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "libsswin3d.so")

_vp, _i64, _i32, _sz = C.c_void_p, C.c_int64, C.c_int, C.c_size_t

class TokenPlanDesc(C.Structure):
    """``sswin_token_plan_desc`` of include/sswin3d.h: the arguments of one deferred sswin_token_plan call."""
    _fields_ = [("indices", _vp), ("N", _i64), ("B", C.c_int32), ("n", C.c_int32), ("H", C.c_int32),
                ("flags", C.c_int32), ("tokens", _vp), ("plan", _vp), ("g_cap", _i64), ("tasks", _vp),
                ("totals_out", _vp), ("ws", _vp), ("ws_bytes", _sz)]


# name -> (restype, argtypes); mirrors include/sswin3d.h one to one
SIGNATURES = {
    "sswin_calibration_copy": (_i32, [_vp, _vp, _i64, _vp]),
    "sswin_last_error": (C.c_char_p, []),
    "sswin_abi_version": (_i32, []),
    "sswin_flatten_indices": (_i32, [_vp, _i32, _i64, _vp, _vp, _vp]),
    "sswin_sort_indices_workspace_bytes": (_sz, [_i64]),
    "sswin_sort_indices": (_i32, [_vp, _i64, _vp, _vp, _sz, _vp]),
    "sswin_unique_consecutive_workspace_bytes": (_sz, [_i64]),
    "sswin_unique_consecutive_indices": (_i32, [_vp, _i32, _i64, _vp, _vp, _sz, _vp]),
    "sswin_unique_consecutive_indices_static": (_i32, [_vp, _i32, _i64, _vp, _vp]),
    "sswin_return_inverse_workspace_bytes": (_sz, [_i64, _i64]),
    "sswin_return_inverse": (_i32, [_vp, _i64, _i64, _vp, _vp, _vp, _sz, _vp]),
    "sswin_qkv_sparse_indices_workspace_bytes": (_sz, [_i64, _i32, _i32]),
    "sswin_qkv_sparse_indices": (_i32, [_vp, _i64, _i32, _i32, _i32, _i32, _vp, _vp, _vp, _vp, _vp, _sz, _i32, _vp, _vp]),
    "sswin_operand_map_workspace_bytes": (_sz, [_i64, _i32, _i32]),
    "sswin_operand_map": (_i32, [_vp, _i64, _i32, _i32, _vp, _vp, _sz, _i32, _vp, _vp]),
    "sswin_operand_copy_qkv": (_i32, [_i32, _i32, _vp, _i64, _i32, _vp, _vp, _vp, _vp, _i64, _i32, _i32, C.c_double, _vp]),
    "sswin_operand_copy": (_i32, [_i32, _i32, _i32, _vp, _i64, _i32, _vp, _vp, _i64, _i32, _i32, C.c_double, _vp]),
    "sswin_sorted_coo_indices": (_i32, [_vp, _vp, _i64, _i32, _i32, _vp, _vp, _vp]),
    "sswin_plan_workspace_bytes": (_sz, [_i64, _i32]),
    "sswin_plan_from_indices": (_i32, [_vp, _i64, _i32, _vp, _i64, _vp, _vp, _sz, _vp]),
    "sswin_permute_heads_order": (_i32, [_vp, _i64, _i32, _vp, _i64, _i64, _vp, _vp, _vp]),
    "sswin_softmax_rows_from_counts": (_i32, [_vp, _vp, _i64, _i64, _vp, _vp]),
    "sswin_group_add_bias_mask": (_i32, [_i32, _vp, _vp, _i64, _vp, _i64, _i64, _i32, _i32, _vp, _vp, _i32, _vp, _vp]),
    "sswin_group_add_table_bias_mask": (_i32, [_i32, _vp, _vp, _i64, _vp, _i64, _i64, _i32, _i32, _vp, _i32, _i32, _vp, _i32, _vp,
                                               _i32, _vp, _vp]),
    "sswin_group_row_positions": (_i32, [_vp, _i64, _vp, _i64, _i64, _vp, _vp]),
    "sswin_scan_counts_workspace_bytes": (_sz, [_i64]),
    "sswin_scan_counts": (_i32, [_vp, _i64, _vp, _vp, _sz, _vp]),
    "sswin_block_matmul": (_i32, [_i32, _i32, _vp, _vp, _vp, _i64, _i32, _vp, _i64, _i64, _i64, _vp, _vp, _i64, _vp]),
    "sswin_block_matmul_grad": (_i32, [_i32, _i32, _vp, _vp, _vp, _vp, _i64, _i32, _i64, _vp, _vp]),
    "sswin_block_transpose": (_i32, [_i32, _i32, _vp, _vp, _vp, _i64, _i32, _vp, _vp]),
    "sswin_softmax_last_dim_forward": (_i32, [_vp, _vp, _i32, _i64, _vp, _vp]),
    "sswin_softmax_last_dim_backward": (_i32, [_vp, _vp, _vp, _i32, _i64, _vp, _vp]),
    "sswin_token_plan_task_ints": (_sz, [_i64, _i64, _i32]),
    "sswin_token_plan_workspace_bytes": (_sz, [_i64, _i32, _i32]),
    "sswin_token_plan": (_i32, [_vp, _i64, _i32, _i32, _i32, _vp, _vp, _i64, _vp, _vp, _vp, _sz, _i32, _vp]),
    "sswin_token_plan_totals": (_i32, [_vp, _i32, _i64]),
    "sswin_token_plan_batch": (_i32, [_vp, _i32, _vp]),
    "sswin_fused_tokens_to_sq": (_i32, [_i32, _i32, _vp, _i64, _i64, _vp, _i64, _i32, _i32, _vp, _i64, _i32,
                                        _vp, _i64, _i32, C.c_float, _vp, _i32, _vp, _i32, _vp, _vp, _vp]),
    "sswin_fused_sq_to_tokens": (_i32, [_i32, _i32, _vp, _i64, _i64, _vp, _i64, _i32, _i32, _vp, _vp, _i64, _i32,
                                        _vp, _i64, _i32, C.c_float, _vp]),
    "sswin_fused_score_grad": (_i32, [_i32, _vp, _i64, _i64, _vp, _i64, _i32, _i32, _i32, _vp, _i64, _i32, _vp, _i64, _i32,
                                      _vp, _i64, _i32, _vp, _vp, _vp]),
    "sswin_group_softmax": (_i32, [_i32, _vp, _i64, _i64, _i64, _i32, _i32, _vp, _vp, _vp, _vp]),
    "sswin_fused_bias_grad_workspace_bytes": (_sz, [_i64, _i32, _i32]),
    "sswin_fused_bias_grad": (_i32, [_vp, _i64, _i64, _vp, _i64, _i32, _i32, _vp, _vp, _vp, _sz, _vp]),
    "sswin_column_sum_workspace_bytes": (_sz, [_i64, _i32]),
    "sswin_column_sum": (_i32, [_vp, _i32, _i64, _i32, _vp, _vp, _sz, _vp]),
    "sswin_bias_from_table": (_i32, [_vp, _i32, _i32, _vp, _i32, _i32, _vp, _vp]),
    "sswin_bias_table_grad_workspace_bytes": (_sz, [_i64, _i32, _i32]),
    "sswin_bias_table_grad": (_i32, [_vp, _i64, _i64, _vp, _i64, _i32, _i32, _vp, _i32, _i32, _vp, _vp, _vp, _sz, _vp]),
    "sswin_bias_table_grad_tasks": (_i32, [_vp, _i64, _vp, _i64, _vp, _i64, _i32, _i32, _vp, _i32, _i32, _vp, _vp, _vp, _sz,
                                           _vp]),
    "sswin_tall_linear_supported": (_i32, [_i32, _i32]),
    "sswin_tall_linear_forward": (_i32, [_vp, _i64, _i32, _vp, _vp, _i32, _vp, _vp]),
    "sswin_tall_linear_input_grad_supported": (_i32, [_i32, _i32]),
    "sswin_tall_linear_input_grad": (_i32, [_vp, _i64, _i32, _vp, _i32, _vp, _vp]),
    "sswin_tall_linear_weight_grad_workspace_bytes": (_sz, [_i64, _i32, _i32]),
    "sswin_tall_linear_weight_grad": (_i32, [_vp, _vp, _i64, _i32, _i32, _vp, _vp, _vp, _sz, _vp]),
    "sswin_window_indices": (_i32, [_vp, _i64, _i32, _vp, _vp, _vp, _vp, _vp]),
    "sswin_shift_mask": (_i32, [_vp, _vp, _vp, _vp, _vp]),
    "sswin_window_coords": (_i32, [_vp, _i64, _i64, _vp, _vp, _vp, _vp]),
    "sswin_pool_windows": (_i32, [_i32, _i32, _i32, _vp, _i64, _i64, _vp, _i64, _vp, _i64, _i32, _vp, _i64, _vp]),
    "sswin_window_attention_forward": (_i32, [_i32, _vp, _i64, _vp, _vp, _i64, _i32, _i32,
                                              _vp, _i64, _i32, _vp, _i64, _i32, _vp, _i64, _i32, C.c_float,
                                              _vp, _i32, _vp, _i32, _vp, _i64, _i32, _vp, _vp]),
    "sswin_window_attention_backward": (_i32, [_i32, _vp, _i64, _vp, _vp, _i64, _i32, _i32,
                                               _vp, _i64, _i32, _vp, _i64, _i32, _vp, _i64, _i32, C.c_float,
                                               _vp, _i32, _vp, _i32, _vp, _i64, _i32, _vp, _i64, _i32, _vp,
                                               _vp, _i64, _i32, _vp, _i64, _i32, _vp, _i64, _i32, _vp, _i32, _vp]),
}

ABI_VERSION = 29
_lib = None

# A list turns on timing of the library's launches: every call that takes a stream is bracketed by events on that
# stream and leaves (name, leading integer arguments, start event, stop event) here.  A benchmark uses it to time the
# kernels where they run, inside a module call or a step; None (the default) costs nothing.
launch_timer = None
launch_timer_only = None        # a set of entry point names restricts the timing to them (fewer events between the kernels)


class _TimedLibrary:
    """The loaded library with every stream-taking entry point bracketed by events (see ``launch_timer``)."""

    def __init__(self, lib):
        self._lib = lib

    def __getattr__(self, name):
        fn = getattr(self._lib, name)
        sig = SIGNATURES.get(name)
        if launch_timer is None or sig is None or sig[0] is not _i32 or not sig[1] or sig[1][-1] is not _vp or \
                (launch_timer_only is not None and name not in launch_timer_only):
            return fn

        def call(*args):
            import torch
            handle = getattr(args[-1], "value", None)
            stream = torch.cuda.ExternalStream(handle) if handle else torch.cuda.current_stream()
            start, stop = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            start.record(stream)
            status = fn(*args)
            stop.record(stream)
            if launch_timer is not None:
                launch_timer.append((name, tuple(a for a in args[:3] if isinstance(a, int)), start, stop))
            return status
        return call


class LibraryMissing(RuntimeError):
    pass


def load():
    """Load the HIP library once.  Raises :class:`LibraryMissing` if it has not been built."""
    global _lib
    if _lib is not None:
        return _lib if launch_timer is None else _TimedLibrary(_lib)
    if not os.path.exists(LIB_PATH):
        raise LibraryMissing(
            f"{LIB_PATH} not found: build it with `python -m sparseswin3d_amd.build` "
            "(there is no CPU fallback for the sparse window-attention operators)")
    # One HIP runtime per process: the tensors and streams handed to the library come from
    # PyTorch, so PyTorch's own libamdhip64 must be the one already resident when the library's
    # dependency on libamdhip64.so.7 is resolved (the loader reuses it by SONAME).
    import torch
    torch_hip = os.path.join(os.path.dirname(torch.__file__), "lib", "libamdhip64.so")
    if os.path.exists(torch_hip):
        C.CDLL(torch_hip, mode=C.RTLD_GLOBAL)
    lib = C.CDLL(LIB_PATH)
    for name, (res, args) in SIGNATURES.items():
        fn = getattr(lib, name)          # AttributeError here means header and library disagree
        fn.restype = res
        fn.argtypes = args
    if lib.sswin_abi_version() != ABI_VERSION:
        raise RuntimeError(f"libsswin3d ABI {lib.sswin_abi_version()} != binding ABI {ABI_VERSION}; rebuild")
    _lib = lib
    return lib


class _NoSwitch:
    def __enter__(self):
        return None

    def __exit__(self, *exc):
        return False


_NO_SWITCH = _NoSwitch()


def on_device(device):
    """Context manager that makes ``device`` the current one for a library call; when it is current already (the
    usual case) nothing is switched: ``torch.cuda.device`` costs several microseconds on the host per use, a
    noticeable share of an operator that takes twenty on the GPU."""
    import torch
    if device.index is None or device.index == torch.cuda.current_device():
        return _NO_SWITCH
    return torch.cuda.device(device)


def stream_handle(device):
    """The current HIP stream of ``device`` as the ``void*`` the library takes."""
    import torch
    index = device.index if device.index is not None else torch.cuda.current_device()
    return C.c_void_p(torch._C._cuda_getCurrentRawStream(index))


def check(status: int):
    """Turn a non-zero status into RuntimeError carrying the library's message."""
    if status != 0:
        raise RuntimeError(load().sswin_last_error().decode("utf-8", "replace"))
