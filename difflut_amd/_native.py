"""ctypes binding of libdifflut_hip.so (the C ABI declared in include/difflut_hip.h).

The library never falls back: if it is missing, or a tensor handed to it is not on a
ROCm device, the calls raise (CPU tensors are dispatched to plain-torch operators before
they get here, difflut_amd/ops.py).  Tensors are passed as raw device pointers together
with torch's current HIP stream; outputs and workspaces are allocated by the
caller with torch's caching allocator.
"""
import ctypes
import os

import torch

_HERE = os.path.dirname(os.path.abspath(__file__))
# DIFFLUT_HIP_LIB points at another build of the same library (kernel experiments)
LIB_PATH = os.environ.get("DIFFLUT_HIP_LIB") or os.path.join(_HERE, "lib", "libdifflut_hip.so")

_P, _I, _F, _Z = ctypes.c_void_p, ctypes.c_int, ctypes.c_float, ctypes.c_size_t

# name -> (restype, argtypes); mirrors include/difflut_hip.h one to one
SIGNATURES = {
    "dl_version": (_I, []),
    "dl_error_string": (ctypes.c_char_p, [_I]),
    "dl_gather_fwd": (_I, [_P, _P, _I, _P, _I, _I, _I, _I, _P]),
    "dl_gather_bwd": (_I, [_P, _P, _P, _P, _I, _I, _I, _I, _P]),
    "dl_dwn_saved_bytes": (_Z, [_I] * 5),
    "dl_dwn_fwd_workspace_bytes": (_Z, [_I] * 5),
    "dl_dwn_bwd_workspace_bytes": (_Z, [_I] * 5),
    "dl_dwn_layer_fwd": (_I, [_P, _P, _P, _P, _P, _P, _Z, _I, _I, _I, _I, _I, _P]),
    "dl_dwn_layer_fwd_static": (_I, [_P, _P, _P, _P, _P, _I, _I, _I, _I, _I, _P]),
    "dl_dwn_layer_bwd": (_I, [_P, _P, _P, _P, _P, _P, _P, _F, _F, _P, _P, _P, _Z, _I, _I, _I, _I, _I, _P]),
    "dl_dwn_layer_bwd_nodes": (_I, [_P, _P, _P, _P, _P, _P, _P, _P, _P, _F, _P, _P, _P, _Z, _I, _I, _I, _I, _I, _P]),
    "dl_dwn_layer_eval": (_I, [_P, _P, _P, _P, _I, _I, _I, _I, _I, _P]),
    "dl_dwn_planes_bytes": (_Z, [_I] * 2),
    "dl_dwn_tiled_bytes": (_Z, [_I] * 2),
    "dl_dwn_pack_planes": (_I, [_P, _P, _I, _I, _P]),
    "dl_dwn_layer_fwd_planes": (_I, [_P, _P, _P, _P, _P, _P, _I, _I, _I, _I, _I, _P]),
    "dl_dwn_layer_bwd_tiled": (_I, [_P, _P, _P, _P, _P, _I, _F, _F, _P, _I, _P, _P, _Z, _I, _I, _I, _I, _I, _P]),
    "dl_dwn_eval_workspace_bytes": (_Z, [_I] * 5),
    "dl_dwn_layer_eval_ws": (_I, [_P, _P, _P, _P, _P, _Z, _I, _I, _I, _I, _I, _P]),
    "dl_dwn_layer_eval_planes": (_I, [_P, _P, _P, _P, _P, _I, _I, _I, _I, _I, _P]),
    "dl_dwn_layer_eval_planes_groups": (_I, [_P, _P, _P, _P, _P, _Z, _I, _I, _I, _I, _I, _I, _F, _P]),
    "dl_dwn_groups_workspace_bytes": (_Z, [_I] * 4),
    "dl_dwn_layer_fwd_planes_groups": (_I, [_P, _P, _P, _P, _P, _P, _Z, _I, _I, _I, _I, _I, _I, _F, _P]),
    "dl_dwn_layer_bwd_groups": (_I, [_P, _P, _P, _P, _P, _I, _F, _F, _F, _P, _I, _P, _P, _Z, _I, _I, _I, _I, _I, _P]),
    "dl_dwn_layer_bwd_chain_nodes": (_I, [_P, _P, _P, _P, _P, _I, _I, _F, _P, _P, _F, _P, _I, _P, _P, _Z, _I, _I, _I, _I, _I, _P]),
    "dl_dwn_chain_fusable": (_I, [_I, _I, _I, _I, _I, _I, _F]),
    "dl_dwn_bwd_fused_workspace_bytes": (_Z, [_I, _I, _I, _I, _I, _I]),
    "dl_dwn_layer_bwd_chain_fused": (_I, [_P, _P, _P, _P, _P, _I, _I, _F, _P, _P, _F, _P, _I, _P, _P, _I, _P, _P, _Z,
                                          _I, _I, _I, _I, _I, _P]),
    "dl_dwn_stable_layer_bwd": (_I, [_P, _P, _P, _P, _P, _P, _P, _P, _P, _P, _P, _Z, _I, _I, _I, _I, _I, _P]),
    "dl_table_sigmoid_fwd": (_I, [_P, _P, ctypes.c_longlong, _P]),
    "dl_table_sigmoid_bwd": (_I, [_P, _P, _P, ctypes.c_longlong, _P]),
    "dl_hybrid_bwd_workspace_bytes": (_Z, [_I] * 5),
    "dl_hybrid_layer_bwd": (_I, [_P, _P, _P, _P, _P, _P, _P, _P, _P, _Z, _I, _I, _I, _I, _I, _P]),
    "dl_prob_saved_bytes": (_Z, [_I] * 5),
    "dl_prob_bwd_workspace_bytes": (_Z, [_I] * 5),
    "dl_prob_layer_fwd": (_I, [_P, _P, _P, _F, _P, _P, _Z, _I, _I, _I, _I, _I, _P]),
    "dl_prob_layer_bwd": (_I, [_P, _P, _P, _P, _P, _P, _F, _P, _P, _P, _P, _Z, _I, _I, _I, _I, _I, _P]),
    "dl_prob_layer_fwd_nodes": (_I, [_P, _P, _P, _P, _P, _P, _Z, _I, _I, _I, _I, _I, _P]),
    "dl_prob_layer_bwd_nodes": (_I, [_P, _P, _P, _P, _P, _P, _P, _P, _P, _P, _P, _Z, _I, _I, _I, _I, _I, _P]),
    "dl_prob_layer_eval_ws_nodes": (_I, [_P, _P, _P, _P, _P, _P, _Z, _I, _I, _I, _I, _I, _P]),
    "dl_prob_eval_workspace_bytes": (_Z, [_I] * 5),
    "dl_prob_layer_eval_ws": (_I, [_P, _P, _P, _F, _P, _P, _Z, _I, _I, _I, _I, _I, _P]),
    "dl_prob_layer_eval": (_I, [_P, _P, _P, _F, _P, _I, _I, _I, _I, _I, _P]),
    "dl_soft_map_saved_bytes": (_Z, [_I] * 4),
    "dl_soft_map_workspace_bytes": (_Z, [_I] * 4),
    "dl_soft_map_fwd": (_I, [_P, _P, _F, _P, _P, _P, _Z, _I, _I, _I, _I, _P]),
    "dl_soft_map_bwd": (_I, [_P, _P, _F, _P, _P, _P, _P, _P, _P, _Z, _I, _I, _I, _I, _P]),
    "dl_row_argmax": (_I, [_P, _P, _I, _I, _P]),
    "dl_hard_select_fwd": (_I, [_P, _P, _P, _I, _I, _I, _P]),
    "dl_hard_select_bwd": (_I, [_P, _P, _P, _P, _I, _I, _I, _P]),
    "dl_thermometer_encode": (_I, [_P, _P, _P, _I, _I, _I, _P]),
    "dl_thermometer_planes": (_I, [_P, _P, _P, _I, _I, _I, _P]),
    "dl_unfold_rows": (ctypes.c_longlong, [_I] * 9),
    "dl_unfold": (_I, [_P, _P, _P] + [_I] * 10 + [_P]),
    "dl_unfold_flip": (_I, [_P, _P, _P, _P] + [_I] * 10 + [_P]),
    "dl_fold": (_I, [_P, _I, _P] + [_I] * 10 + [_P]),
    "dl_group_sum_fwd": (_I, [_P, _P, _I, _I, _I, _F, _P]),
    "dl_cross_entropy_workspace_bytes": (_Z, [_I]),
    "dl_cross_entropy": (_I, [_P, _P, _P, _P, _P, _Z, _I, _I, _P]),
    "dl_group_sum_bwd": (_I, [_P, _P, _I, _I, _I, _F, _P]),
    "dl_adam_step": (_I, [_P, _P, _P, _P, _P, _I, _F, _F, _F, _F, _F, _I, _I, _P]),
    "dl_grad_stabilize_workspace_bytes": (_Z, [ctypes.c_longlong, ctypes.c_longlong, _I]),
    "dl_grad_stabilize": (_I, [_P, _P, ctypes.c_longlong, ctypes.c_longlong, _I, _F, _I, _F, _P, _Z, _P]),
    "dl_profile_enable": (_I, [_I]),
    "dl_profile_read": (_I, [ctypes.c_char_p, _Z, ctypes.POINTER(_F), _I]),
}

_lib = None


def is_built():
    return os.path.exists(LIB_PATH)


def lib():
    """Load the shared library once; raises RuntimeError when it has not been built."""
    global _lib
    if _lib is None:
        if not is_built():
            raise RuntimeError(
                f"HIP extension not available: {LIB_PATH} is missing. Build it with "
                "`python -m difflut_amd.build` (needs hipcc); device tensors have no other path.")
        handle = ctypes.CDLL(LIB_PATH)
        for name, (res, args) in SIGNATURES.items():
            fn = getattr(handle, name)
            fn.restype, fn.argtypes = res, args
        _lib = handle
    return _lib


def check(code):
    if code != 0:
        raise RuntimeError(f"libdifflut_hip: {lib().dl_error_string(code).decode()} (code {code})")


def ptr(t):
    return None if t is None else t.data_ptr()


def stream():
    return torch.cuda.current_stream().cuda_stream


def require_device(*tensors):
    for t in tensors:
        if t is not None and not t.is_cuda:
            raise RuntimeError(
                "difflut_amd kernels run on ROCm devices only; got a tensor on "
                f"'{t.device}'. All tensors of one call must be on the same ROCm device (or all on the CPU).")


def profile_enable(on=True):
    lib().dl_profile_enable(1 if on else 0)


def profile_read(max_entries=64):
    """[(kernel name, milliseconds)] of the kernels launched since the last read (waits for them)."""
    names = ctypes.create_string_buffer(4096)
    ms = (_F * max_entries)()
    n = lib().dl_profile_read(names, 4096, ms, max_entries)
    labels = names.value.decode().split(";")[:n]
    return list(zip(labels, [ms[i] for i in range(n)]))
