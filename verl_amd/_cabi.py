"""ctypes binding of ``libverl_amd.so`` (declared in ``include/verl_amd.h``).

The library is loaded lazily, after ``import torch``, so that it binds to the HIP runtime torch
has already mapped (same ``libamdhip64.so.7`` soname) and torch's streams are valid in it.
"""
from __future__ import annotations

import ctypes
import os
import threading
from ctypes import c_char_p, c_double, c_float, c_int, c_int64, c_size_t, c_uint64, c_void_p

import torch

_LIB_PATH = os.path.join(os.path.dirname(os.path.abspath(__file__)), "lib", "libverl_amd.so")
_lock = threading.Lock()
_lib = None

MASK_F32, MASK_I64, MASK_U8, MASK_I32 = 0, 1, 2, 3
# d_weight_mode of vamd_lce_backward (VAMD_DW_*)
DW_STORE, DW_ADD_BF16, DW_F32_STORE, DW_F32_ADD, DW_F32_ADD_FINISH, DW_NONE = 0, 1, 2, 3, 4, 5
LCE_TIMING_KERNELS = 5
AGG_MODES = {
    "token-mean": 0,
    "seq-mean-token-sum": 1,
    "seq-mean-token-mean": 2,
    "seq-mean-token-sum-norm": 3,
}

# name -> (restype, argtypes); one entry per symbol of include/verl_amd.h
SIGNATURES = {
    "vamd_abi_version": (c_int, []),
    "vamd_last_error": (c_char_p, []),
    "vamd_set_waiting_kernels": (None, [c_int]),
    "vamd_waiting_kernels_enabled": (c_int, []),
    "vamd_copy_bytes": (c_int, [c_void_p, c_void_p, c_int64, c_void_p]),
    "vamd_sum4": (c_int, [c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_int64, c_void_p]),
    "vamd_mfma_yardstick_flops": (c_int64, [c_int, c_int, c_int]),
    "vamd_mfma_yardstick": (c_int, [c_int, c_void_p, c_void_p, c_int, c_int, c_void_p]),
    "vamd_lce_forward_workspace_bytes": (c_size_t, [c_int64, c_int64, c_int64]),
    "vamd_lce_forward": (c_int, [c_void_p, c_void_p, c_void_p, c_int64, c_int64, c_int64, c_float, c_void_p,
                                 c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_size_t, c_void_p]),
    "vamd_lce_forward_static": (c_int, [c_void_p, c_void_p, c_void_p, c_int64, c_int64, c_int64, c_float, c_void_p,
                                        c_void_p, c_void_p, c_void_p, c_void_p, c_void_p]),
    "vamd_lce_backward_workspace_bytes": (c_size_t, [c_int64, c_int64, c_int64, c_int64]),
    "vamd_lce_backward": (c_int, [c_void_p, c_void_p, c_void_p, c_int64, c_int64, c_int64, c_float, c_void_p,
                                  c_void_p, c_void_p, c_void_p, c_float, c_void_p, c_void_p, c_void_p, c_int, c_void_p,
                                  c_int64, c_void_p, c_size_t, c_void_p]),
    "vamd_lce_timing_enable": (c_int, [c_int]),
    "vamd_lce_timing_collect": (c_int, [c_void_p, c_void_p]),
    "vamd_row_softmax_stats": (c_int, [c_void_p, c_int, c_int64, c_int64, c_int64, c_void_p, c_void_p, c_void_p,
                                       c_void_p, c_void_p, c_void_p]),
    "vamd_row_softmax_backward": (c_int, [c_void_p, c_int, c_int64, c_int64, c_int64, c_void_p, c_void_p, c_void_p,
                                          c_void_p, c_void_p, c_void_p, c_int64, c_void_p]),
    "vamd_clip_by_value": (c_int, [c_void_p, c_void_p, c_void_p, c_int64, c_void_p, c_void_p]),
    "vamd_clip_by_value_backward": (c_int, [c_void_p, c_void_p, c_void_p, c_void_p, c_int64, c_void_p, c_void_p,
                                            c_void_p, c_void_p]),
    "vamd_masked_reduce": (c_int, [c_void_p, c_void_p, c_int, c_int64, c_int64, c_int, c_void_p, c_void_p, c_void_p,
                                   c_void_p, c_void_p, c_int, c_void_p, c_size_t, c_void_p]),
    "vamd_masked_moments_workspace_bytes": (c_size_t, [c_int64, c_int64]),
    "vamd_masked_moments": (c_int, [c_void_p, c_void_p, c_int, c_int64, c_int64, c_int, c_void_p, c_void_p,
                                    c_size_t, c_void_p]),
    "vamd_whiten_stats": (c_int, [c_void_p, c_int, c_void_p, c_void_p]),
    "vamd_affine_by_stats": (c_int, [c_void_p, c_void_p, c_int64, c_void_p, c_void_p]),
    "vamd_gae_workspace_bytes": (c_size_t, [c_int64, c_int64]),
    "vamd_gae": (c_int, [c_void_p, c_void_p, c_void_p, c_int, c_int64, c_int64, c_float, c_float, c_int, c_void_p,
                         c_void_p, c_void_p, c_void_p, c_size_t, c_void_p]),
    "vamd_grpo_workspace_bytes": (c_size_t, [c_int64, c_int64, c_int64]),
    "vamd_grpo_advantage": (c_int, [c_void_p, c_void_p, c_int, c_void_p, c_int64, c_int64, c_int64, c_float, c_int,
                                    c_int, c_void_p, c_void_p, c_void_p, c_size_t, c_void_p]),
    "vamd_group_outcome_advantage_workspace_bytes": (c_size_t, [c_int64, c_int64, c_int64]),
    "vamd_group_outcome_advantage": (c_int, [c_void_p, c_void_p, c_int, c_void_p, c_int64, c_int64, c_int64, c_int,
                                             c_float, c_int, c_int, c_float, c_void_p, c_void_p, c_void_p, c_size_t,
                                             c_void_p]),
    "vamd_returns_advantage_workspace_bytes": (c_size_t, [c_int64, c_int64]),
    "vamd_returns_advantage": (c_int, [c_void_p, c_void_p, c_int, c_void_p, c_int64, c_int64, c_float, c_int,
                                       c_void_p, c_void_p, c_void_p, c_void_p, c_size_t, c_void_p]),
    "vamd_apply_kl_penalty_workspace_bytes": (c_size_t, [c_int64, c_int64]),
    "vamd_apply_kl_penalty": (c_int, [c_void_p, c_void_p, c_void_p, c_void_p, c_int, c_int64, c_int64, c_int, c_float,
                                      c_void_p, c_void_p, c_void_p, c_size_t, c_void_p]),
    "vamd_data_metrics_workspace_bytes": (c_size_t, [c_int64, c_int64]),
    "vamd_data_metrics": (c_int, [c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_int, c_void_p, c_int,
                                  c_int64, c_int64, c_int64, c_void_p, c_void_p, c_size_t, c_void_p]),
    "vamd_rollout_correction_workspace_bytes": (c_size_t, [c_int64, c_int64]),
    "vamd_rollout_correction": (c_int, [c_void_p, c_void_p, c_void_p, c_int, c_int64, c_int64, c_int, c_float, c_int,
                                        c_void_p, c_void_p, c_void_p, c_size_t, c_void_p]),
    "vamd_response_window_scatter": (c_int, [c_void_p, c_void_p, c_void_p, c_void_p, c_int64, c_int64, c_int64,
                                             c_int64, c_void_p, c_void_p, c_void_p, c_void_p]),
    "vamd_response_window_gather": (c_int, [c_void_p, c_void_p, c_void_p, c_int64, c_int64, c_int64, c_int64,
                                            c_void_p, c_void_p, c_void_p]),
    "vamd_policy_loss_cov_workspace_bytes": (c_size_t, [c_int64, c_int64]),
    "vamd_policy_loss_cov_forward": (c_int, [c_int, c_void_p, c_void_p, c_void_p, c_void_p, c_int, c_void_p, c_int64,
                                             c_int64, c_float, c_float, c_float, c_float, c_double, c_float, c_uint64,
                                             c_int, c_double, c_double, c_double, c_double, c_void_p, c_void_p,
                                             c_void_p, c_void_p, c_void_p, c_size_t, c_void_p]),
    "vamd_variance_proxy_rows": (c_int, [c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_int, c_int64, c_int64,
                                         c_void_p, c_void_p]),
    "vamd_rollout_rs_chunks": (c_int64, [c_int64]),
    "vamd_rollout_rs_row_stats": (c_int, [c_void_p, c_void_p, c_void_p, c_int, c_int64, c_int64, c_void_p, c_void_p]),
    "vamd_rollout_rs_apply": (c_int, [c_void_p, c_void_p, c_void_p, c_int, c_int64, c_int64, c_void_p, c_int,
                                      c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p]),
    "vamd_otb_advantage_workspace_bytes": (c_size_t, [c_int64, c_int64, c_int]),
    "vamd_otb_advantage": (c_int, [c_void_p, c_void_p, c_int, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p,
                                   c_void_p, c_int64, c_int64, c_int64, c_int, c_float, c_void_p, c_void_p, c_void_p,
                                   c_size_t, c_void_p]),
    "vamd_affine_by_stats_masked": (c_int, [c_void_p, c_void_p, c_void_p, c_int, c_int64, c_void_p, c_void_p]),
    "vamd_group_mean_std": (c_int, [c_void_p, c_void_p, c_int64, c_int64, c_float, c_void_p, c_void_p, c_void_p,
                                    c_void_p]),
    "vamd_agg_loss_workspace_bytes": (c_size_t, [c_int64, c_int64]),
    "vamd_agg_loss_forward": (c_int, [c_void_p, c_void_p, c_int, c_int64, c_int64, c_int, c_double, c_double,
                                      c_double, c_double, c_void_p, c_void_p, c_void_p, c_size_t, c_void_p]),
    "vamd_agg_loss_backward": (c_int, [c_void_p, c_void_p, c_void_p, c_int, c_int64, c_int64, c_void_p, c_void_p]),
    "vamd_policy_loss_workspace_bytes": (c_size_t, [c_int64, c_int64]),
    "vamd_policy_loss_forward": (c_int, [c_void_p, c_void_p, c_void_p, c_void_p, c_int, c_void_p, c_int64, c_int64,
                                         c_float, c_float, c_float, c_int, c_double, c_double, c_double, c_double,
                                         c_void_p, c_void_p, c_void_p, c_void_p, c_size_t, c_void_p]),
    "vamd_policy_loss_variant_workspace_bytes": (c_size_t, [c_int64, c_int64]),
    "vamd_policy_loss_variant_forward": (c_int, [c_int, c_void_p, c_void_p, c_void_p, c_void_p, c_int, c_void_p, c_int64,
                                                 c_int64, c_float, c_float, c_float, c_float, c_float, c_int,
                                                 c_double, c_double, c_double, c_double, c_void_p, c_void_p,
                                                 c_void_p, c_void_p, c_size_t, c_void_p]),
    "vamd_scale_rows": (c_int, [c_void_p, c_void_p, c_void_p, c_float, c_int64, c_int64, c_void_p, c_void_p]),
    "vamd_kl_penalty": (c_int, [c_void_p, c_void_p, c_int64, c_int, c_int, c_void_p, c_void_p, c_void_p]),
    "vamd_kl_loss_workspace_bytes": (c_size_t, [c_int64, c_int64]),
    "vamd_kl_loss_forward": (c_int, [c_void_p, c_void_p, c_void_p, c_int, c_int64, c_int64, c_int, c_int, c_int,
                                     c_double, c_double, c_double, c_double, c_void_p, c_void_p, c_void_p, c_void_p,
                                     c_size_t, c_void_p]),
    "vamd_value_loss_workspace_bytes": (c_size_t, [c_int64, c_int64]),
    "vamd_value_loss_forward": (c_int, [c_void_p, c_void_p, c_void_p, c_void_p, c_int, c_int64, c_int64, c_float,
                                        c_int, c_void_p, c_void_p, c_void_p, c_void_p, c_size_t, c_void_p]),
}


def lib_path() -> str:
    return _LIB_PATH


ABI_VERSION = 5  # VAMD_ABI_VERSION of include/verl_amd.h


def load_library(path: str | None = None) -> ctypes.CDLL:
    """dlopen the library and attach prototypes.  Raises if it has not been built."""
    path = path or _LIB_PATH
    if not os.path.exists(path):
        raise RuntimeError(
            f"{path} is missing: build it with `python -m verl_amd.csrc.build` (hipcc, gfx950). "
            "verl_amd has no CPU fallback."
        )
    lib = ctypes.CDLL(path)
    for name, (res, args) in SIGNATURES.items():
        fn = getattr(lib, name)  # AttributeError names the missing symbol
        fn.restype = res
        fn.argtypes = args
    if lib.vamd_abi_version() != ABI_VERSION:
        raise RuntimeError(f"{path} reports ABI version {lib.vamd_abi_version()}, these bindings are written for "
                           f"{ABI_VERSION}: rebuild it with `python -m verl_amd.csrc.build`")
    return lib


def lib() -> ctypes.CDLL:
    global _lib
    if _lib is None:
        with _lock:
            if _lib is None:
                _lib = load_library()
    return _lib


def check(rc: int) -> None:
    if rc != 0:
        msg = lib().vamd_last_error().decode("utf-8", "replace")
        raise RuntimeError(f"libverl_amd error {rc}: {msg}")


def compute_device(*tensors: torch.Tensor) -> torch.device:
    """Device the kernels will run on: the tensors' GPU, or the current GPU for CPU inputs."""
    for t in tensors:
        if t is not None and t.is_cuda:
            return t.device
    if not torch.cuda.is_available():
        raise RuntimeError("verl_amd needs a ROCm GPU: no device is visible and there is no CPU fallback")
    return torch.device("cuda", torch.cuda.current_device())


def stream_ptr(device: torch.device) -> int:
    """hipStream_t of torch's current stream on `device`, as an integer (one C call, no Stream object)."""
    index = device.index
    if index is None:
        index = torch.cuda.current_device()
    return torch._C._cuda_getCurrentRawStream(index)


class _NoGuard:
    def __enter__(self):
        return None

    def __exit__(self, *exc):
        return False


_NO_GUARD = _NoGuard()


def device_guard(device: torch.device):
    """Context that makes `device` current for the library call inside it; free when it already is."""
    if device.index is None or device.index == torch._C._cuda_getDevice():
        return _NO_GUARD
    return torch.cuda.device(device)


def ptr(t: torch.Tensor | None):
    return None if t is None else t.data_ptr()


def workspace(nbytes: int, device: torch.device) -> torch.Tensor:
    """Uninitialised scratch for the head kernels."""
    return torch.empty(max(int(nbytes), 256), dtype=torch.uint8, device=device)


_ticket_ws: dict[tuple[int, int], torch.Tensor] = {}


def ticket_workspace(nbytes: int, device: torch.device) -> torch.Tensor:
    """Scratch for the single-launch reductions.  Their contract: the first VAMD_TICKET_BYTES (arrival
    counters) are zero on entry and zero again on exit, so one zero-initialised buffer per
    (device, stream) is kept and reused; kernels on one stream run in order and never share it."""
    key = (device.index if device.index is not None else torch.cuda.current_device(), stream_ptr(device))
    need = max(int(nbytes), 4096)
    with _lock:
        buf = _ticket_ws.get(key)
        if buf is None or buf.numel() < need:
            buf = torch.zeros(max(need, 1 << 20), dtype=torch.uint8, device=device)
            _ticket_ws[key] = buf
    return buf


GAVE_UP_OFFSET = 136  # VAMD_TICKET_GAVE_UP_OFFSET


def waiting_gave_up(ticket_ws: torch.Tensor) -> int:
    """How many workgroups have given up a bounded wait on this counter buffer since it was zeroed (waits for the
    stream: it reads four bytes back)."""
    return int(ticket_ws[GAVE_UP_OFFSET:GAVE_UP_OFFSET + 4].view(torch.int32).item())


def mask_code(mask: torch.Tensor) -> tuple[torch.Tensor, int]:
    """Contiguous mask in one of the element types the kernels read, with its VAMD_MASK_* code."""
    dt = mask.dtype
    if dt is torch.float32:
        code = MASK_F32
    elif dt is torch.int64:
        code = MASK_I64
    elif dt is torch.bool or dt is torch.uint8:
        code = MASK_U8
    elif dt is torch.int32:
        code = MASK_I32
    else:  # fp16 / bf16 / fp64 / int8 / int16: exact in fp32 for 0/1 masks
        mask = mask.to(torch.float32)
        code = MASK_F32
    return (mask if mask.is_contiguous() else mask.contiguous()), code


def as_f32(t: torch.Tensor, device: torch.device) -> torch.Tensor:
    """fp32, contiguous, on `device`, detached (the tensor itself when it already is all that: the kernels only
    take its address)."""
    if t.dtype is torch.float32 and t.device == device and t.is_contiguous():
        return t.detach() if t.requires_grad else t
    return t.detach().to(device=device, dtype=torch.float32).contiguous()


def on_device(t: torch.Tensor, device: torch.device) -> torch.Tensor:
    """`t` detached on `device` (itself when it already is)."""
    if t.device == device:
        return t.detach() if t.requires_grad else t
    return t.detach().to(device)
