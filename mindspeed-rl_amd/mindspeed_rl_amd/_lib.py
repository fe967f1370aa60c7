"""ctypes binding of libmrl_hip.so (the C ABI declared in include/mrl_hip.h).

The library is the only compute path of this package: if it is missing, loading raises - there
is no CPU or eager-torch fallback.  torch is used for device memory and streams only.
"""
import ctypes
import os

import torch

from . import _build

# enum mrl_dtype
F32, BF16, F16, I32, I64, U8, F64 = 0, 1, 2, 3, 4, 5, 6
# enum mrl_kl_penalty
KL_NONE, KL_KL, KL_ABS, KL_MSE, KL_LOW_VAR = 0, 1, 2, 3, 4
KL_BY_NAME = {"kl": KL_KL, "abs": KL_ABS, "mse": KL_MSE, "low_var_kl": KL_LOW_VAR}

_TORCH_DTYPE = {
    torch.float32: F32, torch.bfloat16: BF16, torch.float16: F16, torch.int32: I32,
    torch.int64: I64, torch.uint8: U8, torch.bool: U8, torch.float64: F64,
}

_vp = ctypes.c_void_p
_i64 = ctypes.c_int64
_int = ctypes.c_int
_f32 = ctypes.c_float

# name -> argtypes; the order is that of include/mrl_hip.h
SIGNATURES = {
    "mrl_version": [],
    "mrl_last_error": [],
    "mrl_vocab_logprob_fwd": [_vp, _int, _i64, _i64, _i64, _vp, _int, _vp, _f32, _vp, _vp, _vp, _vp],
    "mrl_vocab_logprob_bwd": [_vp, _int, _i64, _i64, _i64, _vp, _int, _f32, _vp, _vp, _vp, _vp, _vp, _int, _i64, _vp],
    "mrl_pack_index_build": [_vp, _int, _i64, _i64, _i64, _vp, _vp, _vp, _vp],
    "mrl_pack_rows": [_vp, _vp, _vp, _vp, _int, _i64, _i64, _vp, _vp, _i64, _vp, _vp],
    "mrl_unpad_gather": [_vp, _int, _i64, _i64, _vp, _vp, _vp, _int, _i64, _i64, _vp, _vp],
    "mrl_pad_scatter": [_vp, _i64, _i64, _vp, _vp, _vp, _int, _i64, _vp, _vp],
    "mrl_window_gather": [_vp, _int, _i64, _i64, _i64, _vp, _int, _i64, ctypes.c_uint64, _vp, _vp],
    "mrl_window_scatter": [_vp, _i64, _i64, _vp, _int, _i64, _vp, _vp],
    "mrl_generate_mask": [_vp, _int, _i64, _i64, _vp, _vp],
    "mrl_ragged_layout": [_vp, _int, _i64, _i64, _vp, _int, _i64, _int, _vp, _vp, _vp, _vp],
    "mrl_ragged_to_padded": [_vp, _int, _i64, _i64, _vp, _i64, _i64, ctypes.c_uint64, _vp, _vp],
    "mrl_padded_to_ragged": [_vp, _int, _i64, _i64, _vp, _int, _i64, _vp, _vp],
    "mrl_group_advantage": [_vp, _int, _i64, _i64, _vp, _int, _i64, _vp, _vp, _vp],
    "mrl_group_keep_mask": [_vp, _int, _i64, _i64, _vp, _vp],
    "mrl_policy_loss_fwd": [_vp, _vp, _vp, _vp, _vp, _vp, _int, _vp, _int, _i64, _i64, _f32, _f32, _int, _f32, _f32,
                            _int, _f32, _vp, _vp, _vp],
    "mrl_policy_loss_bwd": [_vp, _vp, _vp, _vp, _vp, _int, _vp, _int, _i64, _i64, _f32, _f32, _int, _f32, _f32, _int,
                            _f32, _vp, _vp, _vp, _vp, _vp, _vp],
    "mrl_fused_max_vocab": [_int],
    "mrl_fused_loss_prepare": [_int, _i64, _i64, _i64, _vp, _vp, _i64, _vp, _int, _vp, _int, _vp, _vp, _vp, _vp, _int,
                               _int, _vp, _vp, _vp, _vp, _vp, _i64, _vp, _f32, _vp, _vp],
    "mrl_fused_workspace_bytes": [_int, _i64, _i64],
    "mrl_fused_logprob_loss": [_vp, _int, _i64, _i64, _i64, _vp, _int, _f32, _vp, _int, _f32, _f32, _int, _f32, _f32,
                               _f32, _vp, _vp, _i64, _vp, _vp, _vp, _vp, _i64, _int, _vp],
    "mrl_set_wide_spin_limit": [_i64],
    "mrl_fused_loss_reduce": [_vp, _vp, _vp, _i64, _i64, _vp, _vp, _vp, _vp, _int, _vp, _int, _f32, _f32, _int, _f32,
                              _f32, _int, _f32, _vp, _vp, _vp, _vp, _vp],
    "mrl_scale_rows": [_vp, _int, _i64, _i64, _i64, _vp, _vp, _vp],
    "mrl_grad_scale_note": [_vp, _vp, _vp, _vp, _vp],
    "mrl_scale_rows_note": [_vp, _int, _i64, _i64, _i64, _vp, _vp, _vp, _vp, _vp],
    "mrl_lmhead_workspace_bytes": [_i64, _i64],
    "mrl_lmhead_logprob_fwd": [_vp, _vp, _i64, _i64, _i64, _vp, _int, _f32, _vp, _vp, _vp, _vp, _i64, _vp],
    "mrl_lmhead_logits": [_vp, _vp, _i64, _i64, _i64, _vp, _i64, _vp],
    "mrl_lmhead_logprob_bwd": [_vp, _vp, _vp, _i64, _i64, _i64, _i64, _vp, _vp, _vp],
    "mrl_lmhead_static_max_tokens": [],
    "mrl_lmhead_logprob_fwd_static": [_vp, _vp, _i64, _i64, _i64, _vp, _int, _f32, _vp, _vp, _vp, _vp],
    "mrl_group_standardize": [_vp, _int, _i64, _i64, ctypes.c_double, _vp, _vp],
    "mrl_first_match": [_vp, _int, _i64, _i64, _i64, _int, _vp, _vp],
    "mrl_kl_token_rewards": [_vp, _vp, _vp, _int, _vp, _i64, _i64, _int, _f32, _vp, _vp, _vp],
    "mrl_gae_scan": [_vp, _vp, _i64, _i64, _f32, _f32, _vp, _vp, _vp],
    "mrl_masked_whiten": [_vp, _vp, _int, _i64, _int, _vp, _vp, _vp],
    "mrl_value_loss_fwd": [_vp, _vp, _vp, _vp, _int, _vp, _int, _i64, _i64, _f32, _f32, _vp, _vp],
    "mrl_value_loss_bwd": [_vp, _vp, _vp, _vp, _int, _vp, _int, _i64, _i64, _f32, _f32, _vp, _vp, _vp, _vp],
    "mrl_copy_bytes": [_vp, _vp, _i64, _vp],
    "mrl_bandwidth_probe": [_int, _vp, _vp, _i64, _i64, _vp],
}
_RESTYPES = {"mrl_last_error": ctypes.c_char_p, "mrl_fused_workspace_bytes": ctypes.c_int64, "mrl_fused_max_vocab": ctypes.c_int64,
             "mrl_lmhead_workspace_bytes": ctypes.c_int64, "mrl_lmhead_static_max_tokens": ctypes.c_int64,
             "mrl_set_wide_spin_limit": ctypes.c_int64}

_lib = None


class MrlError(RuntimeError):
    """A libmrl_hip entry point returned a negative status."""

    def __init__(self, fn, code, message):
        super().__init__("%s failed (%d): %s" % (fn, code, message))
        self.code = code


def library_path():
    """The in-tree library; MRL_LIB_PATH points at another build of the same ABI (for experiments)."""
    return os.environ.get("MRL_LIB_PATH") or _build.LIB_PATH


def load():
    """Loads libmrl_hip.so once and declares every prototype.  Raises if it is not built."""
    global _lib
    if _lib is not None:
        return _lib
    path = library_path()
    if not os.path.exists(path):
        raise RuntimeError(
            "libmrl_hip.so is not built (%s missing): run `python -m mindspeed_rl_amd._build`; "
            "this package has no fallback path" % path)
    lib = ctypes.CDLL(path)
    for name, argtypes in SIGNATURES.items():
        fn = getattr(lib, name)       # AttributeError if the library lacks a declared symbol
        fn.argtypes = argtypes
        fn.restype = _RESTYPES.get(name, ctypes.c_int)
    _lib = lib
    return lib


def call(name, *args):
    """Calls an entry point; a negative status becomes MrlError (ValueError-like codes included)."""
    lib = load()
    rc = getattr(lib, name)(*args)
    if rc != 0:
        raise MrlError(name, rc, lib.mrl_last_error().decode("utf-8", "replace"))


def dtype_code(t):
    try:
        return _TORCH_DTYPE[t.dtype]
    except KeyError:
        raise TypeError("unsupported tensor dtype %s" % t.dtype) from None


def ptr(t):
    """Device pointer of a tensor (None -> NULL)."""
    return None if t is None else t.data_ptr()


def require_device(*tensors):
    """All given tensors (None skipped) must live on one HIP device; returns it."""
    dev = None
    for t in tensors:
        if t is None:
            continue
        if not t.is_cuda:
            raise RuntimeError("mindspeed_rl_amd runs on the GPU only: got a %s tensor (no CPU fallback exists)"
                               % t.device)
        if dev is None:
            dev = t.device
        elif t.device != dev:
            raise RuntimeError("tensors on different devices: %s and %s" % (dev, t.device))
    if dev is not None and dev.index is not None and dev.index != torch.cuda.current_device():
        # kernels are launched on the current device's context: one process drives one GPU here
        raise RuntimeError("tensors live on %s but the current device is cuda:%d (call torch.cuda.set_device first)"
                           % (dev, torch.cuda.current_device()))
    return dev


def stream(device):
    """Raw hipStream_t of torch's current stream on `device` (kernels are enqueued there)."""
    return torch.cuda.current_stream(device).cuda_stream
