"""ctypes binding of libspgt_hip.so (the C ABI declared in include/spgt_hip.h).

There is no fallback: if the library has not been built, or a call is made
with tensors that do not live on a GPU, an exception is raised.
"""
import ctypes
import os
import threading

import torch

PKG_DIR = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(PKG_DIR, "libspgt_hip.so")

_c_float_p = ctypes.c_void_p  # device pointers travel as integers
_i = ctypes.c_int
_i64 = ctypes.c_int64
_sz = ctypes.c_size_t
_f = ctypes.c_float
_p = ctypes.c_void_p

# name -> (restype, argtypes); must list every function of include/spgt_hip.h
SIGNATURES = {
    "spgt_version": (_i, []),
    "spgt_last_error": (ctypes.c_char_p, []),
    "spgt_multihead_projection_with_position_rrc_forward": (_i, [_p, _p, _p, _p, _p, _i, _i, _i, _i, _i, _i, _p]),
    "spgt_multihead_projection_layernorm_with_position_rrc_forward": (
        _i, [_p, _p, _p, _p, _p, _f, _p, _p, _p, _i, _i, _i, _i, _i, _i, _p]),
    "spgt_galerkin_attention_cccr_workspace_bytes": (_sz, [_i, _i, _i, _i]),
    "spgt_galerkin_attention_cccr_forward": (_i, [_p, _p, _p, _p, _p, _sz, _i, _i, _i, _i, _p]),
    "spgt_batched_skinny_gemm_workspace_bytes": (_sz, [_i, _i, _i, _i]),
    "spgt_batched_skinny_gemm": (_i, [_p, _p, _p, _f, _i, _i, _i, _i64, _i64, _i64, _i, _i, _p, _sz, _p]),
    "spgt_batched_small_k_gemm": (_i, [_p, _p, _p, _f, _i, _i, _i, _i64, _i64, _i64, _i, _i, _p]),
    "spgt_galerkin_attention_fused_workspace_bytes": (_sz, [_i, _i, _i, _i]),
    "spgt_galerkin_attention_fused_forward": (
        _i, [_p, _p, _p, _i64, _p, _p, _p, _p, _p, _f, _p, _p, _p, _sz, _i, _i, _i, _i, _p]),
    "spgt_galerkin_attention_fused_backward_workspace_bytes": (_sz, [_i, _i, _i, _i]),
    "spgt_galerkin_attention_fused_backward": (
        _i, [_p, _p, _p, _p, _i64, _p, _p, _p, _p, _p, _f, _p, _p, _p, _p, _i64, _p, _p, _sz, _i, _i, _i, _i, _p]),
    "spgt_galerkin_attention_fused_static_max_bytes": (_sz, []),
    "spgt_galerkin_attention_fused_forward_static": (
        _i, [_p, _p, _p, _i64, _p, _p, _p, _p, _p, _f, _p, _p, _i, _i, _i, _i, _p]),
    "spgt_galerkin_attention_cccr_backward_workspace_bytes": (_sz, [_i, _i, _i, _i]),
    "spgt_galerkin_attention_cccr_backward": (_i, [_p, _p, _p, _p, _p, _p, _p, _p, _sz, _i, _i, _i, _i, _p]),
    "spgt_heads_feature_to_token_major": (_i, [_p, _p, _i, _i, _i, _i, _i, _p]),
    "spgt_layernorm_heads_backward_workspace_bytes": (_sz, [_i64, _i]),
    "spgt_layernorm_heads_backward": (_i, [_p, _p, _p, _f, _p, _p, _p, _p, _sz, _i64, _i, _p]),
    "spgt_batched_transpose": (_i, [_p, _p, _i, _i, _i, _p]),
    "spgt_transpose_gather_dual": (_i, [_p, _p, _p, _i, _i, _i, _i, _i, _i, _i, _i, _i, _p]),
    "spgt_transpose_scatter_dual": (_i, [_p, _p, _p, _i, _i, _i, _i, _i, _i, _i, _i, _i, _p]),
    "spgt_spectral_mode_contract": (_i, [_p, _p, _p, _p, _i, _i, _i, _i, _i, _i, _i, _i, _i, _i, _i, _p]),
    "spgt_spectral_modes_compact": (_i, [_p, _p, _p, _p, _i, _i, _i, _i, _i, _p]),
    "spgt_bilinear_align_corners": (_i, [_p, _p, _i, _i, _i, _i, _i, _p]),
    "spgt_bilinear_align_corners_nhwc": (_i, [_p, _p, _i, _i, _i, _i, _i, _i, _p]),
    "spgt_bilinear_resample": (_i, [_p, _p, _p, _i, _i, _i, _i, _i, _i, _i, _i, _i, _i, _i, _p]),
    "spgt_bilinear_nhwc_affine": (_i, [_p, _p, _i, _i, _i, _i, _i, _i, _p, _p, _i, _p]),
    "spgt_bilinear_adjoint": (_i, [_p, _p, _i, _i, _i, _i, _i, _i, _i, _p]),
    "spgt_upsample_conv3x3_gather": (_i, [_p, _p, _p, _i, _i, _i, _i, _i, _i, _i, _i, _p]),
    "spgt_upsample_conv3x3_gather_adjoint": (_i, [_p, _p, _i, _i, _i, _i, _i, _i, _p]),
    "spgt_bilinear_resample_concat": (_i, [_p, _p, _p, _p, _i, _p, _i, _i, _i, _i, _i, _i, _i, _i, _p]),
    "spgt_bilinear_resample_concat_dropout": (
        _i, [_p, _p, _p, _p, _i, _p, _i, _i, _i, _i, _i, _i, _i, _i, _p, _f, _p]),
    "spgt_bias_activation_nchw": (_i, [_p, _p, _i, _i, _i64, _i, _i, _p]),
    "spgt_bias_activation_nchw_dropout": (_i, [_p, _p, _i, _i, _i64, _i, _i, _p, _f, _p]),
    "spgt_denormalize_boundary": (_i, [_p, _p, _p, _i, _p, _i, _i, _i, _i, _i, _p]),
    "spgt_spectral_inverse_linear_supported": (_i, [_i, _i, _i, _i]),
    "spgt_spectral_inverse_linear": (_i, [_p, _p, _p, _p, _p, _i, _p, _i64, _i, _i, _i, _i, _p]),
    "spgt_truncated_dft_rows_supported": (_i, [_i, _i, _i]),
    "spgt_truncated_dft_rows_forward": (_i, [_p, _p, _p, _i64, _i, _i, _i, _i, _p]),
    "spgt_truncated_dft_rows_inverse": (_i, [_p, _p, _p, _i64, _i, _i, _i, _i, _p]),
    "spgt_spectral_modes_middle_supported": (_i, [_i, _i, _i, _i]),
    "spgt_spectral_modes_middle_workspace_bytes": (_sz, [_i, _i, _i]),
    "spgt_spectral_modes_middle": (_i, [_p, _p, _p, _p, _p, _p, _p, _sz, _i, _i, _i, _i, _i, _p]),
    "spgt_conv3x3_resample_supported": (_i, [_i]),
    "spgt_conv3x3_resample": (_i, [_p, _p, _p, _p, _i, _i, _i, _i, _i, _i, _i, _i, _i, _p]),
    "spgt_conv3x3_resample_dropout": (_i, [_p, _p, _p, _p, _i, _i, _i, _i, _i, _i, _i, _i, _i, _p, _f, _p]),
    "spgt_conv3x3_resample_backward_workspace_bytes": (_sz, [_i, _i, _i, _i, _i]),
    "spgt_conv3x3_resample_backward": (
        _i, [_p, _p, _p, _p, _p, _p, _sz, _i, _i, _i, _i, _i, _i, _i, _i, _p, _f, _p]),
    "spgt_linear_supported": (_i, [_i, _i]),
    "spgt_linear_forward": (_i, [_p, _i64, _p, _p, _p, _i64, _i, _i, _p, _i64, _p, _i, _p, _i64, _i, _i64, _i64, _i, _i,
                                 _p]),
    "spgt_ffn_scalar_supported": (_i, [_i, _i]),
    "spgt_ffn_scalar_forward": (_i, [_p, _i64, _p, _p, _p, _p, _i, _p, _i64, _i, _i, _p]),
    "spgt_encoder_tail_supported": (_i, [_i, _i, _i]),
    "spgt_encoder_tail_forward": (_i, [_p, _i64, _p, _p, _p, _p, _p, _p, _p, _i, _p, _i64, _i, _i, _i, _p]),
    "spgt_encoder_tail_forward_dropout": (
        _i, [_p, _i64, _p, _p, _p, _p, _p, _p, _p, _i, _p, _i64, _i, _i, _i, _p, _f, _f, _p]),
    "spgt_galerkin_attention_ktv_forward": (
        _i, [_p, _p, _i64, _p, _p, _p, _p, _p, _f, _p, _p, _sz, _i, _i, _i, _i, _p]),
    "spgt_fold_ktv_into_fc": (_i, [_p, _p, _p, _p, _i, _i, _i, _i, _p]),
    "spgt_encoder_tail_folded_forward": (
        _i, [_p, _i64, _p, _p, _p, _p, _p, _p, _p, _p, _p, _i, _p, _i, _i64, _i, _i, _i, _p]),
    "spgt_encoder_tail_folded_forward_dropout": (
        _i, [_p, _i64, _p, _p, _p, _p, _p, _p, _p, _p, _p, _i, _p, _i, _i64, _i, _i, _i, _p, _f, _f, _p]),
    "spgt_strided_copy_batch": (_i, [_p, _i, _p]),
    "spgt_linear_weight_grad_workspace_bytes": (_sz, [_i64, _i, _i, _i]),
    "spgt_linear_weight_grad": (_i, [_p, _i64, _i64, _p, _i64, _i64, _p, _p, _sz, _i64, _i, _i, _i, _p]),
    "spgt_dropout_add": (_i, [_p, _p, _p, _i64, _i, _p, _f, _i, _p]),
    "spgt_galerkin_attention_fused_profile": (
        _i, [_p, _p, _p, _p, _i, _i64, _p, _p, _p, _p, _p, _f, _p, _p, _sz, _i, _i, _i, _i, _p, _i,
             ctypes.POINTER(ctypes.c_float)]),
}



class CopyDesc(ctypes.Structure):
    """spgt_copy_desc of include/spgt_hip.h."""
    _fields_ = [("src", ctypes.c_void_p), ("dst", ctypes.c_void_p), ("size", ctypes.c_int32 * 3),
                ("src_stride", ctypes.c_int32 * 3), ("dst_stride", ctypes.c_int32 * 3)]


_lock = threading.Lock()
_lib = None


class SpgtError(RuntimeError):
    """A libspgt_hip.so entry point rejected its arguments or failed to launch."""


def load():
    """Returns the loaded library, loading it on first use."""
    global _lib
    if _lib is not None:
        return _lib
    with _lock:
        if _lib is None:
            if not os.path.exists(LIB_PATH):
                raise SpgtError(
                    f"{LIB_PATH} is missing: build it with `python -m spgt_amd.build` "
                    "(there is no non-HIP implementation of these operators)")
            lib = ctypes.CDLL(LIB_PATH)
            for name, (restype, argtypes) in SIGNATURES.items():
                fn = getattr(lib, name)
                fn.restype = restype
                fn.argtypes = argtypes
            _lib = lib
    return _lib


def open_library(path: str):
    """A handle to a build of the library at `path` with every entry point's signature set; not cached and not
    used by the operators (tests compare builds with it)."""
    lib = ctypes.CDLL(path)
    for name, (restype, argtypes) in SIGNATURES.items():
        fn = getattr(lib, name)
        fn.restype = restype
        fn.argtypes = argtypes
    return lib


def last_error() -> str:
    return load().spgt_last_error().decode("utf-8", "replace")


def check(rc: int) -> None:
    if rc != 0:
        raise SpgtError(f"libspgt_hip error {rc}: {last_error()}")


def require_gpu_f32(name: str, t: torch.Tensor, dtype=torch.float32, contiguous: bool = True) -> None:
    if not isinstance(t, torch.Tensor):
        raise TypeError(f"{name} must be a torch.Tensor")
    if not t.is_cuda:
        raise SpgtError(f"{name} must live on a GPU (got device {t.device}); there is no CPU implementation")
    if t.dtype != dtype:
        raise TypeError(f"{name} must have dtype {dtype} (got {t.dtype})")
    if contiguous and not t.is_contiguous():
        raise ValueError(f"{name} must be contiguous")


def ptr(t: torch.Tensor):
    return ctypes.c_void_p(t.data_ptr())


def stream_of(t: torch.Tensor):
    """torch's current stream on t's device, as the raw handle the C ABI takes."""
    index = t.device.index
    return ctypes.c_void_p(torch._C._cuda_getCurrentRawStream(torch.cuda.current_device() if index is None else index))


class _NoGuard:
    def __enter__(self):
        return None

    def __exit__(self, *exc):
        return False


_NO_GUARD = _NoGuard()


def device_guard(device):
    """`with device_guard(t.device):` makes t's device current for the launch inside, like torch.cuda.device, and
    costs nothing when it is current already."""
    index = device.index
    if index is None or index == torch.cuda.current_device():
        return _NO_GUARD
    return torch.cuda.device(device)


def workspace(nbytes: int, like: torch.Tensor) -> torch.Tensor:
    """Scratch from torch's caching allocator on `like`'s device (at least 16 bytes)."""
    return torch.empty(max(int(nbytes), 16), dtype=torch.uint8, device=like.device)


_seed_tls = threading.local()
_SEED_POOL_WORDS = 128


class seed_scope:
    """Within this context (one model forward), dropout_seed hands out consecutive word pairs of one drawn
    pool instead of launching a generator kernel per call.  The pool never outlives the context: a forward
    captured into a graph draws its pool inside the capture, so every replay gets new words."""

    def __enter__(self):
        self.outer = getattr(_seed_tls, "pool", None), getattr(_seed_tls, "used", 0), getattr(_seed_tls, "on", False)
        _seed_tls.pool, _seed_tls.used, _seed_tls.on = None, 0, True
        return self

    def __exit__(self, *exc):
        _seed_tls.pool, _seed_tls.used, _seed_tls.on = self.outer
        return False


def dropout_seed(device):
    """Two 32-bit words from torch's generator of `device`, in device memory, for the kernels that apply dropout
    themselves.  Drawn by a generator kernel: torch.manual_seed governs it, and inside a captured graph every
    replay draws new words.  Every call gives a different pair."""
    if not getattr(_seed_tls, "on", False):
        return torch.randint(0, 2 ** 31 - 1, (2,), dtype=torch.int32, device=device)
    device = torch.device(device)
    pool, used = _seed_tls.pool, _seed_tls.used
    if pool is None or pool.device != device or used + 2 > pool.numel():
        pool, used = torch.randint(0, 2 ** 31 - 1, (_SEED_POOL_WORDS,), dtype=torch.int32, device=device), 0
        _seed_tls.pool = pool
    _seed_tls.used = used + 2
    return pool[used:used + 2]