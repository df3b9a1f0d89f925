"""Operator API of the FNO data-movement path, backed by libspgt_hip.so.

Same function names, argument order and result layouts as the reference's
extension/bind/datamove.py:68-87 (python surface) and
extension/bind/datamove.cu:66-70 (the `dexts` module surface), plus the
operators the reference leaves to library calls: the fused spectral-mode
contraction, the truncated-DFT stages, bilinear resampling (with its backward)
and the scalers' fused forms.  Tensors must be contiguous and on a GPU.
"""
import ctypes
from math import prod
from types import SimpleNamespace
from typing import Any, List, Tuple

import torch
from torch import Tensor

from ... import _lib
from ..._lib import check, dropout_seed, ptr, require_gpu_f32, stream_of, workspace


# --------------------------------------------------------------------------- #
# `dexts` surface: plain functions on tensors, no autograd
# --------------------------------------------------------------------------- #

def _batched_transpose(src: Tensor, batch_list: List[int], M_list: List[int], N_list: List[int]) -> Tensor:
    """src viewed as [prod(batch), prod(M), prod(N)] -> shape batch_list + N_list + M_list
    (reference: extension/bind/datamove.cu:8-23)."""
    require_gpu_f32("src", src)
    b, M, N = prod(batch_list), prod(M_list), prod(N_list)
    if src.numel() != b * M * N:
        raise ValueError(f"src has {src.numel()} elements, the lists describe {b}x{M}x{N}")
    out = torch.empty(list(batch_list) + list(N_list) + list(M_list), dtype=src.dtype, device=src.device)
    if src.numel() == 0:
        return out
    with _lib.device_guard(src.device):
        check(_lib.load().spgt_batched_transpose(ptr(src), ptr(out), b, M, N, stream_of(src)))
    return out


def _transpose_gather_dual(src: Tensor, dim_list: List[int], H_all: int, W_all: int, H_low: int, W_low: int,
                           H_base_1: int, W_base_1: int, H_base_2: int, W_base_2: int) -> Tuple[Tensor, Tensor]:
    """src complex64 [*dim_list, H_all, W_all] -> two [H_low, W_low, *dim_list] windows
    (reference: extension/bind/datamove.cu:25-44)."""
    require_gpu_f32("src", src, torch.complex64)
    dim = prod(dim_list)
    if src.numel() != dim * H_all * W_all:
        raise ValueError(f"src has {src.numel()} elements, expected {dim}x{H_all}x{W_all}")
    shape = [H_low, W_low] + list(dim_list)
    out1 = torch.empty(shape, dtype=src.dtype, device=src.device)
    out2 = torch.empty(shape, dtype=src.dtype, device=src.device)
    with _lib.device_guard(src.device):
        check(_lib.load().spgt_transpose_gather_dual(
            ptr(src), ptr(out1), ptr(out2), dim, H_all, W_all, H_low, W_low, H_base_1, W_base_1, H_base_2, W_base_2,
            stream_of(src)))
    return out1, out2


def _transpose_scatter_dual(src1: Tensor, src2: Tensor, dim_list: List[int], H_all: int, W_all: int, H_low: int,
                            W_low: int, H_base_1: int, W_base_1: int, H_base_2: int, W_base_2: int) -> Tensor:
    """Inverse of the gather into a zero-filled complex64 [*dim_list, H_all, W_all]
    (reference: extension/bind/datamove.cu:46-64)."""
    require_gpu_f32("src1", src1, torch.complex64)
    require_gpu_f32("src2", src2, torch.complex64)
    dim = prod(dim_list)
    for name, t in (("src1", src1), ("src2", src2)):
        if t.numel() != H_low * W_low * dim:
            raise ValueError(f"{name} has {t.numel()} elements, expected {H_low}x{W_low}x{dim}")
    out = torch.empty(list(dim_list) + [H_all, W_all], dtype=src1.dtype, device=src1.device)
    with _lib.device_guard(src1.device):
        check(_lib.load().spgt_transpose_scatter_dual(
            ptr(src1), ptr(src2), ptr(out), dim, H_all, W_all, H_low, W_low, H_base_1, W_base_1, H_base_2, W_base_2,
            stream_of(src1)))
    return out


def _spectral_mode_contract(X_ft: Tensor, weight_1: Tensor, weight_2: Tensor, H_low: int, W_low: int, H_base_1: int,
                            W_base_1: int, H_base_2: int, W_base_2: int) -> Tensor:
    """X_ft complex64 [N, Cin, H_all, W_all]; weight_k fp32 [H_low, W_low, Cin, Cout, 2] (or complex64
    [H_low, W_low, Cin, Cout]) -> complex64 [N, Cout, H_all, W_all], zero outside the two windows."""
    require_gpu_f32("X_ft", X_ft, torch.complex64)
    if X_ft.dim() != 4:
        raise ValueError("X_ft must be [N, Cin, H_all, W_all]")
    N, Cin, H_all, W_all = X_ft.shape
    ws = []
    for name, w in (("weight_1", weight_1), ("weight_2", weight_2)):
        if w.is_complex():
            w = torch.view_as_real(w)
        require_gpu_f32(name, w)
        if w.dim() != 5 or tuple(w.shape[:3]) != (H_low, W_low, Cin) or w.shape[-1] != 2:
            raise ValueError(f"{name} must be [{H_low}, {W_low}, {Cin}, Cout, 2], got {tuple(w.shape)}")
        ws.append(w)
    Cout = ws[0].shape[3]
    if ws[1].shape[3] != Cout:
        raise ValueError("weight_1 and weight_2 disagree on Cout")
    out = torch.empty((N, Cout, H_all, W_all), dtype=torch.complex64, device=X_ft.device)
    with _lib.device_guard(X_ft.device):
        check(_lib.load().spgt_spectral_mode_contract(
            ptr(X_ft), ptr(ws[0]), ptr(ws[1]), ptr(out), N, Cin, Cout, H_all, W_all, H_low, W_low, H_base_1,
            W_base_1, H_base_2, W_base_2, stream_of(X_ft)))
    return out


def _spectral_modes_compact(Z: Tensor, weight_1: Tensor, weight_2: Tensor) -> Tensor:
    """Z complex64 [N, 2*m_h, Cin, m_w] (the two retained windows stacked along the second axis);
    weight_k fp32 [m_h, m_w, Cin, Cout, 2] -> complex64 [N, 2*m_h, Cout, m_w]."""
    require_gpu_f32("Z", Z, torch.complex64)
    ws = []
    for name, w in (("weight_1", weight_1), ("weight_2", weight_2)):
        if w.is_complex():
            w = torch.view_as_real(w)
        require_gpu_f32(name, w)
        ws.append(w)
    m_h, m_w, Cin, Cout, _ = ws[0].shape
    if tuple(ws[1].shape) != tuple(ws[0].shape):
        raise ValueError("weight_1 and weight_2 must have the same shape")
    N = Z.shape[0]
    if tuple(Z.shape) != (N, 2 * m_h, Cin, m_w):
        raise ValueError(f"Z has shape {tuple(Z.shape)}, expected {(N, 2 * m_h, Cin, m_w)}")
    out = torch.empty((N, 2 * m_h, Cout, m_w), dtype=torch.complex64, device=Z.device)
    with _lib.device_guard(Z.device):
        check(_lib.load().spgt_spectral_modes_compact(ptr(Z), ptr(ws[0]), ptr(ws[1]), ptr(out), N, Cin, Cout, m_h,
                                                      m_w, stream_of(Z)))
    return out


def _bilinear_align_corners(X: Tensor, size) -> Tensor:
    """X [..., H_in, W_in] -> [..., H_out, W_out], F.interpolate(mode='bilinear', align_corners=True)."""
    require_gpu_f32("X", X)
    if X.dim() < 2:
        raise ValueError("X needs at least two dimensions")
    H_out, W_out = (size, size) if isinstance(size, int) else tuple(size)
    lead = tuple(X.shape[:-2])
    H_in, W_in = X.shape[-2:]
    out = torch.empty(lead + (H_out, W_out), dtype=X.dtype, device=X.device)
    planes = prod(lead)
    if planes == 0:
        return out
    with _lib.device_guard(X.device):
        check(_lib.load().spgt_bilinear_align_corners(ptr(X), ptr(out), planes, H_in, W_in, H_out, W_out,
                                                       stream_of(X)))
    return out


def _bilinear_align_corners_nhwc(X: Tensor, size) -> Tensor:
    """X [N, C, H_in, W_in] -> [N, H_out, W_out, C]: the resampling and the permute to channels-last in one pass."""
    require_gpu_f32("X", X)
    if X.dim() != 4:
        raise ValueError("X must be [N, C, H, W]")
    H_out, W_out = (size, size) if isinstance(size, int) else tuple(size)
    N, C, H_in, W_in = X.shape
    out = torch.empty((N, H_out, W_out, C), dtype=X.dtype, device=X.device)
    if out.numel() == 0:
        return out
    with _lib.device_guard(X.device):
        check(_lib.load().spgt_bilinear_align_corners_nhwc(ptr(X), ptr(out), N, C, H_in, W_in, H_out, W_out,
                                                            stream_of(X)))
    return out


def _bilinear_adjoint(grad: Tensor, in_size, nhwc: bool = False) -> Tensor:
    """The gradient of the source of a bilinear align_corners resampling from in_size = (H_in, W_in) to grad's
    size: grad [N, C, H_out, W_out] -> [N, C, H_in, W_in], or with nhwc both tensors channels-last
    ([N, H, W, C], C a multiple of 4).  A gather per source position in a fixed order."""
    require_gpu_f32("grad", grad)
    if grad.dim() != 4:
        raise ValueError("grad must have four dimensions")
    H_in, W_in = (in_size, in_size) if isinstance(in_size, int) else tuple(in_size)
    if nhwc:
        N, H_out, W_out, C = grad.shape
        if C % 4:
            raise ValueError("the channel count must be a multiple of 4")
        out = torch.empty((N, H_in, W_in, C), dtype=grad.dtype, device=grad.device)
    else:
        N, C, H_out, W_out = grad.shape
        out = torch.empty((N, C, H_in, W_in), dtype=grad.dtype, device=grad.device)
    if out.numel() == 0:
        return out
    if grad.numel() == 0:
        return out.zero_()
    with _lib.device_guard(grad.device):
        check(_lib.load().spgt_bilinear_adjoint(ptr(grad), ptr(out), N, C, H_in, W_in, H_out, W_out, 1 if nhwc else 0,
                                                stream_of(grad)))
    return out


def _truncated_dft_rows_supported(r: int, channels: int, modes: int) -> bool:
    return bool(_lib.load().spgt_truncated_dft_rows_supported(int(r), int(channels), int(modes)))


def pad_dft_table(table: Tensor, inverse: bool) -> Tensor:
    """The [r, 2m] twiddle table in the zero-padded layout the row kernels keep in LDS:
    [2*ceil(r/2), 32] (64 columns when 2m > 32) for the forward kernel, [32*ceil(r/32), 2m + 1] for the inverse
    one."""
    r, m2 = table.shape
    if inverse:
        out = table.new_zeros(((r + 31) // 32 * 32, m2 + 1))
    else:
        out = table.new_zeros(((r + 1) // 2 * 2, 32 if m2 <= 32 else 64))
    out[:r, :m2] = table
    return out


_PADDED = {}


def _padded(table: Tensor, inverse: bool) -> Tensor:
    key = (table.data_ptr(), table._version, tuple(table.shape), str(table.device), inverse)
    hit = _PADDED.get(key)
    if hit is None or hit[0]() is not table:
        import weakref
        if len(_PADDED) > 64:
            _PADDED.clear()
        hit = (weakref.ref(table), pad_dft_table(table, inverse))
        _PADDED[key] = hit
    return hit[1]


def _truncated_dft_rows(src: Tensor, table: Tensor, inverse: bool, planar: bool = False) -> Tensor:
    """forward: src [..., r, C] x table [r, 2m] -> [..., C, 2m], or planar [N, 2m, r, C] from src [N, r, r, C];
    inverse: src [..., C, 2m] (or planar [N, 2m, r, C]) -> [..., r, C].  The table is padded to the kernels'
    layout once per table tensor."""
    require_gpu_f32("src", src)
    require_gpu_f32("table", table)
    r, m2 = table.shape
    if m2 > 64 or m2 % 2:
        raise ValueError("the table must have an even number of at most 64 columns")
    padded = _padded(table, inverse)
    if inverse:
        if planar:
            if src.dim() != 4 or src.shape[1] != m2 or src.shape[2] != r:
                raise ValueError(f"planar src must be [N, {m2}, {r}, C]")
            N, C = src.shape[0], src.shape[3]
            lead = (N, r)
        else:
            C = src.shape[-2]
            if src.shape[-1] != m2:
                raise ValueError(f"src has last dimension {src.shape[-1]}, the table has {m2} columns")
            lead = tuple(src.shape[:-2])
        out = torch.empty(lead + (r, C), dtype=src.dtype, device=src.device)
    else:
        C = src.shape[-1]
        if src.shape[-2] != r:
            raise ValueError(f"src has {src.shape[-2]} grid points per row, the table has {r} rows")
        lead = tuple(src.shape[:-2])
        if planar:
            if src.dim() != 4 or src.shape[1] != r:
                raise ValueError(f"planar output needs src [N, {r}, {r}, C]")
            out = torch.empty((src.shape[0], m2, r, C), dtype=src.dtype, device=src.device)
        else:
            out = torch.empty(lead + (C, m2), dtype=src.dtype, device=src.device)
    rows = prod(lead)
    if rows == 0:
        return out
    fn = _lib.load().spgt_truncated_dft_rows_inverse if inverse else _lib.load().spgt_truncated_dft_rows_forward
    with _lib.device_guard(src.device):
        check(fn(ptr(src), ptr(padded), ptr(out), rows, r, C, m2 // 2, int(planar), stream_of(src)))
    return out


def _spectral_modes_middle_supported(r: int, cin: int, cout: int, modes: int) -> bool:
    return bool(_lib.load().spgt_spectral_modes_middle_supported(int(r), int(cin), int(cout), int(modes)))


def _spectral_modes_middle(Y: Tensor, table_h: Tensor, table_h_inverse: Tensor, weight_1: Tensor,
                           weight_2: Tensor) -> Tensor:
    """Y planar [N, 2m, r, Cin] -> U planar [N, 2m, r, Cout]: DFT along h onto the 2m kept rows, complex
    channel contraction with weight_1 | weight_2 [m, m, Cin, Cout, 2], inverse DFT along h."""
    require_gpu_f32("Y", Y)
    require_gpu_f32("table_h", table_h, torch.complex64)
    require_gpu_f32("table_h_inverse", table_h_inverse, torch.complex64)
    require_gpu_f32("weight_1", weight_1)
    require_gpu_f32("weight_2", weight_2)
    N, m2, r, cin = Y.shape
    m = m2 // 2
    cout = weight_1.shape[3]
    if tuple(weight_1.shape) != (m, m, cin, cout, 2) or weight_2.shape != weight_1.shape:
        raise ValueError(f"weights must be [{m}, {m}, {cin}, Cout, 2]")
    if tuple(table_h.shape) != (m2, r) or tuple(table_h_inverse.shape) != (r, m2):
        raise ValueError(f"tables must be [{m2}, {r}] and [{r}, {m2}]")
    U = torch.empty((N, m2, r, cout), dtype=Y.dtype, device=Y.device)
    if U.numel() == 0:
        return U
    lib = _lib.load()
    ws = workspace(lib.spgt_spectral_modes_middle_workspace_bytes(N, cout, m), Y)
    with _lib.device_guard(Y.device):
        check(lib.spgt_spectral_modes_middle(ptr(Y), ptr(table_h), ptr(table_h_inverse), ptr(weight_1), ptr(weight_2),
                                             ptr(U), ptr(ws), ws.numel(), N, r, cin, cout, m, stream_of(Y)))
    return U


_ACT = {None: 0, "none": 0, "relu": 1, "silu": 2}


def _bilinear_resample(X: Tensor, size, src_nhwc: bool = False, dst_nhwc: bool = False, pre_activation=None,
                       pre_count: int = 1, post_activation=None, pre_bias: Tensor = None) -> Tensor:
    """Bilinear align_corners resampling between layouts with the surrounding elementwise steps fused in:
    X [N, C, H, W] (or [N, H, W, C] with src_nhwc) -> [N, C, H', W'] (or [N, H', W', C] with dst_nhwc);
    pre_bias [C] is added to the source samples, pre_activation is then applied to them pre_count times,
    post_activation is applied to the result."""
    require_gpu_f32("X", X)
    if X.dim() != 4:
        raise ValueError("X must have four dimensions")
    if src_nhwc and dst_nhwc:
        raise ValueError("channels-last to channels-last resampling is not provided")
    if pre_activation not in _ACT or post_activation not in _ACT:
        raise ValueError("activations must be None, 'none', 'relu' or 'silu'")
    H_out, W_out = (size, size) if isinstance(size, int) else tuple(size)
    if src_nhwc:
        N, H_in, W_in, C = X.shape
    else:
        N, C, H_in, W_in = X.shape
    shape = (N, H_out, W_out, C) if dst_nhwc else (N, C, H_out, W_out)
    out = torch.empty(shape, dtype=X.dtype, device=X.device)
    if out.numel() == 0:
        return out
    npre = int(pre_count) if _ACT[pre_activation] else 0
    if pre_bias is not None:
        require_gpu_f32("pre_bias", pre_bias)
        if pre_bias.numel() != C:
            raise ValueError(f"pre_bias has {pre_bias.numel()} elements, expected {C}")
    with _lib.device_guard(X.device):
        check(_lib.load().spgt_bilinear_resample(ptr(X), ptr(pre_bias) if pre_bias is not None else None, ptr(out), N, C, H_in, W_in, H_out, W_out, int(src_nhwc),
                                                 int(dst_nhwc), _ACT[pre_activation], npre, _ACT[post_activation],
                                                 stream_of(X)))
    return out


def _drop_seed(device, droprate: float, seed):
    """(rate, seed tensor or None): a seed is drawn when the rate is not zero and none was given."""
    droprate = float(droprate)
    if not 0.0 <= droprate < 1.0:
        raise ValueError("the drop rate must lie in [0, 1)")
    if droprate == 0.0:
        return 0.0, None
    if seed is None:
        seed = dropout_seed(device)
    if not (seed.is_cuda and seed.device == device and seed.dtype == torch.int32 and seed.numel() >= 2 and
            seed.is_contiguous()):
        raise ValueError("seed must be a contiguous int32 tensor of two words on the operands' device")
    return droprate, seed


def _bilinear_resample_concat(sources, size, pre_biases=None, pre_flags=None, pre_activation=None,
                              pre_count: int = 1, post_activation=None, pre_droprate: float = 0.0, seed=None) -> Tensor:
    """post(interpolate(cat(sources, dim=1))) into channels-last without the concatenated tensor: sources are 1 to 4
    NCHW tensors [N, C_s, H, W] whose channel counts add up to a multiple of 4.  Where pre_flags[s] is set, source s
    first gets pre_biases[s] (or nothing, if None) added, is dropped at pre_droprate (ConvResBlock2D's dropout,
    between the convolution and its activation) and has pre_activation applied pre_count times."""
    n = len(sources)
    if not 1 <= n <= 4:
        raise ValueError("1 to 4 sources")
    if pre_activation not in _ACT or post_activation not in _ACT:
        raise ValueError("activations must be None, 'none', 'relu' or 'silu'")
    pre_biases = list(pre_biases) if pre_biases is not None else [None] * n
    pre_flags = [int(bool(f)) for f in pre_flags] if pre_flags is not None else [0] * n
    if len(pre_biases) != n or len(pre_flags) != n:
        raise ValueError("pre_biases and pre_flags need one entry per source")
    for s, X in enumerate(sources):
        require_gpu_f32(f"sources[{s}]", X)
        if X.dim() != 4 or X.shape[0] != sources[0].shape[0] or X.shape[2:] != sources[0].shape[2:]:
            raise ValueError("sources must be [N, C_s, H, W] with the same N, H and W")
        if pre_biases[s] is not None:
            require_gpu_f32(f"pre_biases[{s}]", pre_biases[s])
            if pre_biases[s].numel() != X.shape[1]:
                raise ValueError(f"pre_biases[{s}] has {pre_biases[s].numel()} elements, expected {X.shape[1]}")
    N, _, H_in, W_in = sources[0].shape
    C = sum(X.shape[1] for X in sources)
    if C % 4:
        raise ValueError("the channel counts must add up to a multiple of 4")
    H_out, W_out = (size, size) if isinstance(size, int) else tuple(size)
    out = torch.empty((N, H_out, W_out, C), dtype=sources[0].dtype, device=sources[0].device)
    if out.numel() == 0:
        return out
    srcs = (ctypes.c_void_p * n)(*[X.data_ptr() for X in sources])
    biases = (ctypes.c_void_p * n)(*[b.data_ptr() if b is not None else None for b in pre_biases])
    chans = (ctypes.c_int * n)(*[int(X.shape[1]) for X in sources])
    flags = (ctypes.c_int * n)(*pre_flags)
    npre = int(pre_count) if _ACT[pre_activation] else 0
    pre_droprate, seed = _drop_seed(out.device, pre_droprate if any(pre_flags) else 0.0, seed)
    with _lib.device_guard(out.device):
        if seed is None:
            check(_lib.load().spgt_bilinear_resample_concat(srcs, biases, chans, flags, n, ptr(out), N, H_in, W_in,
                                                            H_out, W_out, _ACT[pre_activation], npre,
                                                            _ACT[post_activation], stream_of(out)))
        else:
            check(_lib.load().spgt_bilinear_resample_concat_dropout(
                srcs, biases, chans, flags, n, ptr(out), N, H_in, W_in, H_out, W_out, _ACT[pre_activation], npre,
                _ACT[post_activation], ptr(seed), pre_droprate, stream_of(out)))
    return out


def _upsample_conv3x3_gather(Z: Tensor, bias, size, activation=None, count: int = 1) -> Tensor:
    """Z [N, H, W, 9, C] (the nine per-tap 1x1 products of a 3x3 convolution's input at low resolution) ->
    act^count(conv3x3(interpolate(X)) + bias) as [N, H', W', C] channels-last; C a multiple of 4."""
    require_gpu_f32("Z", Z)
    if Z.dim() != 5 or Z.shape[3] != 9:
        raise ValueError("Z must be [N, H, W, 9, C]")
    if activation not in _ACT:
        raise ValueError("activation must be None, 'none', 'relu' or 'silu'")
    N, H_in, W_in, _, C = Z.shape
    if C % 4:
        raise ValueError("the channel count must be a multiple of 4")
    if bias is not None:
        require_gpu_f32("bias", bias)
        if bias.numel() != C:
            raise ValueError(f"bias has {bias.numel()} elements, expected {C}")
    H_out, W_out = (size, size) if isinstance(size, int) else tuple(size)
    out = torch.empty((N, H_out, W_out, C), dtype=Z.dtype, device=Z.device)
    if out.numel() == 0:
        return out
    with _lib.device_guard(Z.device):
        check(_lib.load().spgt_upsample_conv3x3_gather(ptr(Z), ptr(bias) if bias is not None else None, ptr(out), N, C,
                                                       H_in, W_in, H_out, W_out, _ACT[activation], int(count),
                                                       stream_of(Z)))
    return out


def _upsample_conv3x3_gather_adjoint(grad: Tensor, in_size) -> Tensor:
    """The gradient of the per-tap products of upsample_conv3x3_gather (no bias, no activation): grad
    [N, H', W', C] -> dZ [N, H, W, 9, C] with in_size = (H, W); C a multiple of 4."""
    require_gpu_f32("grad", grad)
    if grad.dim() != 4:
        raise ValueError("grad must be [N, H', W', C]")
    N, H_out, W_out, C = grad.shape
    if C % 4:
        raise ValueError("the channel count must be a multiple of 4")
    H_in, W_in = (in_size, in_size) if isinstance(in_size, int) else tuple(in_size)
    out = torch.empty((N, H_in, W_in, 9, C), dtype=grad.dtype, device=grad.device)
    if out.numel() == 0:
        return out
    if grad.numel() == 0:
        return out.zero_()
    with _lib.device_guard(grad.device):
        check(_lib.load().spgt_upsample_conv3x3_gather_adjoint(ptr(grad), ptr(out), N, C, H_in, W_in, H_out, W_out,
                                                               stream_of(grad)))
    return out


def _bilinear_nhwc_affine(X: Tensor, size, extra: Tensor = None, weight_extra_kn: Tensor = None) -> Tensor:
    """Channels-last bilinear align_corners resampling X [N, H, W, C] -> [N, H', W', C] (C a multiple of 4), plus
    extra @ weight_extra_kn for extra [N, H', W', E] and weight_extra_kn [E, C], E <= 4: the few columns that a
    Linear applied before the resampling could not see."""
    require_gpu_f32("X", X)
    if X.dim() != 4:
        raise ValueError("X must have four dimensions")
    N, H_in, W_in, C = X.shape
    if C % 4:
        raise ValueError("the channel count must be a multiple of 4")
    H_out, W_out = (size, size) if isinstance(size, int) else tuple(size)
    E = 0
    if extra is not None:
        require_gpu_f32("extra", extra)
        require_gpu_f32("weight_extra_kn", weight_extra_kn)
        E = weight_extra_kn.shape[0]
        if E > 4 or tuple(weight_extra_kn.shape) != (E, C) or tuple(extra.shape) != (N, H_out, W_out, E):
            raise ValueError("extra must be [N, H', W', E] and weight_extra_kn [E, C] with E <= 4")
    out = torch.empty((N, H_out, W_out, C), dtype=X.dtype, device=X.device)
    if out.numel() == 0:
        return out
    with _lib.device_guard(X.device):
        check(_lib.load().spgt_bilinear_nhwc_affine(ptr(X), ptr(out), N, C, H_in, W_in, H_out, W_out,
                                                    ptr(extra) if E else None, ptr(weight_extra_kn) if E else None, E,
                                                    stream_of(X)))
    return out


def _bias_activation_nchw_(X: Tensor, bias, activation=None, count: int = 1, droprate: float = 0.0, seed=None) -> Tensor:
    """In place on X [N, C, ...]: X = activation^count(dropout(X + bias[c], droprate)); returns X."""
    require_gpu_f32("X", X)
    if X.dim() < 2:
        raise ValueError("X needs at least two dimensions")
    if activation not in _ACT:
        raise ValueError("activation must be None, 'none', 'relu' or 'silu'")
    N, C = X.shape[:2]
    HW = prod(X.shape[2:])
    if bias is not None:
        require_gpu_f32("bias", bias)
        if bias.numel() != C:
            raise ValueError(f"bias has {bias.numel()} elements, expected {C}")
    if X.numel() == 0:
        return X
    droprate, seed = _drop_seed(X.device, droprate, seed)
    with _lib.device_guard(X.device):
        if seed is None:
            check(_lib.load().spgt_bias_activation_nchw(ptr(X), ptr(bias) if bias is not None else None, N, C, HW,
                                                        _ACT[activation], int(count), stream_of(X)))
        else:
            check(_lib.load().spgt_bias_activation_nchw_dropout(ptr(X), ptr(bias) if bias is not None else None, N, C,
                                                                HW, _ACT[activation], int(count), ptr(seed), droprate,
                                                                stream_of(X)))
    return X


def _denormalize_boundary(X: Tensor, scale: Tensor, shift: Tensor, zero_boundary: bool) -> Tensor:
    """X * scale + shift on X [N, H, W, C], zero on the grid's boundary if asked; scale and shift hold one
    value or H*W*C values."""
    require_gpu_f32("X", X)
    require_gpu_f32("scale", scale)
    require_gpu_f32("shift", shift)
    if X.dim() != 4:
        raise ValueError("X must be [N, H, W, C]")
    N, H, W, C = X.shape
    if scale.numel() != shift.numel() or scale.numel() not in (1, H * W * C):
        raise ValueError("scale and shift must hold one value or H*W*C values")
    if zero_boundary and min(H, W) < 2:
        raise ValueError("a grid with fewer than two rows or columns has no interior to pad")
    out = torch.empty_like(X)
    if X.numel() == 0:
        return out
    with _lib.device_guard(X.device):
        check(_lib.load().spgt_denormalize_boundary(ptr(X), ptr(scale), ptr(shift), int(scale.numel() > 1), ptr(out),
                                                    N, H, W, C, int(bool(zero_boundary)), stream_of(X)))
    return out


def _spectral_inverse_linear_supported(r: int, cin: int, cout: int, modes: int) -> bool:
    return bool(_lib.load().spgt_spectral_inverse_linear_supported(int(r), int(cin), int(cout), int(modes)))


def _spectral_inverse_linear(U: Tensor, table_operand: Tensor, X: Tensor, weight_kn: Tensor, bias, activation) -> Tensor:
    """act(X @ weight_kn + bias + inverse row DFT of U): U planar [N, 2m, r, Cout], X [N, r, r, Cin],
    weight_kn [Cin, Cout] -> [N, r, r, Cout]."""
    for name, t in (("U", U), ("table_operand", table_operand), ("X", X), ("weight_kn", weight_kn)):
        require_gpu_f32(name, t)
    if activation not in _ACT:
        raise ValueError("activation must be None, 'none', 'relu' or 'silu'")
    if X.dim() != 4 or X.shape[1] != X.shape[2]:
        raise ValueError("X must be [N, r, r, Cin]")
    N, r, _, cin = X.shape
    if weight_kn.dim() != 2 or weight_kn.shape[0] != cin:
        raise ValueError("weight_kn must be [Cin, Cout]")
    cout = weight_kn.shape[1]
    if U.dim() != 4 or U.shape[0] != N or U.shape[2] != r or U.shape[3] != cout or U.shape[1] % 2:
        raise ValueError("U must be planar [N, 2*modes, r, Cout]")
    modes = U.shape[1] // 2
    steps = 16 if modes <= 16 else 32
    if tuple(table_operand.shape) != ((r + 31) // 32, steps, 64):
        raise ValueError(f"table_operand must be [ceil(r/32), {steps}, 64]")
    if bias is not None:
        require_gpu_f32("bias", bias)
        if bias.numel() != cout:
            raise ValueError(f"bias has {bias.numel()} elements, expected {cout}")
    if not _spectral_inverse_linear_supported(r, cin, cout, modes):
        raise ValueError("spectral_inverse_linear: needs (Cin, Cout) in {32->32, 64->64, 64->32, 128->32, 128->64}, "
                         "2*modes <= min(64, r), r <= 1024")
    out = torch.empty((N, r, r, cout), dtype=X.dtype, device=X.device)
    if X.numel() == 0:
        return out
    with _lib.device_guard(X.device):
        check(_lib.load().spgt_spectral_inverse_linear(ptr(U), ptr(table_operand), ptr(X), ptr(weight_kn),
                                                       ptr(bias) if bias is not None else None, _ACT[activation],
                                                       ptr(out), N * r, r, cin, cout, modes, stream_of(X)))
    return out


def _conv3x3_resample(X: Tensor, weight: Tensor, bias, size, pre_activation=None, post_activation=None,
                      droprate: float = 0.0, seed=None) -> Tensor:
    """post(interpolate(pre(dropout(conv3x3(X, weight, padding=1) + bias, droprate)))) for X [N, H, W, Cin]
    channels-last with Cin <= 4: [N, Cout, H', W'] without the full-resolution convolution output ever being stored."""
    require_gpu_f32("X", X)
    require_gpu_f32("weight", weight)
    if X.dim() != 4 or weight.dim() != 4 or tuple(weight.shape[2:]) != (3, 3) or weight.shape[1] != X.shape[3]:
        raise ValueError("X must be [N, H, W, Cin] and weight [Cout, Cin, 3, 3]")
    if pre_activation not in _ACT or post_activation not in _ACT:
        raise ValueError("activations must be None, 'none', 'relu' or 'silu'")
    N, H, W, Cin = X.shape
    Cout = weight.shape[0]
    if bias is not None:
        require_gpu_f32("bias", bias)
        if bias.numel() != Cout:
            raise ValueError(f"bias has {bias.numel()} elements, expected {Cout}")
    H_out, W_out = (size, size) if isinstance(size, int) else tuple(size)
    out = torch.empty((N, Cout, H_out, W_out), dtype=X.dtype, device=X.device)
    if out.numel() == 0:
        return out
    droprate, seed = _drop_seed(X.device, droprate, seed)
    with _lib.device_guard(X.device):
        if seed is None:
            check(_lib.load().spgt_conv3x3_resample(ptr(X), ptr(weight), ptr(bias) if bias is not None else None,
                                                    ptr(out), N, Cin, Cout, H, W, H_out, W_out, _ACT[pre_activation],
                                                    _ACT[post_activation], stream_of(X)))
        else:
            check(_lib.load().spgt_conv3x3_resample_dropout(ptr(X), ptr(weight), ptr(bias) if bias is not None else None,
                                                            ptr(out), N, Cin, Cout, H, W, H_out, W_out,
                                                            _ACT[pre_activation], _ACT[post_activation], ptr(seed),
                                                            droprate, stream_of(X)))
    return out


def _conv3x3_resample_backward(X: Tensor, weight: Tensor, bias, grad: Tensor, pre_activation=None,
                               droprate: float = 0.0, seed=None):
    """(dW [Cout, Cin, 3, 3], db [Cout]) of P = interpolate(pre(dropout(conv3x3(X, weight, padding=1) + bias)))
    from grad = dL/dP [N, Cout, H', W'], for X [N, H, W, Cin] (Cin <= 4) that needs no gradient.  The
    full-resolution chain is formed again from X, the weights and the forward's seed."""
    require_gpu_f32("X", X)
    require_gpu_f32("weight", weight)
    require_gpu_f32("grad", grad)
    if X.dim() != 4 or weight.dim() != 4 or tuple(weight.shape[2:]) != (3, 3) or weight.shape[1] != X.shape[3]:
        raise ValueError("X must be [N, H, W, Cin] and weight [Cout, Cin, 3, 3]")
    if pre_activation not in _ACT:
        raise ValueError("activation must be None, 'none', 'relu' or 'silu'")
    N, H, W, Cin = X.shape
    Cout = weight.shape[0]
    if grad.dim() != 4 or grad.shape[0] != N or grad.shape[1] != Cout:
        raise ValueError("grad must be [N, Cout, H', W']")
    if bias is not None:
        require_gpu_f32("bias", bias)
    if droprate > 0 and seed is None:
        raise ValueError("the backward needs the forward's seed")
    droprate, seed = _drop_seed(X.device, droprate, seed)
    H_out, W_out = grad.shape[2:]
    lib = _lib.load()
    nbytes = lib.spgt_conv3x3_resample_backward_workspace_bytes(N, Cin, Cout, H, W)
    if nbytes == 0:
        raise ValueError(f"unsupported shape: N={N} Cin={Cin} Cout={Cout} H={H}")
    ws = workspace(nbytes, X)
    R = (1 + 9 * Cin + 3) // 4 * 4
    out = torch.empty((Cout, R), dtype=torch.float32, device=X.device)
    with _lib.device_guard(X.device):
        check(lib.spgt_conv3x3_resample_backward(ptr(X), ptr(weight), ptr(bias) if bias is not None else None, ptr(grad),
                                                 ptr(out), ptr(ws), ws.numel(), N, Cin, Cout, H, W, H_out, W_out,
                                                 _ACT[pre_activation], ptr(seed) if seed is not None else None, droprate,
                                                 stream_of(X)))
    return out[:, 1:1 + 9 * Cin].reshape(Cout, Cin, 3, 3), out[:, 0]


dexts = SimpleNamespace(
    conv3x3_resample=_conv3x3_resample,
    conv3x3_resample_backward=_conv3x3_resample_backward,
    spectral_inverse_linear_supported=_spectral_inverse_linear_supported,
    spectral_inverse_linear=_spectral_inverse_linear,
    denormalize_boundary=_denormalize_boundary,
    truncated_dft_rows_supported=_truncated_dft_rows_supported,
    truncated_dft_rows=_truncated_dft_rows,
    spectral_modes_middle_supported=_spectral_modes_middle_supported,
    spectral_modes_middle=_spectral_modes_middle,
    bias_activation_nchw_=_bias_activation_nchw_,
    bilinear_resample=_bilinear_resample,
    bilinear_nhwc_affine=_bilinear_nhwc_affine,
    upsample_conv3x3_gather=_upsample_conv3x3_gather,
    bilinear_resample_concat=_bilinear_resample_concat,
    bilinear_align_corners_nhwc=_bilinear_align_corners_nhwc,
    batched_transpose=_batched_transpose,
    transpose_gather_dual=_transpose_gather_dual,
    transpose_scatter_dual=_transpose_scatter_dual,
    spectral_mode_contract=_spectral_mode_contract,
    spectral_modes_compact=_spectral_modes_compact,
    bilinear_align_corners=_bilinear_align_corners,
    bilinear_adjoint=_bilinear_adjoint,
    upsample_conv3x3_gather_adjoint=_upsample_conv3x3_gather_adjoint,
)


# --------------------------------------------------------------------------- #
# python surface (autograd-aware; each backward is another of these operators)
# --------------------------------------------------------------------------- #

class Batched_Transpose_Function(torch.autograd.Function):
    @staticmethod
    def forward(ctx: Any, X: Tensor, batch_list: List[int], M_list: List[int], N_list: List[int]):
        ctx.extras_shape = [batch_list, M_list, N_list]
        return dexts.batched_transpose(X, batch_list, M_list, N_list)

    @staticmethod
    def backward(ctx: Any, grad_out: Tensor):
        batch_list, M_list, N_list = ctx.extras_shape
        return dexts.batched_transpose(grad_out.contiguous(), batch_list, N_list, M_list), None, None, None


class Transpose_Gather_Dual_Function(torch.autograd.Function):
    @staticmethod
    def forward(ctx: Any, src: Tensor, dim_list, H_all, W_all, H_low, W_low, H_base_1, W_base_1, H_base_2, W_base_2):
        ctx.extras_shape = [dim_list, H_all, W_all, H_low, W_low, H_base_1, W_base_1, H_base_2, W_base_2]
        return dexts.transpose_gather_dual(src, *ctx.extras_shape)

    @staticmethod
    def backward(ctx: Any, grad_out1: Tensor, grad_out2: Tensor):
        grad_src = dexts.transpose_scatter_dual(grad_out1.contiguous(), grad_out2.contiguous(), *ctx.extras_shape)
        return (grad_src,) + (None,) * 9


class Transpose_Scatter_Dual_Function(torch.autograd.Function):
    @staticmethod
    def forward(ctx: Any, src1: Tensor, src2: Tensor, dim_list, H_all, W_all, H_low, W_low, H_base_1, W_base_1,
                H_base_2, W_base_2):
        ctx.extras_shape = [dim_list, H_all, W_all, H_low, W_low, H_base_1, W_base_1, H_base_2, W_base_2]
        return dexts.transpose_scatter_dual(src1, src2, *ctx.extras_shape)

    @staticmethod
    def backward(ctx: Any, grad_out: Tensor):
        g1, g2 = dexts.transpose_gather_dual(grad_out.contiguous(), *ctx.extras_shape)
        return (g1, g2) + (None,) * 9


def batched_transpose(X: Tensor, batch_list: List[int], M_list: List[int], N_list: List[int]) -> Tensor:
    return Batched_Transpose_Function.apply(X, batch_list, M_list, N_list)


def transpose_gather_dual(src: Tensor, dim_list: List[int], H_all, W_all, H_low, W_low, H_base_1, W_base_1, H_base_2,
                          W_base_2) -> Tuple[Tensor, Tensor]:
    return Transpose_Gather_Dual_Function.apply(src, dim_list, H_all, W_all, H_low, W_low, H_base_1, W_base_1,
                                                H_base_2, W_base_2)


def transpose_scatter_dual(src1: Tensor, src2: Tensor, dim_list: List[int], H_all, W_all, H_low, W_low, H_base_1,
                           W_base_1, H_base_2, W_base_2) -> Tensor:
    return Transpose_Scatter_Dual_Function.apply(src1, src2, dim_list, H_all, W_all, H_low, W_low, H_base_1, W_base_1,
                                                 H_base_2, W_base_2)


def spectral_mode_contract(X_ft: Tensor, weight_1: Tensor, weight_2: Tensor, H_low: int, W_low: int, H_base_1: int,
                           W_base_1: int, H_base_2: int, W_base_2: int) -> Tensor:
    """Gather of the two corner windows, per-mode complex channel contraction and scatter
    into a zero-filled spectrum, in one call (inference only: no autograd graph is recorded)."""
    return dexts.spectral_mode_contract(X_ft.detach(), weight_1.detach(), weight_2.detach(), H_low, W_low, H_base_1,
                                        W_base_1, H_base_2, W_base_2)


def spectral_modes_compact(Z: Tensor, weight_1: Tensor, weight_2: Tensor) -> Tensor:
    """Per-mode complex channel contraction on operands that hold only the retained modes (inference only)."""
    return dexts.spectral_modes_compact(Z.detach(), weight_1.detach(), weight_2.detach())


def bilinear_align_corners(X: Tensor, size) -> Tensor:
    """F.interpolate(X, size, mode='bilinear', align_corners=True) (inference only)."""
    return dexts.bilinear_align_corners(X.detach(), size)


def bilinear_align_corners_nhwc(X: Tensor, size) -> Tensor:
    """F.interpolate(X, size, mode='bilinear', align_corners=True).permute(0, 2, 3, 1), contiguous (inference only)."""
    return dexts.bilinear_align_corners_nhwc(X.detach(), size)


def _pair(size):
    return (size, size) if isinstance(size, int) else tuple(size)


class Bilinear_Function(torch.autograd.Function):
    """F.interpolate(X, size, mode='bilinear', align_corners=True) on [N, C, H, W]; backward = bilinear_adjoint."""

    @staticmethod
    def forward(ctx: Any, X: Tensor, size):
        ctx.in_size = tuple(X.shape[-2:])
        return dexts.bilinear_align_corners(X.contiguous(), _pair(size))

    @staticmethod
    def backward(ctx: Any, grad_out: Tensor):
        return dexts.bilinear_adjoint(grad_out.contiguous(), ctx.in_size, False), None


class Bilinear_To_Nhwc_Function(torch.autograd.Function):
    """The same from [N, C, H, W] to channels-last [N, H', W', C].  The backward gathers channels-last (C a multiple
    of 4) and transposes the result into the input's [N, C, H, W] layout."""

    @staticmethod
    def forward(ctx: Any, X: Tensor, size):
        ctx.in_size = tuple(X.shape[-2:])
        return dexts.bilinear_align_corners_nhwc(X.contiguous(), _pair(size))

    @staticmethod
    def backward(ctx: Any, grad_out: Tensor):
        g = dexts.bilinear_adjoint(grad_out.contiguous(), ctx.in_size, True)  # [N, H, W, C]
        N, H, W, C = g.shape
        # handed back in the input's own layout: a permuted view would send every elementwise backward upstream
        # (activations, dropout) down torch's strided path, three to four times slower than one transpose here
        return dexts.batched_transpose(g, [N], [H * W], [C]).view(N, C, H, W), None


class Bilinear_Nhwc_Function(torch.autograd.Function):
    """The same with channels-last tensors on both sides, [N, H, W, C] -> [N, H', W', C], C a multiple of 4."""

    @staticmethod
    def forward(ctx: Any, X: Tensor, size):
        ctx.in_size = tuple(X.shape[1:3])
        return dexts.bilinear_nhwc_affine(X.contiguous(), _pair(size))

    @staticmethod
    def backward(ctx: Any, grad_out: Tensor):
        return dexts.bilinear_adjoint(grad_out.contiguous(), ctx.in_size, True), None


class Upsample_Conv3x3_Gather_Function(torch.autograd.Function):
    """conv3x3(interpolate(X)) + bias from the per-tap products Z [N, H, W, 9, C] of X at low resolution, no
    activation; backward: the gather's adjoint for Z, a sum over the pixels for the bias."""

    @staticmethod
    def forward(ctx: Any, Z: Tensor, bias, size):
        ctx.in_size = tuple(Z.shape[1:3])
        ctx.has_bias = bias is not None
        return dexts.upsample_conv3x3_gather(Z.contiguous(), bias, _pair(size), None, 0)

    @staticmethod
    def backward(ctx: Any, grad_out: Tensor):
        g = grad_out.contiguous()
        dZ = dexts.upsample_conv3x3_gather_adjoint(g, ctx.in_size) if ctx.needs_input_grad[0] else None
        db = g.sum((0, 1, 2)) if ctx.has_bias and ctx.needs_input_grad[1] else None
        return dZ, db, None


def upsample_conv3x3_gather_train(Z: Tensor, bias, size) -> Tensor:
    """conv3x3(interpolate(X)) + bias from the per-tap products Z of X, with an autograd graph (no activation)."""
    return Upsample_Conv3x3_Gather_Function.apply(Z, bias, size)


def upsample_conv3x3_gather_adjoint(grad: Tensor, in_size) -> Tensor:
    """Gradient of the per-tap products of upsample_conv3x3_gather from the gradient of its (unactivated) result."""
    return dexts.upsample_conv3x3_gather_adjoint(grad.detach(), in_size)


class Conv3x3_Resample_Function(torch.autograd.Function):
    """interpolate(pre(dropout(conv3x3(X) + bias))) for a channels-last X [N, H, W, Cin <= 4] that needs no gradient
    (the down-scaler's first stage on the model's input): one kernel forward, one backward that forms the
    full-resolution chain again instead of storing it."""

    @staticmethod
    def forward(ctx: Any, X: Tensor, weight: Tensor, bias, size, pre_activation, droprate: float):
        seed = dropout_seed(X.device) if droprate > 0 else None
        ctx.save_for_backward(X, weight, bias if bias is not None else weight.new_empty(0))
        ctx.has_bias, ctx.pre, ctx.droprate, ctx.seed = bias is not None, pre_activation, droprate, seed
        return dexts.conv3x3_resample(X.contiguous(), weight.contiguous(), bias, _pair(size), pre_activation, None,
                                      droprate, seed)

    @staticmethod
    def backward(ctx: Any, grad_out: Tensor):
        X, weight, bias = ctx.saved_tensors
        dW, db = dexts.conv3x3_resample_backward(X.contiguous(), weight.contiguous(), bias if ctx.has_bias else None,
                                                 grad_out.contiguous(), ctx.pre, ctx.droprate, ctx.seed)
        return None, dW, (db if ctx.has_bias else None), None, None, None


def conv3x3_resample_train(X: Tensor, weight: Tensor, bias, size, pre_activation=None, droprate: float = 0.0) -> Tensor:
    """interpolate(pre(dropout(conv3x3(X) + bias))) with an autograd graph for the weight and the bias; X itself
    must not need a gradient."""
    if X.requires_grad:
        raise ValueError("conv3x3_resample_train has no gradient for its input")
    return Conv3x3_Resample_Function.apply(X, weight, bias, size, pre_activation, float(droprate))


def bilinear_adjoint(grad: Tensor, in_size, nhwc: bool = False) -> Tensor:
    """Gradient of the source of a bilinear align_corners resampling from in_size to grad's size."""
    return dexts.bilinear_adjoint(grad.detach(), in_size, nhwc)


def bilinear_train(X: Tensor, size) -> Tensor:
    """F.interpolate(X, size, mode='bilinear', align_corners=True) on [N, C, H, W] with an autograd graph."""
    return Bilinear_Function.apply(X, size)


def bilinear_to_nhwc_train(X: Tensor, size) -> Tensor:
    """interpolate(X).permute(0, 2, 3, 1), contiguous, with an autograd graph; X [N, C, H, W], C a multiple of 4."""
    return Bilinear_To_Nhwc_Function.apply(X, size)


def bilinear_nhwc_train(X: Tensor, size) -> Tensor:
    """Channels-last interpolate, [N, H, W, C] -> [N, H', W', C], with an autograd graph; C a multiple of 4."""
    return Bilinear_Nhwc_Function.apply(X, size)


def bilinear_resample(X: Tensor, size, src_nhwc: bool = False, dst_nhwc: bool = False, pre_activation=None,
                      pre_count: int = 1, post_activation=None, pre_bias: Tensor = None) -> Tensor:
    """post(interpolate(pre^pre_count(X + pre_bias))) between NCHW / NHWC layouts in one pass (inference only)."""
    return dexts.bilinear_resample(X.detach(), size, src_nhwc, dst_nhwc, pre_activation, pre_count, post_activation,
                                   None if pre_bias is None else pre_bias.detach())


def bilinear_resample_concat(sources, size, pre_biases=None, pre_flags=None, pre_activation=None, pre_count: int = 1,
                             post_activation=None, pre_droprate: float = 0.0, seed=None) -> Tensor:
    """post(interpolate(cat(sources, dim=1))) into channels-last, the concatenation never stored (inference only)."""
    return dexts.bilinear_resample_concat([X.detach() for X in sources], size,
                                          None if pre_biases is None else [None if b is None else b.detach()
                                                                           for b in pre_biases],
                                          pre_flags, pre_activation, pre_count, post_activation, pre_droprate, seed)


def upsample_conv3x3_gather(Z: Tensor, bias, size, activation=None, count: int = 1) -> Tensor:
    """act^count(conv3x3(interpolate(X)) + bias) from the per-tap products Z of X at low resolution (inference only)."""
    return dexts.upsample_conv3x3_gather(Z.detach(), None if bias is None else bias.detach(), size, activation, count)


def bilinear_nhwc_affine(X: Tensor, size, extra: Tensor = None, weight_extra_kn: Tensor = None) -> Tensor:
    """interpolate(X) + extra @ weight_extra_kn, channels-last on both sides (inference only)."""
    return dexts.bilinear_nhwc_affine(X.detach(), size, None if extra is None else extra.detach(),
                                      None if weight_extra_kn is None else weight_extra_kn.detach())


def bias_activation_nchw_(X: Tensor, bias, activation=None, count: int = 1, droprate: float = 0.0, seed=None) -> Tensor:
    """In place: X = activation^count(dropout(X + bias[c], droprate)) on [N, C, ...] (inference only)."""
    return dexts.bias_activation_nchw_(X, None if bias is None else bias.detach(), activation, count, droprate, seed)


def spectral_inverse_linear_supported(r: int, cin: int, cout: int, modes: int) -> bool:
    """True when spectral_inverse_linear has a kernel for this shape."""
    return dexts.spectral_inverse_linear_supported(r, cin, cout, modes)


def inverse_table_operand(table: Tensor) -> Tensor:
    """The inverse row-DFT table [r, 2m] in the order the fused kernel's lanes read it: [ceil(r/32), steps, 64]
    with entry (t, kk, l) = table[32 t + l % 32, 2 kk + l // 32], zero outside the table; steps = 16 for
    m <= 16, else 32."""
    r, m2 = table.shape
    wt = (r + 31) // 32
    steps = 16 if m2 <= 32 else 32
    full = torch.zeros(wt * 32, 2 * steps, dtype=table.dtype, device=table.device)
    full[:r, :m2] = table
    # [t, w', kk, kh] -> [t, kk, kh, w'] -> lanes l = kh*32 + w'
    return full.view(wt, 32, steps, 2).permute(0, 2, 3, 1).reshape(wt, steps, 64).contiguous()


def spectral_inverse_linear(U: Tensor, table_operand: Tensor, X: Tensor, weight_kn: Tensor, bias, activation) -> Tensor:
    """The end of Sp_SpectralConv2D.forward in one pass: act(X @ weight_kn + bias + y) with y the inverse DFT
    along w of the planar spectrum U [N, 2m, r, C] (what truncated_dft_rows_inverse(U, table, planar=True)
    returns); X [N, r, r, C], 32 or 64 channels (inference only)."""
    return dexts.spectral_inverse_linear(U.detach(), table_operand, X.detach(), weight_kn,
                                         None if bias is None else bias.detach(), activation)


def denormalize_boundary(X: Tensor, scale: Tensor, shift: Tensor, zero_boundary: bool) -> Tensor:
    """The end of the model's forward in one pass: X * scale + shift on [N, H, W, C] (multiply and add rounded
    separately), then zero on the outermost rows and columns of the grid if asked (inference only)."""
    return dexts.denormalize_boundary(X.detach(), scale, shift, zero_boundary)


def truncated_dft_rows_supported(r: int, channels: int, modes: int) -> bool:
    """True when truncated_dft_rows_forward / _inverse have a kernel for this shape."""
    return dexts.truncated_dft_rows_supported(r, channels, modes)


def truncated_dft_rows_forward(X: Tensor, table: Tensor, planar: bool = False) -> Tensor:
    """Y[..., c, j] = sum_w X[..., w, c] table[w, j]: X [..., r, C], table [r, 2m] -> [..., C, 2m], or with
    planar X [N, r, r, C] -> [N, 2m, r, C] (inference only)."""
    return dexts.truncated_dft_rows(X.detach(), table, False, planar)


def truncated_dft_rows_inverse(U: Tensor, table: Tensor, planar: bool = False) -> Tensor:
    """y[..., w, o] = sum_j table[w, j] U[..., o, j]: U [..., C, 2m] (or planar [N, 2m, r, C]), table [r, 2m]
    -> [..., r, C] (inference only)."""
    return dexts.truncated_dft_rows(U.detach(), table, True, planar)


def spectral_modes_middle_supported(r: int, cin: int, cout: int, modes: int) -> bool:
    """True when spectral_modes_middle has a kernel for this shape."""
    return dexts.spectral_modes_middle_supported(r, cin, cout, modes)


def spectral_modes_middle(Y: Tensor, table_h: Tensor, table_h_inverse: Tensor, weight_1: Tensor,
                          weight_2: Tensor) -> Tensor:
    """DFT along h onto the kept rows, mode-wise complex channel contraction, inverse DFT along h, on the
    planar operands of the row kernels (inference only)."""
    return dexts.spectral_modes_middle(Y.detach(), table_h, table_h_inverse, weight_1.detach(), weight_2.detach())


def conv3x3_resample_supported(cin: int) -> bool:
    """True when conv3x3_resample has a kernel for this number of input channels."""
    return bool(_lib.load().spgt_conv3x3_resample_supported(int(cin)))


def conv3x3_resample(X: Tensor, weight: Tensor, bias, size, pre_activation=None, post_activation=None,
                     droprate: float = 0.0, seed=None) -> Tensor:
    """3x3 convolution (padding 1) of a channels-last input with few channels, bias, dropout, activation, bilinear
    align_corners resampling and a second activation in one pass: [N, H, W, Cin] -> [N, Cout, H', W'] (inference only)."""
    return dexts.conv3x3_resample(X.detach(), weight.detach(), None if bias is None else bias.detach(), size,
                                  pre_activation, post_activation, droprate, seed)
