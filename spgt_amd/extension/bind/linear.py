"""Fused token-major linear layers, backed by libspgt_hip.so.

The reference's modules call nn.Linear and then separate elementwise kernels for
the activation and the residual add (network/layer.py:155-174,
network/sp_layer.py:75, 97-103 and 132, 155, network/sp_model.py:60, 63); here the three
are one kernel (fused_linear, fused_ffn_scalar, fused_encoder_tail).  These functions build no
autograd graph themselves: the modules call them under torch.no_grad() and, when gradients are
required, through autograd functions (network/layer.py) whose backward uses linear_weight_grad
(dW, db in one pass over the tokens) and dropout_add from this file.
"""
from typing import Optional

import torch
from torch import Tensor

from ... import _lib
from ..._lib import check, dropout_seed, ptr, require_gpu_f32, stream_of

ACTIVATIONS = {"none": 0, "relu": 1, "silu": 2}
RES_NONE, RES_BEFORE_ACT, RES_AFTER_ACT = 0, 1, 2


def linear_supported(in_features: int, out_features: int) -> bool:
    """True when fused_linear has a kernel for this shape."""
    return bool(_lib.load().spgt_linear_supported(int(in_features), int(out_features)))


def _rows(name: str, t: Tensor, width: int):
    """View `t` [..., width] as rows with one stride; returns (tensor to keep alive, row count, row stride)."""
    require_gpu_f32(name, t, contiguous=False)
    if t.shape[-1] != width:
        raise ValueError(f"{name} has last dimension {t.shape[-1]}, expected {width}")
    if t.stride(-1) == 1 and t.dim() == 2 and t.stride(0) >= width and t.stride(0) % 4 == 0 and t.data_ptr() % 16 == 0:
        return t, t.shape[0], t.stride(0)
    t = t.contiguous()
    return t, t.numel() // max(width, 1), width


def fused_linear(x: Tensor, weight_kn: Tensor, bias: Optional[Tensor] = None, activation: str = "none",
                 residual: Optional[Tensor] = None, residual_after_activation: bool = False,
                 planes: int = 1, x_extra: Optional[Tensor] = None,
                 weight_extra_kn: Optional[Tensor] = None) -> Tensor:
    """act(x @ weight_kn + bias [+ residual]) or act(x @ weight_kn + bias) + residual.

    x [..., K] (a 2-D x may have a row stride larger than K), weight_kn [K, N] contiguous
    (the transpose of nn.Linear.weight), bias [N] or None, residual [..., N] or None.
    x_extra [..., E] with weight_extra_kn [E, N] (E <= 4) adds x_extra @ weight_extra_kn before the residual and
    the activation: a few more input columns without a concatenation.
    Returns a new contiguous [..., N] tensor, or with planes > 1 a [planes, ..., N / planes] tensor whose
    plane p holds output columns p*N/planes .. (p+1)*N/planes - 1.
    """
    if activation not in ACTIVATIONS:
        raise ValueError(f"activation must be one of {sorted(ACTIVATIONS)}")
    require_gpu_f32("weight_kn", weight_kn)
    K, N = weight_kn.shape
    xr, T, ldx = _rows("x", x, K)
    lead = list(x.shape[:-1])
    if bias is not None:
        require_gpu_f32("bias", bias)
        if bias.numel() != N:
            raise ValueError(f"bias has {bias.numel()} elements, expected {N}")
    if planes < 1 or N % planes or (N // planes) % 32:
        raise ValueError("planes must divide the output width into multiples of 32 columns")
    pc = N // planes
    out = torch.empty(([planes] if planes > 1 else []) + lead + [pc], dtype=x.dtype, device=x.device)
    mode, rr, ldr = RES_NONE, None, 0
    if residual is not None:
        if list(residual.shape[:-1]) != lead and residual.numel() != T * N:
            raise ValueError("residual must have the shape of the output")
        rr, Tr, ldr = _rows("residual", residual if residual.dim() == 2 else residual.reshape(-1, N), N)
        if Tr != T:
            raise ValueError("residual must have the shape of the output")
        mode = RES_AFTER_ACT if residual_after_activation else RES_BEFORE_ACT
    xe, we, ne, ldxe = None, None, 0, 0
    if x_extra is not None:
        require_gpu_f32("weight_extra_kn", weight_extra_kn)
        ne = weight_extra_kn.shape[0]
        if weight_extra_kn.shape[1] != N or x_extra.shape[-1] != ne or x_extra.numel() != T * ne:
            raise ValueError("x_extra must be [..., E] and weight_extra_kn [E, N]")
        require_gpu_f32("x_extra", x_extra, contiguous=False)
        xe, we, ldxe = x_extra.contiguous(), weight_extra_kn, ne
    if T == 0:
        return out
    with _lib.device_guard(x.device):
        check(_lib.load().spgt_linear_forward(
            ptr(xr), ldx, ptr(weight_kn), ptr(bias) if bias is not None else None,
            ptr(rr) if rr is not None else None, ldr, mode, ACTIVATIONS[activation],
            ptr(xe) if xe is not None else None, ldxe, ptr(we) if we is not None else None, ne, ptr(out), pc, pc,
            T * pc, T, K, N,
            stream_of(x)))
    return out


def ffn_scalar_supported(in_features: int, hidden_features: int) -> bool:
    """True when fused_ffn_scalar has a kernel for this shape."""
    return bool(_lib.load().spgt_ffn_scalar_supported(int(in_features), int(hidden_features)))


def fused_ffn_scalar(x: Tensor, weight1_kn: Tensor, bias1: Optional[Tensor], weight2: Tensor,
                     bias2: Optional[Tensor], activation: str) -> Tensor:
    """act(x @ weight1_kn + bias1) @ weight2 + bias2 for a single output feature, in one kernel.

    x [..., K], weight1_kn [K, HID] contiguous, weight2 [HID] (or [1, HID]), bias2 [1] -> [..., 1].
    """
    if activation not in ACTIVATIONS:
        raise ValueError(f"activation must be one of {sorted(ACTIVATIONS)}")
    require_gpu_f32("weight1_kn", weight1_kn)
    require_gpu_f32("weight2", weight2)
    K, HID = weight1_kn.shape
    if weight2.numel() != HID:
        raise ValueError(f"weight2 has {weight2.numel()} elements, expected {HID}")
    for name, b, n in (("bias1", bias1, HID), ("bias2", bias2, 1)):
        if b is not None:
            require_gpu_f32(name, b)
            if b.numel() != n:
                raise ValueError(f"{name} has {b.numel()} elements, expected {n}")
    xr, T, ldx = _rows("x", x, K)
    out = torch.empty(list(x.shape[:-1]) + [1], dtype=x.dtype, device=x.device)
    if T == 0:
        return out
    with _lib.device_guard(x.device):
        check(_lib.load().spgt_ffn_scalar_forward(
            ptr(xr), ldx, ptr(weight1_kn), ptr(bias1) if bias1 is not None else None, ptr(weight2),
            ptr(bias2) if bias2 is not None else None, ACTIVATIONS[activation], ptr(out), T, K, HID, stream_of(x)))
    return out


def encoder_tail_supported(attn_features: int, dim_hidden: int, ffn_hidden: int) -> bool:
    """True when fused_encoder_tail has a kernel for this shape."""
    return bool(_lib.load().spgt_encoder_tail_supported(int(attn_features), int(dim_hidden), int(ffn_hidden)))


def _dropout_args(x: Tensor, fc_droprate: float, ffn_droprate: float, seed):
    fc_droprate, ffn_droprate = float(fc_droprate), float(ffn_droprate)
    if not (0.0 <= fc_droprate < 1.0 and 0.0 <= ffn_droprate < 1.0):
        raise ValueError("drop rates must lie in [0, 1)")
    if fc_droprate == 0.0 and ffn_droprate == 0.0:
        return 0.0, 0.0, None
    if seed is None:
        seed = dropout_seed(x.device)
    if not (seed.is_cuda and seed.device == x.device and seed.dtype == torch.int32 and seed.numel() >= 2 and
            seed.is_contiguous()):
        raise ValueError("seed must be a contiguous int32 tensor of two words on x's device")
    return fc_droprate, ffn_droprate, seed


def fused_encoder_tail(attn_out: Tensor, x: Tensor, fc_weight_kn: Tensor, fc_bias: Tensor, ffn1_weight_kn: Tensor,
                       ffn1_bias: Tensor, ffn2_weight_kn: Tensor, ffn2_bias: Tensor, activation: str,
                       fc_droprate: float = 0.0, ffn_droprate: float = 0.0, seed: Optional[Tensor] = None) -> Tensor:
    """y1 = x + attn_out @ fc_weight_kn + fc_bias;  returns y1 + act(y1 @ ffn1_weight_kn + ffn1_bias) @ ffn2_weight_kn
    + ffn2_bias: the attention's output projection, both residual adds and the feed-forward net of an encoder layer
    in one kernel.  attn_out [..., K1], x [..., D]; weights [in, out] contiguous.
    With drop rates above 0 the two terms added to the residual stream are dropped first, as the reference's
    F.dropout calls do (masks from this library's own generator, seeded by `seed` or by dropout_seed)."""
    if activation not in ACTIVATIONS:
        raise ValueError(f"activation must be one of {sorted(ACTIVATIONS)}")
    for name, w in (("fc_weight_kn", fc_weight_kn), ("fc_bias", fc_bias), ("ffn1_weight_kn", ffn1_weight_kn),
                    ("ffn1_bias", ffn1_bias), ("ffn2_weight_kn", ffn2_weight_kn), ("ffn2_bias", ffn2_bias)):
        require_gpu_f32(name, w)
    K1, D = fc_weight_kn.shape
    F = ffn1_weight_kn.shape[1]
    if tuple(ffn1_weight_kn.shape) != (D, F) or tuple(ffn2_weight_kn.shape) != (F, D):
        raise ValueError("ffn weights must be [D, F] and [F, D]")
    if fc_bias.numel() != D or ffn1_bias.numel() != F or ffn2_bias.numel() != D:
        raise ValueError("bias sizes do not match the weights")
    ar, T, lda = _rows("attn_out", attn_out, K1)
    require_gpu_f32("x", x)
    if x.shape[-1] != D or x.numel() != T * D:
        raise ValueError("x must be [..., D] with as many rows as attn_out")
    out = torch.empty_like(x)
    if T == 0:
        return out
    fc_droprate, ffn_droprate, seed = _dropout_args(x, fc_droprate, ffn_droprate, seed)
    with _lib.device_guard(x.device):
        if seed is None:
            check(_lib.load().spgt_encoder_tail_forward(
                ptr(ar), lda, ptr(x), ptr(fc_weight_kn), ptr(fc_bias), ptr(ffn1_weight_kn), ptr(ffn1_bias),
                ptr(ffn2_weight_kn), ptr(ffn2_bias), ACTIVATIONS[activation], ptr(out), T, K1, D, F, stream_of(x)))
        else:
            check(_lib.load().spgt_encoder_tail_forward_dropout(
                ptr(ar), lda, ptr(x), ptr(fc_weight_kn), ptr(fc_bias), ptr(ffn1_weight_kn), ptr(ffn1_bias),
                ptr(ffn2_weight_kn), ptr(ffn2_bias), ACTIVATIONS[activation], ptr(out), T, K1, D, F, ptr(seed),
                fc_droprate, ffn_droprate, stream_of(x)))
    return out


def fused_encoder_tail_folded(q: Tensor, position, x: Tensor, folded_fc: Tensor, folded_pos, fc_bias: Tensor,
                              ffn1_weight_kn: Tensor, ffn1_bias: Tensor, ffn2_weight_kn: Tensor, ffn2_bias: Tensor,
                              activation: str, fc_droprate: float = 0.0, ffn_droprate: float = 0.0,
                              seed: Optional[Tensor] = None) -> Tensor:
    """fused_encoder_tail with the attention's last product folded into the output projection (see
    galerkin_attention.fold_ktv_into_fc): y1 = x + q @ folded_fc[b] + position @ folded_pos[b] + fc_bias, then the
    feed-forward net.  q [B, S, 128] (the projected Q; a column slice of the packed projection is fine),
    position [B, S, 2] or None, x [B, S, 128], folded_fc [B, 128, 128], folded_pos [B, 2, 128] or None."""
    if activation not in ACTIVATIONS:
        raise ValueError(f"activation must be one of {sorted(ACTIVATIONS)}")
    for name, w in (("folded_fc", folded_fc), ("fc_bias", fc_bias), ("ffn1_weight_kn", ffn1_weight_kn),
                    ("ffn1_bias", ffn1_bias), ("ffn2_weight_kn", ffn2_weight_kn), ("ffn2_bias", ffn2_bias), ("x", x)):
        require_gpu_f32(name, w)
    require_gpu_f32("q", q, contiguous=False)
    if q.dim() != 3 or x.dim() != 3 or q.shape != x.shape or q.shape[-1] != 128:
        raise ValueError("q and x must be [B, S, 128]")
    B, S, D = x.shape
    ld = q.stride(1)
    if q.stride(2) != 1 or ld < D or ld % 4 or (B > 1 and q.stride(0) != S * ld) or q.data_ptr() % 16:
        raise ValueError("q must have unit stride on the last axis, one row stride (a multiple of 4) and 16-byte alignment")
    F = ffn1_weight_kn.shape[1]
    if tuple(folded_fc.shape) != (B, D, D) or tuple(ffn1_weight_kn.shape) != (D, F) or tuple(ffn2_weight_kn.shape) != (F, D):
        raise ValueError("folded_fc must be [B, 128, 128], the ffn weights [128, F] and [F, 128]")
    if fc_bias.numel() != D or ffn1_bias.numel() != F or ffn2_bias.numel() != D:
        raise ValueError("bias sizes do not match the weights")
    dp = 0
    if folded_pos is not None:
        require_gpu_f32("folded_pos", folded_pos)
        require_gpu_f32("position", position)
        dp = 2
        if tuple(folded_pos.shape) != (B, 2, D) or tuple(position.shape) != (B, S, 2):
            raise ValueError("folded_pos must be [B, 2, 128] and position [B, S, 2]")
    out = torch.empty_like(x)
    if out.numel() == 0:
        return out
    fc_droprate, ffn_droprate, seed = _dropout_args(x, fc_droprate, ffn_droprate, seed)
    with _lib.device_guard(x.device):
        if seed is None:
            check(_lib.load().spgt_encoder_tail_folded_forward(
                ptr(q), ld, ptr(position) if dp else None, ptr(x), ptr(folded_fc), ptr(folded_pos) if dp else None,
                ptr(fc_bias), ptr(ffn1_weight_kn), ptr(ffn1_bias), ptr(ffn2_weight_kn), ptr(ffn2_bias),
                ACTIVATIONS[activation], ptr(out), B, S, dp, D, F, stream_of(x)))
        else:
            check(_lib.load().spgt_encoder_tail_folded_forward_dropout(
                ptr(q), ld, ptr(position) if dp else None, ptr(x), ptr(folded_fc), ptr(folded_pos) if dp else None,
                ptr(fc_bias), ptr(ffn1_weight_kn), ptr(ffn1_bias), ptr(ffn2_weight_kn), ptr(ffn2_bias),
                ACTIVATIONS[activation], ptr(out), B, S, dp, D, F, ptr(seed), fc_droprate, ffn_droprate, stream_of(x)))
    return out


def linear_weight_grad(x: Tensor, grad: Tensor):
    """(dW [in, out], db [out]) of y = x @ W + b from dL/dy: dW = x^T grad and db = column sums of grad over all
    leading dimensions, in one pass over x and grad with a fixed summation order (reference:
    extension/bind/galerkin_attention.cu:41-46).  x [..., in], grad [..., out], out a multiple of 4."""
    K, N = x.shape[-1], grad.shape[-1]
    xr, T, ldx = _rows("x", x, K)
    gr, Tg, ldg = _rows("grad", grad, N)
    if T != Tg:
        raise ValueError(f"x has {T} rows and grad {Tg}")
    lib = _lib.load()
    nbytes = lib.spgt_linear_weight_grad_workspace_bytes(T, K, N, 1)
    if nbytes == 0:
        raise ValueError(f"unsupported weight-gradient shape: tokens={T} in={K} out={N} (out must be a multiple of 4)")
    ws = _lib.workspace(nbytes, xr)
    out = torch.empty(K * N + N, dtype=torch.float32, device=xr.device)
    with _lib.device_guard(xr.device):
        check(lib.spgt_linear_weight_grad(ptr(xr), ldx, 0, ptr(gr), ldg, 0, ptr(out), ptr(ws), ws.numel(), T, K, N, 1,
                                          stream_of(xr)))
    return out[:K * N].view(K, N), out[K * N:]


def linear_weight_grad_batched(x: Tensor, grads: Tensor):
    """The same for several gradient planes against one input in one call: x [..., in], grads [P, ..., out]
    (contiguous planes) -> (dW [P, in, out], db [P, out]).  The backward of a packed projection such as
    [W_Q | W_K | W_V], whose three outputs are separate planes."""
    K, N, P = x.shape[-1], grads.shape[-1], grads.shape[0]
    xr, T, ldx = _rows("x", x, K)
    require_gpu_f32("grads", grads)
    if grads.numel() != P * T * N:
        raise ValueError(f"grads has {grads.numel()} elements, expected {P} planes of {T} x {N}")
    lib = _lib.load()
    nbytes = lib.spgt_linear_weight_grad_workspace_bytes(T, K, N, P)
    if nbytes == 0:
        raise ValueError(f"unsupported weight-gradient shape: tokens={T} in={K} out={N} (out must be a multiple of 4)")
    ws = _lib.workspace(nbytes, xr)
    out = torch.empty((P, K * N + N), dtype=torch.float32, device=xr.device)
    with _lib.device_guard(xr.device):
        check(lib.spgt_linear_weight_grad(ptr(xr), ldx, 0, ptr(grads), N, T * N, ptr(out), ptr(ws), ws.numel(), T, K, N,
                                          P, stream_of(xr)))
    return out[:, :K * N].view(P, K, N), out[:, K * N:]


def dropout_add(y: Tensor, residual: Optional[Tensor], droprate: float, seed: Tensor, site: int = 5) -> Tensor:
    """residual + dropout(y, droprate) (or dropout(y) alone) on [..., C], C a multiple of 4, in one pass with the
    library's own masks: a hash of (seed, site, row, column).  Called on a gradient with the forward's seed it is
    the dropout's backward.  seed: two int32 words on y's device (_lib.dropout_seed)."""
    require_gpu_f32("y", y)
    C = y.shape[-1]
    if C % 4:
        raise ValueError("the last dimension must be a multiple of 4")
    if residual is not None:
        require_gpu_f32("residual", residual)
        if residual.shape != y.shape:
            raise ValueError("residual must have y's shape")
    if not (seed.is_cuda and seed.device == y.device and seed.dtype == torch.int32 and seed.numel() >= 2):
        raise ValueError("seed must be an int32 tensor of two words on y's device")
    out = torch.empty_like(y)
    if y.numel() == 0:
        return out
    with _lib.device_guard(y.device):
        check(_lib.load().spgt_dropout_add(ptr(y), ptr(residual) if residual is not None else None, ptr(out),
                                           y.numel() // C, C, ptr(seed), float(droprate), int(site), stream_of(y)))
    return out
