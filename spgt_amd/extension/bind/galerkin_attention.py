"""Operator API of the Galerkin attention path, backed by libspgt_hip.so.

Same function names, argument order and result layouts as the reference's
extension/bind/galerkin_attention.py:87-107 (python surface) and
extension/bind/galerkin_attention.cu:200-226 (the `gexts` module surface).
Tensors must be fp32, contiguous and on a GPU; anything else raises.
"""
from types import SimpleNamespace
from typing import Any

import torch
from torch import Tensor

from ... import _lib
from ..._lib import check, ptr, require_gpu_f32, stream_of, workspace
from .linear import linear_weight_grad

GEMM_ORDER = {"RRR": 0, "RRC": 1, "RCR": 2, "RCC": 3, "CRR": 4, "CRC": 5, "CCR": 6, "CCC": 7}


# --------------------------------------------------------------------------- #
# `gexts` surface: plain functions on tensors, no autograd
# --------------------------------------------------------------------------- #

def _check_projection_args(input, weight, bias, position, seqlen, dim_hidden, num_head, dim_head, dim_position, batch):
    require_gpu_f32("input", input)
    require_gpu_f32("weight", weight)
    require_gpu_f32("bias", bias)
    if tuple(input.shape) != (batch, seqlen, dim_hidden):
        raise ValueError(f"input has shape {tuple(input.shape)}, expected {(batch, seqlen, dim_hidden)}")
    if tuple(weight.shape) != (dim_hidden, dim_hidden) or bias.numel() != dim_hidden:
        raise ValueError("weight must be [dim_hidden, dim_hidden] and bias [dim_hidden]")
    if num_head * dim_head != dim_hidden:
        raise ValueError("num_head * dim_head must equal dim_hidden")
    if dim_position:
        require_gpu_f32("position", position)
        if tuple(position.shape) != (batch, seqlen, dim_position):
            raise ValueError(f"position has shape {tuple(position.shape)}, expected {(batch, seqlen, dim_position)}")


def _projection_forward(input: Tensor, weight: Tensor, bias: Tensor, position: Tensor, seqlen: int, dim_hidden: int,
                        num_head: int, dim_head: int, dim_position: int, batch: int) -> Tensor:
    """x @ W + b split into heads, position rows first -> [batch, num_head, dim_position + dim_head, seqlen]
    (reference: extension/bind/galerkin_attention.cu:9-24)."""
    _check_projection_args(input, weight, bias, position, seqlen, dim_hidden, num_head, dim_head, dim_position, batch)
    out = torch.empty((batch, num_head, dim_position + dim_head, seqlen), dtype=input.dtype, device=input.device)
    with _lib.device_guard(input.device):
        check(_lib.load().spgt_multihead_projection_with_position_rrc_forward(
            ptr(input), ptr(weight), ptr(bias), ptr(position) if dim_position else None, ptr(out), seqlen, dim_hidden,
            num_head, dim_head, dim_position, batch, stream_of(input)))
    return out


def _projection_layernorm_forward(input: Tensor, weight: Tensor, bias: Tensor, lnw: Tensor, lnb: Tensor,
                                  norm_eps: float, position: Tensor, seqlen: int, dim_hidden: int, num_head: int,
                                  dim_head: int, dim_position: int, batch: int):
    """As above with per-head LayerNorm; returns (hat_ln, invsigma [batch, num_head, seqlen])
    (reference: extension/bind/galerkin_attention.cu:50-68)."""
    _check_projection_args(input, weight, bias, position, seqlen, dim_hidden, num_head, dim_head, dim_position, batch)
    require_gpu_f32("lnw", lnw)
    require_gpu_f32("lnb", lnb)
    if lnw.numel() != dim_hidden or lnb.numel() != dim_hidden:
        raise ValueError("LayerNorm weight and bias must be [num_head, dim_head]")
    hat_ln = torch.empty((batch, num_head, dim_position + dim_head, seqlen), dtype=input.dtype, device=input.device)
    invsigma = torch.empty((batch, num_head, seqlen), dtype=input.dtype, device=input.device)
    with _lib.device_guard(input.device):
        check(_lib.load().spgt_multihead_projection_layernorm_with_position_rrc_forward(
            ptr(input), ptr(weight), ptr(bias), ptr(lnw), ptr(lnb), float(norm_eps),
            ptr(position) if dim_position else None, ptr(hat_ln), ptr(invsigma), seqlen, dim_hidden, num_head,
            dim_head, dim_position, batch, stream_of(input)))
    return hat_ln, invsigma


def _attention_cccr_forward(Q: Tensor, K: Tensor, V: Tensor, batch: int, num_head: int, d_posk: int,
                            seqlen: int) -> Tensor:
    """Q, K, V [batch, num_head, d_posk, seqlen] -> [batch, num_head, seqlen, d_posk]
    (reference: extension/bind/galerkin_attention.cu:104-124)."""
    for name, t in (("Q", Q), ("K", K), ("V", V)):
        require_gpu_f32(name, t)
        if tuple(t.shape) != (batch, num_head, d_posk, seqlen):
            raise ValueError(f"{name} has shape {tuple(t.shape)}, expected {(batch, num_head, d_posk, seqlen)}")
    lib = _lib.load()
    out = torch.empty((batch, num_head, seqlen, d_posk), dtype=Q.dtype, device=Q.device)
    nbytes = lib.spgt_galerkin_attention_cccr_workspace_bytes(batch, num_head, d_posk, seqlen)
    if nbytes == 0:
        raise ValueError(f"unsupported attention shape: batch={batch} num_head={num_head} d_posk={d_posk} "
                         f"seqlen={seqlen} (d_posk must be 32 or 34)")
    ws = workspace(nbytes, Q)
    with _lib.device_guard(Q.device):
        check(lib.spgt_galerkin_attention_cccr_forward(
            ptr(Q), ptr(K), ptr(V), ptr(out), ptr(ws), ws.numel(), batch, num_head, d_posk, seqlen, stream_of(Q)))
    return out


def _attention_cccr_backward(grad_out: Tensor, Q: Tensor, K: Tensor, V: Tensor, batch: int, num_head: int,
                             d_posk: int, seqlen: int):
    """grad_out [batch, num_head, seqlen, d_posk] -> (dQ, dK, dV), each [batch, num_head, d_posk, seqlen]
    (reference: extension/bind/galerkin_attention.cu:126-173)."""
    grad_out = grad_out.contiguous()
    require_gpu_f32("grad_out", grad_out)
    if tuple(grad_out.shape) != (batch, num_head, seqlen, d_posk):
        raise ValueError(f"grad_out has shape {tuple(grad_out.shape)}, expected {(batch, num_head, seqlen, d_posk)}")
    for name, t in (("Q", Q), ("K", K), ("V", V)):
        require_gpu_f32(name, t)
        if tuple(t.shape) != (batch, num_head, d_posk, seqlen):
            raise ValueError(f"{name} has shape {tuple(t.shape)}, expected {(batch, num_head, d_posk, seqlen)}")
    lib = _lib.load()
    dQ, dK, dV = torch.empty_like(Q), torch.empty_like(K), torch.empty_like(V)
    nbytes = lib.spgt_galerkin_attention_cccr_backward_workspace_bytes(batch, num_head, d_posk, seqlen)
    if nbytes == 0:
        raise ValueError("unsupported attention shape (d_posk must be 32 or 34)")
    ws = workspace(nbytes, Q)
    with _lib.device_guard(Q.device):
        check(lib.spgt_galerkin_attention_cccr_backward(
            ptr(grad_out), ptr(Q), ptr(K), ptr(V), ptr(dQ), ptr(dK), ptr(dV), ptr(ws), ws.numel(), batch, num_head,
            d_posk, seqlen, stream_of(Q)))
    return dQ, dK, dV


def _heads_feature_to_token_major(src: Tensor, batch: int, num_head: int, dim_position: int, dim_head: int,
                                  seqlen: int) -> Tensor:
    """[batch, num_head, dim_position + dim_head, seqlen] -> [batch, seqlen, num_head * dim_head]
    (reference: datamove::batched_transpose_gather, extension/native/datamove.cu:121-163)."""
    src = src.contiguous()
    require_gpu_f32("src", src)
    if tuple(src.shape) != (batch, num_head, dim_position + dim_head, seqlen):
        raise ValueError(f"src has shape {tuple(src.shape)}")
    dst = torch.empty((batch, seqlen, num_head * dim_head), dtype=src.dtype, device=src.device)
    with _lib.device_guard(src.device):
        check(_lib.load().spgt_heads_feature_to_token_major(ptr(src), ptr(dst), batch, num_head, dim_position,
                                                            dim_head, seqlen, stream_of(src)))
    return dst


def _linear_backward(grad_tm: Tensor, input: Tensor, weight: Tensor):
    """Gradients of y = x @ W + b given dL/dy token-major (reference: extension/bind/galerkin_attention.cu:41-46):
    dX by a library GEMM, dW and db by this package's split-over-tokens kernel."""
    grad_input = torch.matmul(grad_tm, weight.t())
    # x^T g over hundreds of thousands of tokens and the column sums of g: one pass, fixed summation order
    grad_weight, grad_bias = linear_weight_grad(input, grad_tm)
    return grad_input, grad_weight, grad_bias


def _projection_backward(grad_out: Tensor, input: Tensor, weight: Tensor, seqlen: int, dim_hidden: int, num_head: int,
                         dim_head: int, dim_position: int, batch: int):
    """-> (dX, dW, db) (reference: extension/bind/galerkin_attention.cu:26-48)."""
    g = _heads_feature_to_token_major(grad_out, batch, num_head, dim_position, dim_head, seqlen)
    return _linear_backward(g, input, weight)


def _projection_layernorm_backward_from_output(grad_ln: Tensor, input: Tensor, weight: Tensor, hat_ln: Tensor,
                                               invsigma: Tensor, lnw: Tensor, lnb: Tensor, seqlen: int,
                                               dim_hidden: int, num_head: int, dim_head: int, dim_position: int,
                                               batch: int):
    """-> (dX, dW, db, dgamma, dbeta) with the reference's own arguments
    (extension/bind/galerkin_attention.cu:70-102; extension/native/multihead_dim32.cu:148-271): the normalised
    values are recovered from the saved LayerNorm output as x_hat = (hat_ln - beta) / gamma and the reciprocal
    standard deviations are taken from invsigma [batch, num_head, seqlen].  Where a gamma is zero x_hat cannot be
    recovered: the reference divides by zero there, this function uses x_hat = 0 (exact for dgamma's other entries,
    dbeta, and the part of dX, dW, db that does not pass through that feature's x_hat).  The autograd function of
    this package uses the recomputing form below instead and has no such case."""
    for name, t in (("hat_ln", hat_ln), ("invsigma", invsigma), ("lnw", lnw), ("lnb", lnb)):
        require_gpu_f32(name, t)
    if tuple(invsigma.shape) != (batch, num_head, seqlen):
        raise ValueError(f"invsigma has shape {tuple(invsigma.shape)}, expected {(batch, num_head, seqlen)}")
    g = _heads_feature_to_token_major(grad_ln, batch, num_head, dim_position, dim_head, seqlen)
    y = _heads_feature_to_token_major(hat_ln, batch, num_head, dim_position, dim_head, seqlen)
    g = g.view(batch, seqlen, num_head, dim_head)
    y = y.view(batch, seqlen, num_head, dim_head)
    gamma, beta = lnw.view(1, 1, num_head, dim_head), lnb.view(1, 1, num_head, dim_head)
    x_hat = torch.where(gamma != 0, (y - beta) / torch.where(gamma != 0, gamma, torch.ones_like(gamma)),
                        torch.zeros_like(y))
    dxh = g * gamma
    inv = invsigma.permute(0, 2, 1).unsqueeze(-1)  # [batch, seqlen, num_head, 1]
    grad_pre = inv * (dxh - dxh.mean(-1, keepdim=True) - x_hat * (dxh * x_hat).mean(-1, keepdim=True))
    grad_lnw = (g * x_hat).sum(dim=(0, 1))
    grad_lnb = g.sum(dim=(0, 1))
    grad_input, grad_weight, grad_bias = _linear_backward(grad_pre.reshape(batch, seqlen, dim_hidden), input, weight)
    return grad_input, grad_weight, grad_bias, grad_lnw, grad_lnb


def _projection_layernorm_backward(grad_ln: Tensor, input: Tensor, weight: Tensor, bias: Tensor, lnw: Tensor,
                                   norm_eps: float, seqlen: int, dim_hidden: int, num_head: int, dim_head: int,
                                   dim_position: int, batch: int):
    """-> (dX, dW, db, dgamma, dbeta): what the autograd function of this package calls.

    Unlike the reference (see _projection_layernorm_backward_from_output), which recovers x_hat from the saved
    LayerNorm output as (y - beta) / gamma and therefore fails when a gamma is zero, the pre-LayerNorm projection
    is recomputed from input, weight and bias; that is why `bias` and `norm_eps` are arguments here and hat_ln /
    invsigma are not."""
    require_gpu_f32("lnw", lnw)
    g = _heads_feature_to_token_major(grad_ln, batch, num_head, dim_position, dim_head, seqlen)
    pre = torch.addmm(bias, input.reshape(-1, dim_hidden), weight)
    lib = _lib.load()
    tokens = batch * seqlen
    grad_pre = torch.empty_like(pre)
    grad_lnw = torch.empty((num_head, dim_head), dtype=pre.dtype, device=pre.device)
    grad_lnb = torch.empty((num_head, dim_head), dtype=pre.dtype, device=pre.device)
    ws = workspace(lib.spgt_layernorm_heads_backward_workspace_bytes(tokens, num_head), pre)
    with _lib.device_guard(pre.device):
        check(lib.spgt_layernorm_heads_backward(
            ptr(pre), ptr(g), ptr(lnw), float(norm_eps), ptr(grad_pre), ptr(grad_lnw), ptr(grad_lnb), ptr(ws),
            ws.numel(), tokens, num_head, stream_of(pre)))
    grad_input, grad_weight, grad_bias = _linear_backward(grad_pre.view(batch, seqlen, dim_hidden), input, weight)
    return grad_input, grad_weight, grad_bias, grad_lnw, grad_lnb


def _batched_skinny_gemm(A: Tensor, B: Tensor, alpha: float) -> Tensor:
    """A [..., M, K] @ B [..., K, N] * alpha, all row-major
    (reference: extension/bind/galerkin_attention.cu:175-198)."""
    require_gpu_f32("A", A)
    require_gpu_f32("B", B)
    if A.dim() < 2 or A.dim() != B.dim() or A.shape[:-2] != B.shape[:-2] or A.shape[-1] != B.shape[-2]:
        raise ValueError(f"incompatible shapes {tuple(A.shape)} and {tuple(B.shape)}")
    M, K = A.shape[-2], A.shape[-1]
    N = B.shape[-1]
    lead = tuple(A.shape[:-2])
    batch = 1
    for n in lead:
        batch *= n
    C = torch.empty(lead + (M, N), dtype=A.dtype, device=A.device)
    if batch == 0 or M == 0 or N == 0:
        return C
    if K == 0:
        return C.zero_()
    lib = _lib.load()
    ws = workspace(lib.spgt_batched_skinny_gemm_workspace_bytes(M, N, K, batch), A)
    with _lib.device_guard(A.device):
        check(lib.spgt_batched_skinny_gemm(
            ptr(A), ptr(B), ptr(C), float(alpha), M, N, K, M * K, K * N, M * N, GEMM_ORDER["RRR"], batch,
            ptr(ws), ws.numel(), stream_of(A)))
    return C


def _attention_fused_forward(QKV_or_Q, K, V, position, ln_weight_K, ln_bias_K, ln_weight_V, ln_bias_V,
                             norm_eps: float, num_head: int, dim_position: int, return_ktv: bool = False):
    """Token-major fused attention core (no reference counterpart as one call).

    Either pass Q, K, V as three [B, S, H*32] tensors (contiguous, or equal-stride
    column slices of one [B, S, 3*H*32] projection output), position [B, S, dp].
    Returns out [B, S, H*(dp+32)] (and K'^T V'/S [B, H, d, d] if return_ktv).
    """
    Q = QKV_or_Q
    H = num_head
    for name, t in (("Q", Q), ("K", K), ("V", V)):
        if not t.is_cuda:
            raise _lib.SpgtError(f"{name} must live on a GPU; there is no CPU implementation")
        if t.dtype != torch.float32:
            raise TypeError(f"{name} must be float32")
        if t.dim() != 3 or t.shape[-1] != H * 32 or t.stride(-1) != 1:
            raise ValueError(f"{name} must be [B, S, {H * 32}] with unit stride on the last axis")
    B, S, _ = Q.shape
    ld = Q.stride(1)
    for name, t in (("Q", Q), ("K", K), ("V", V)):
        if tuple(t.shape) != (B, S, H * 32) or t.stride(1) != ld or (B > 1 and t.stride(0) != S * ld):
            raise ValueError(f"{name}: all of Q, K, V must share shape and strides [S*ld, ld, 1]")
    for name, t in (("ln_weight_K", ln_weight_K), ("ln_bias_K", ln_bias_K), ("ln_weight_V", ln_weight_V),
                    ("ln_bias_V", ln_bias_V)):
        require_gpu_f32(name, t)
        if t.numel() != H * 32:
            raise ValueError(f"{name} must have {H * 32} elements")
    if dim_position not in (0, 2):
        raise ValueError("dim_position must be 0 or 2")
    if dim_position == 2:
        require_gpu_f32("position", position)
        if tuple(position.shape) != (B, S, 2):
            raise ValueError(f"position must be [{B}, {S}, 2]")
    D = dim_position + 32
    lib = _lib.load()
    out = torch.empty((B, S, H * D), dtype=torch.float32, device=Q.device)
    ktv = torch.empty((B, H, D, D), dtype=torch.float32, device=Q.device)
    ws = workspace(lib.spgt_galerkin_attention_fused_workspace_bytes(B, S, H, dim_position), Q)
    pos_ptr = ptr(position) if dim_position == 2 else None
    with _lib.device_guard(Q.device):
        check(lib.spgt_galerkin_attention_fused_forward(
            ptr(Q), ptr(K), ptr(V), ld, pos_ptr, ptr(ln_weight_K), ptr(ln_bias_K), ptr(ln_weight_V),
            ptr(ln_bias_V), float(norm_eps), ptr(out), ptr(ktv), ptr(ws), ws.numel(), B, S, H, dim_position,
            stream_of(Q)))
    return (out, ktv) if return_ktv else out


def _attention_fused_backward(grad_out, Q, K, V, position, ln_weight_K, ln_bias_K, ln_weight_V, ln_bias_V,
                              norm_eps: float, ktv, num_head: int, dim_position: int):
    """Backward of _attention_fused_forward on the same operands: grad_out [B, S, H*(dp+32)] ->
    (dQ, dK, dV [B, S, H*32] w.r.t. the plain projections, d ln_weight_K, d ln_bias_K, d ln_weight_V, d ln_bias_V
    [H, 32]) (reference: extension/bind/galerkin_attention.cu:126-173, extension/native/multihead_dim32.cu:148-271)."""
    H = num_head
    D = dim_position + 32
    B, S, _ = Q.shape
    ld = Q.stride(1)
    for name, t in (("Q", Q), ("K", K), ("V", V)):
        require_gpu_f32(name, t, contiguous=False)
        if tuple(t.shape) != (B, S, H * 32) or t.stride(2) != 1 or t.stride(1) != ld or (B > 1 and t.stride(0) != S * ld):
            raise ValueError(f"{name}: Q, K, V must share shape [B, S, {H * 32}] and strides [S*ld, ld, 1]")
    grad_out = grad_out.contiguous()
    require_gpu_f32("grad_out", grad_out)
    if tuple(grad_out.shape) != (B, S, H * D):
        raise ValueError(f"grad_out has shape {tuple(grad_out.shape)}, expected {(B, S, H * D)}")
    require_gpu_f32("ktv", ktv)
    if tuple(ktv.shape) != (B, H, D, D):
        raise ValueError(f"ktv has shape {tuple(ktv.shape)}, expected {(B, H, D, D)}")
    for name, t in (("ln_weight_K", ln_weight_K), ("ln_bias_K", ln_bias_K), ("ln_weight_V", ln_weight_V),
                    ("ln_bias_V", ln_bias_V)):
        require_gpu_f32(name, t)
        if t.numel() != H * 32:
            raise ValueError(f"{name} must have {H * 32} elements")
    if dim_position == 2:
        require_gpu_f32("position", position)
        if tuple(position.shape) != (B, S, 2):
            raise ValueError(f"position must be [{B}, {S}, 2]")
    lib = _lib.load()
    nbytes = lib.spgt_galerkin_attention_fused_backward_workspace_bytes(B, S, H, dim_position)
    if nbytes == 0:
        raise ValueError("unsupported shape: num_head must be a multiple of 4, dim_position 0 or 2")
    ws = workspace(nbytes, Q)
    grads = torch.empty((3, B, S, H * 32), dtype=torch.float32, device=Q.device)
    grad_ln = torch.empty((4, H, 32), dtype=torch.float32, device=Q.device)
    with _lib.device_guard(Q.device):
        check(lib.spgt_galerkin_attention_fused_backward(
            ptr(grad_out), ptr(Q), ptr(K), ptr(V), ld, ptr(position) if dim_position == 2 else None,
            ptr(ln_weight_K), ptr(ln_bias_K), ptr(ln_weight_V), ptr(ln_bias_V), float(norm_eps), ptr(ktv),
            ptr(grads[0]), ptr(grads[1]), ptr(grads[2]), H * 32, ptr(grad_ln), ptr(ws), ws.numel(), B, S, H,
            dim_position, stream_of(Q)))
    return grads[0], grads[1], grads[2], grad_ln[0], grad_ln[1], grad_ln[2], grad_ln[3]


def _attention_ktv_forward(K, V, position, ln_weight_K, ln_bias_K, ln_weight_V, ln_bias_V, norm_eps: float,
                           num_head: int, dim_position: int):
    """K'^T V' / S [B, H, d, d] of the fused attention core (K/V pass and tile reduction, no pass over Q):
    K, V [B, S, H*32] (contiguous, or equal-stride column slices of one projection output), position [B, S, dp]."""
    H = num_head
    for name, t in (("K", K), ("V", V)):
        if not t.is_cuda:
            raise _lib.SpgtError(f"{name} must live on a GPU; there is no CPU implementation")
        if t.dtype != torch.float32:
            raise TypeError(f"{name} must be float32")
        if t.dim() != 3 or t.shape[-1] != H * 32 or t.stride(-1) != 1:
            raise ValueError(f"{name} must be [B, S, {H * 32}] with unit stride on the last axis")
    B, S, _ = K.shape
    ld = K.stride(1)
    for name, t in (("K", K), ("V", V)):
        if tuple(t.shape) != (B, S, H * 32) or t.stride(1) != ld or (B > 1 and t.stride(0) != S * ld):
            raise ValueError(f"{name}: K and V must share shape and strides [S*ld, ld, 1]")
    for name, t in (("ln_weight_K", ln_weight_K), ("ln_bias_K", ln_bias_K), ("ln_weight_V", ln_weight_V),
                    ("ln_bias_V", ln_bias_V)):
        require_gpu_f32(name, t)
        if t.numel() != H * 32:
            raise ValueError(f"{name} must have {H * 32} elements")
    if dim_position not in (0, 2):
        raise ValueError("dim_position must be 0 or 2")
    if dim_position == 2:
        require_gpu_f32("position", position)
        if tuple(position.shape) != (B, S, 2):
            raise ValueError(f"position must be [{B}, {S}, 2]")
    D = dim_position + 32
    lib = _lib.load()
    ktv = torch.empty((B, H, D, D), dtype=torch.float32, device=K.device)
    ws = workspace(lib.spgt_galerkin_attention_fused_workspace_bytes(B, S, H, dim_position), K)
    with _lib.device_guard(K.device):
        check(lib.spgt_galerkin_attention_ktv_forward(
            ptr(K), ptr(V), ld, ptr(position) if dim_position == 2 else None, ptr(ln_weight_K), ptr(ln_bias_K),
            ptr(ln_weight_V), ptr(ln_bias_V), float(norm_eps), ptr(ktv), ptr(ws), ws.numel(), B, S, H, dim_position,
            stream_of(K)))
    return ktv


def _fold_ktv_into_fc(ktv, fc_weight_kn, dim_position: int):
    """(folded [B, H*32, N], folded_pos [B, dp, N] or None): M_h Wfc_h per head with the rows arranged for
    fused_encoder_tail_folded; ktv [B, H, d, d], fc_weight_kn [H*d, N] (the transposed fc_layer weight)."""
    require_gpu_f32("ktv", ktv)
    require_gpu_f32("fc_weight_kn", fc_weight_kn)
    B, H, D, D2 = ktv.shape
    if D != D2 or D != dim_position + 32 or dim_position not in (0, 2):
        raise ValueError("ktv must be [B, H, dp + 32, dp + 32] with dp 0 or 2")
    if fc_weight_kn.dim() != 2 or fc_weight_kn.shape[0] != H * D:
        raise ValueError(f"fc_weight_kn must be [{H * D}, N]")
    N = fc_weight_kn.shape[1]
    folded = torch.empty((B, H * 32, N), dtype=torch.float32, device=ktv.device)
    folded_pos = torch.empty((B, dim_position, N), dtype=torch.float32, device=ktv.device) if dim_position else None
    with _lib.device_guard(ktv.device):
        check(_lib.load().spgt_fold_ktv_into_fc(ptr(ktv), ptr(fc_weight_kn), ptr(folded),
                                                ptr(folded_pos) if folded_pos is not None else None, B, H,
                                                dim_position, N, stream_of(ktv)))
    return folded, folded_pos


def _attention_fused_profile(input_sets, position, ln_weight_K, ln_bias_K, ln_weight_V, ln_bias_V, norm_eps: float,
                             num_head: int, dim_position: int, iterations: int):
    """Per-iteration milliseconds [iterations][3] of the three launches of the fused attention core (K/V pass,
    tile reduction, Q pass) over `iterations` back-to-back calls, iteration i on input_sets[i % len(input_sets)]
    (a list of (Q, K, V) triples of one shape) and writing an output buffer of its own per set, measured with HIP
    events on the current stream."""
    import ctypes
    Q0 = input_sets[0][0]
    B, S, _ = Q0.shape
    H, D = num_head, dim_position + 32
    for trip in input_sets:
        for t in trip:
            require_gpu_f32("profile input", t)
            if t.shape != Q0.shape:
                raise ValueError("all profile inputs must share one shape")
    lib = _lib.load()
    n = len(input_sets)
    outs = [torch.empty((B, S, H * D), dtype=torch.float32, device=Q0.device) for _ in range(n)]
    ktv = torch.empty((B, H, D, D), dtype=torch.float32, device=Q0.device)
    ws = workspace(lib.spgt_galerkin_attention_fused_workspace_bytes(B, S, H, dim_position), Q0)
    arrs = [(ctypes.c_void_p * n)(*[trip[j].data_ptr() for trip in input_sets]) for j in range(3)]
    out_arr = (ctypes.c_void_p * n)(*[o.data_ptr() for o in outs])
    stage = (ctypes.c_float * (3 * int(iterations)))()
    with _lib.device_guard(Q0.device):
        check(lib.spgt_galerkin_attention_fused_profile(
            arrs[0], arrs[1], arrs[2], out_arr, n, Q0.stride(1), ptr(position) if dim_position == 2 else None,
            ptr(ln_weight_K), ptr(ln_bias_K), ptr(ln_weight_V), ptr(ln_bias_V), float(norm_eps), ptr(ktv),
            ptr(ws), ws.numel(), B, S, H, dim_position, stream_of(Q0), int(iterations), stage))
    return [[float(stage[3 * i + k]) for k in range(3)] for i in range(int(iterations))]


gexts = SimpleNamespace(
    multihead_projection_with_position_rrc_forward=_projection_forward,
    multihead_projection_with_position_rrc_backward=_projection_backward,
    multihead_projection_layernorm_with_position_rrc_forward=_projection_layernorm_forward,
    multihead_projection_layernorm_with_position_rrc_backward=_projection_layernorm_backward_from_output,
    multihead_projection_layernorm_with_position_rrc_backward_recompute=_projection_layernorm_backward,
    multihead_galerkin_attention_cccr_backward=_attention_cccr_backward,
    heads_feature_to_token_major=_heads_feature_to_token_major,
    galerkin_attention_fused_profile=_attention_fused_profile,
    galerkin_attention_ktv_forward=_attention_ktv_forward,
    fold_ktv_into_fc=_fold_ktv_into_fc,
    multihead_galerkin_attention_cccr_forward=_attention_cccr_forward,
    batched_skinny_gemm=_batched_skinny_gemm,
    galerkin_attention_fused_forward=_attention_fused_forward,
    galerkin_attention_fused_backward=_attention_fused_backward,
)


# --------------------------------------------------------------------------- #
# python surface
# --------------------------------------------------------------------------- #

class Multihead_Porjection_with_Position_Function(torch.autograd.Function):
    @staticmethod
    def forward(ctx: Any, input: Tensor, weight: Tensor, bias: Tensor, position: Tensor, num_head, dim_head,
                dim_position):
        batch, seqlen, d_model = input.size()
        out = gexts.multihead_projection_with_position_rrc_forward(
            input, weight, bias, position, seqlen, d_model, num_head, dim_head, dim_position, batch)
        ctx.save_for_backward(input, weight)
        ctx.shape_kwargs = [num_head, dim_head, dim_position]
        return out

    @staticmethod
    def backward(ctx: Any, grad_out: Tensor):
        input, weight = ctx.saved_tensors
        num_head, dim_head, dim_position = ctx.shape_kwargs
        batch, seqlen, d_model = input.size()
        grad_input, grad_weight, grad_bias = gexts.multihead_projection_with_position_rrc_backward(
            grad_out, input, weight, seqlen, d_model, num_head, dim_head, dim_position, batch)
        return grad_input, grad_weight, grad_bias, None, None, None, None


class Multihead_Porjection_Layernorm_with_Position_Function(torch.autograd.Function):
    @staticmethod
    def forward(ctx: Any, input: Tensor, weight: Tensor, bias: Tensor, lnw: Tensor, lnb: Tensor, position: Tensor,
                norm_eps: float, num_head, dim_head, dim_position):
        batch, seqlen, d_model = input.size()
        hat_ln, invsigma = gexts.multihead_projection_layernorm_with_position_rrc_forward(
            input, weight, bias, lnw, lnb, norm_eps, position, seqlen, d_model, num_head, dim_head, dim_position,
            batch)
        ctx.save_for_backward(input, weight, bias, lnw)
        ctx.shape_kwargs = [num_head, dim_head, dim_position]
        ctx.norm_eps = norm_eps
        return hat_ln

    @staticmethod
    def backward(ctx: Any, grad_ln: Tensor):
        input, weight, bias, lnw = ctx.saved_tensors
        num_head, dim_head, dim_position = ctx.shape_kwargs
        batch, seqlen, d_model = input.size()
        grads = gexts.multihead_projection_layernorm_with_position_rrc_backward_recompute(
            grad_ln, input, weight, bias, lnw, ctx.norm_eps, seqlen, d_model, num_head, dim_head, dim_position, batch)
        return (*grads, None, None, None, None, None)


class Multihead_Galerkin_Attention_cccr_Function(torch.autograd.Function):
    @staticmethod
    def forward(ctx: Any, Q: Tensor, K: Tensor, V: Tensor):
        batch, num_head, d_posk, seqlen = Q.size()
        Attn = gexts.multihead_galerkin_attention_cccr_forward(Q, K, V, batch, num_head, d_posk, seqlen)
        ctx.save_for_backward(Q, K, V)
        return Attn

    @staticmethod
    def backward(ctx: Any, grad_Attn):
        Q, K, V = ctx.saved_tensors
        batch, num_head, d_posk, seqlen = Q.size()
        return gexts.multihead_galerkin_attention_cccr_backward(grad_Attn, Q, K, V, batch, num_head, d_posk, seqlen)


def multihead_projection_with_position_rrc_cuda(input: Tensor, weight: Tensor, bias: Tensor, position: Tensor,
                                                num_head, dim_head, dim_position) -> Tensor:
    """[B, S, Dm] -> [B, H, dim_position + dim_head, S]: (x @ W + b) per head, position rows first."""
    return Multihead_Porjection_with_Position_Function.apply(input, weight, bias, position, num_head, dim_head,
                                                             dim_position)


def multihead_projection_layernorm_with_position_rrc_cuda(input: Tensor, weight: Tensor, bias: Tensor,
                                                          ln_weight: Tensor, ln_bias: Tensor, position: Tensor,
                                                          norm_eps, num_head, dim_head, dim_position) -> Tensor:
    """As above with each head LayerNorm'ed over its dim_head features."""
    return Multihead_Porjection_Layernorm_with_Position_Function.apply(
        input, weight, bias, ln_weight, ln_bias, position, norm_eps, num_head, dim_head, dim_position)


def multihead_galerkin_attention_cccr_cuda(Q: Tensor, K: Tensor, V: Tensor) -> Tensor:
    """Q, K, V [B, H, d, S] -> Q^T (K V^T / S) laid out [B, H, S, d]."""
    return Multihead_Galerkin_Attention_cccr_Function.apply(Q, K, V)


def batched_skinny_gemm(A: Tensor, B: Tensor, alpha: float = 1.0) -> Tensor:
    return gexts.batched_skinny_gemm(A, B, alpha)


def galerkin_attention_ktv(K: Tensor, V: Tensor, position, ln_weight_K: Tensor, ln_bias_K: Tensor,
                           ln_weight_V: Tensor, ln_bias_V: Tensor, norm_eps: float, num_head: int,
                           dim_position: int) -> Tensor:
    """LayerNorm(K), LayerNorm(V) and K'^T V'/S [B, H, d, d] on token-major projections (inference only)."""
    return gexts.galerkin_attention_ktv_forward(K, V, position, ln_weight_K, ln_bias_K, ln_weight_V, ln_bias_V,
                                                norm_eps, num_head, dim_position)


def fold_ktv_into_fc(ktv: Tensor, fc_weight_kn: Tensor, dim_position: int):
    """The attention's last product folded into its output projection: (folded [B, H*32, N], folded_pos [B, dp, N]
    or None) such that Q~ (K'^T V'/S) @ fc_weight_kn = q @ folded[b] + position @ folded_pos[b] (inference only)."""
    return gexts.fold_ktv_into_fc(ktv, fc_weight_kn, dim_position)


class Galerkin_Attention_Fused_Function(torch.autograd.Function):
    """The fused token-major attention core with its backward (no counterpart as one operator in the reference,
    whose autograd functions are the three above; this one computes what their composition computes, starting
    from the plain projections)."""

    @staticmethod
    def forward(ctx: Any, Q: Tensor, K: Tensor, V: Tensor, position, lnwK: Tensor, lnbK: Tensor, lnwV: Tensor,
                lnbV: Tensor, norm_eps: float, num_head: int, dim_position: int):
        out, ktv = gexts.galerkin_attention_fused_forward(Q, K, V, position, lnwK, lnbK, lnwV, lnbV, norm_eps,
                                                          num_head, dim_position, True)
        ctx.save_for_backward(Q, K, V, position if dim_position == 2 else None, lnwK, lnbK, lnwV, lnbV, ktv)
        ctx.args = (float(norm_eps), int(num_head), int(dim_position))
        return out

    @staticmethod
    def backward(ctx: Any, grad_out: Tensor):
        Q, K, V, position, lnwK, lnbK, lnwV, lnbV, ktv = ctx.saved_tensors
        norm_eps, num_head, dim_position = ctx.args
        dQ, dK, dV, dgK, dbK, dgV, dbV = gexts.galerkin_attention_fused_backward(
            grad_out, Q, K, V, position, lnwK, lnbK, lnwV, lnbV, norm_eps, ktv, num_head, dim_position)
        shape = lnwK.shape
        return (dQ, dK, dV, None, dgK.view(shape), dbK.view(shape), dgV.view(shape), dbV.view(shape), None, None, None)


def galerkin_attention_fused(Q: Tensor, K: Tensor, V: Tensor, position, ln_weight_K: Tensor, ln_bias_K: Tensor,
                             ln_weight_V: Tensor, ln_bias_V: Tensor, norm_eps: float, num_head: int,
                             dim_position: int, return_ktv: bool = False):
    """LayerNorm(K), LayerNorm(V), K'^T V'/S and Q' (K'^T V'/S) in one call on token-major projections.
    Differentiable w.r.t. Q, K, V and the four LayerNorm parameters (not w.r.t. position); with return_ktv the
    call is inference-only and also returns K'^T V'/S."""
    needs_graph = torch.is_grad_enabled() and any(
        t.requires_grad for t in (Q, K, V, ln_weight_K, ln_bias_K, ln_weight_V, ln_bias_V))
    if needs_graph and not return_ktv:
        return Galerkin_Attention_Fused_Function.apply(Q, K, V, position, ln_weight_K, ln_bias_K, ln_weight_V,
                                                       ln_bias_V, norm_eps, num_head, dim_position)
    return gexts.galerkin_attention_fused_forward(
        Q, K, V, position, ln_weight_K, ln_bias_K, ln_weight_V, ln_bias_V, norm_eps, num_head, dim_position,
        return_ktv)
