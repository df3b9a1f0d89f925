"""Truncated 2-D DFTs for the spectral layer.

Sp_SpectralConv2D keeps only the modes kh in [0, m) and [r-m, r), kw in [0, m) of rfft2(x) and feeds
irfft2 a spectrum that is zero everywhere else (reference: network/sp_layer.py:138-150).  Computing
exactly those modes as two small matrix products per direction,

    forward   Y[n,h,c,kw]  = sum_w x[n,h,w,c] e^{-2 pi i kw w / r} / sqrt(r)
              Z[n,kh,c,kw] = sum_h Y[n,h,c,kw] e^{-2 pi i kh h / r} / sqrt(r)
    inverse   U[n,h,o,kw]  = sum_kh O[n,kh,o,kw] e^{+2 pi i kh h / r} / sqrt(r)
              y[n,h,w,o]   = Re sum_kw c_kw U[n,h,o,kw] e^{+2 pi i kw w / r} / sqrt(r),   c_0 = 1, c_kw = 2
                             (c = 1 as well for the Nyquist column of an even r),

gives the same result as the FFT route up to fp32 rounding (the real part in the last line is what the
complex-to-real transform of irfft2 computes from a half spectrum), works directly on the [N, r, r, C]
layout of the module - both full-tensor transposes, the full-size spectra, the corner gather/scatter and
the zero fill disappear - and does not depend on r having small prime factors (r = 211 is prime).
The two products along w, which touch the full tensor, are the HIP kernels behind `truncated_dft_rows_*`;
the two small ones along h are library GEMMs; the per-mode channel contraction between them is the HIP
kernel behind `spectral_modes_compact`.
"""
import math
from typing import Dict, Tuple

import torch
from torch import Tensor

from ..extension.bind.linear import fused_linear, linear_supported, linear_weight_grad
from ..extension.bind.datamove import (inverse_table_operand, spectral_inverse_linear,
                                       spectral_inverse_linear_supported, spectral_modes_compact, spectral_modes_middle,
                                       spectral_modes_middle_supported, truncated_dft_rows_forward,
                                       truncated_dft_rows_inverse, truncated_dft_rows_supported)

_TABLES: Dict[Tuple[int, int, str], Tuple[Tensor, Tensor, Tensor, Tensor]] = {}


def dft_tables(r: int, m: int, device) -> Tuple[Tensor, Tensor, Tensor, Tensor]:
    """(Fw [r, 2m] real, Gh [2m, r] complex, Ghi [r, 2m] complex, Fwi [r, 2m] real), built in fp64."""
    key = (r, m, str(device))
    if key not in _TABLES:
        idx = torch.arange(r, dtype=torch.float64)
        kw = torch.arange(m, dtype=torch.float64)
        kh = torch.cat([torch.arange(m), torch.arange(r - m, r)]).to(torch.float64)
        s = 1.0 / math.sqrt(r)
        ang_w = 2.0 * math.pi * idx[:, None] * kw[None, :] / r                  # [r, m]
        fw = torch.stack([torch.cos(ang_w), -torch.sin(ang_w)], dim=-1) * s      # columns (kw, re|im)
        c = torch.full((m,), 2.0, dtype=torch.float64)
        c[0] = 1.0
        if r % 2 == 0 and m - 1 == r // 2:
            c[-1] = 1.0
        fwi = torch.stack([torch.cos(ang_w) * c, -torch.sin(ang_w) * c], dim=-1) * s
        ang_h = 2.0 * math.pi * kh[:, None] * idx[None, :] / r                  # [2m, r]
        gh = torch.complex(torch.cos(ang_h), -torch.sin(ang_h)) * s
        ghi = torch.complex(torch.cos(ang_h), torch.sin(ang_h)).t() * s
        _TABLES[key] = (fw.reshape(r, 2 * m).float().to(device).contiguous(),
                        gh.to(torch.complex64).to(device).contiguous(),
                        ghi.to(torch.complex64).to(device).contiguous(),
                        fwi.reshape(r, 2 * m).float().to(device).contiguous())
    return _TABLES[key]


def supported(r: int, m: int) -> bool:
    """The two retained row windows must not overlap."""
    return 2 * m <= r


_OPERAND_TABLES: Dict[Tuple[int, int, str], Tensor] = {}


def fused_tail_supported(r: int, cin: int, cout: int, m: int) -> bool:
    """True when spectral_modes_apply_linear runs in three launches (row DFT, retained modes, inverse row DFT fused
    with the residual Linear and the activation)."""
    return (truncated_dft_rows_supported(r, cin, m) and spectral_modes_middle_supported(r, cin, cout, m) and
            spectral_inverse_linear_supported(r, cin, cout, m))


def spectral_modes_apply_linear(x: Tensor, weight_1: Tensor, weight_2: Tensor, m: int, linear_weight_kn: Tensor,
                                linear_bias, activation) -> Tensor:
    """act(x @ linear_weight_kn + linear_bias + irfft2(W . truncate(rfft2(x)))) for x [N, r, r, C]: the whole
    spectral layer after dropout; requires fused_tail_supported."""
    N, r, _, cin = x.shape
    fw, gh, ghi, fwi = dft_tables(r, m, x.device)
    yp = truncated_dft_rows_forward(x, fw, planar=True)             # [N, 2m, r, Cin]
    up = spectral_modes_middle(yp, gh, ghi, weight_1, weight_2)     # [N, 2m, r, Cout]
    return spectral_inverse_linear(up, _operand_table(r, m, x.device), x, linear_weight_kn, linear_bias, activation)


def _operand_table(r: int, m: int, device) -> Tensor:
    key = (r, m, str(device))
    if key not in _OPERAND_TABLES:
        _OPERAND_TABLES[key] = inverse_table_operand(dft_tables(r, m, device)[3])
    return _OPERAND_TABLES[key]


class _SpectralLinearFunction(torch.autograd.Function):
    """x @ W_lin^T + b + irfft2(W_f . truncate(rfft2(x))) on the truncated-DFT route, with its backward on the same
    kernels.  Every stage is linear, so the backward runs the adjoint stages in reverse: the inverse row transform's
    adjoint is a forward row transform with the inverse table, the forward one's an inverse row transform with the
    forward table, and the adjoint of the complex-linear middle (DFT along h, channel contraction, inverse DFT
    along h) is the same kernel with conjugate-transposed tables and weights.  The Fourier weights' gradient,
    dW[kh, kw, c, o] = sum_n conj(Z[n, kh, c, kw]) dO[n, kh, o, kw], is formed from the retained modes (a few MB)
    by library products."""

    @staticmethod
    def forward(ctx, x, weight_1, weight_2, lin_weight, lin_bias, lin_weight_kn, m):
        N, r, _, cin = x.shape
        fw, gh, ghi, _ = dft_tables(r, m, x.device)
        yp = truncated_dft_rows_forward(x, fw, planar=True)                         # [N, 2m, r, Cin]
        up = spectral_modes_middle(yp, gh, ghi, weight_1, weight_2)                 # [N, 2m, r, Cout]
        out = spectral_inverse_linear(up, _operand_table(r, m, x.device), x, lin_weight_kn, lin_bias, None)
        ctx.save_for_backward(x, weight_1, weight_2, lin_weight, yp)
        ctx.m, ctx.has_bias = m, lin_bias is not None
        return out

    @staticmethod
    def backward(ctx, g):
        x, weight_1, weight_2, lin_weight, yp = ctx.saved_tensors
        m = ctx.m
        g = g.contiguous()
        N, r, _, cout = g.shape
        cin = x.shape[-1]
        fw, gh, ghi, fwi = dft_tables(r, m, x.device)
        ghi_h = ghi.conj().t().contiguous()                                         # [2m, r]
        dup = truncated_dft_rows_forward(g, fwi, planar=True)                       # [N, 2m, r, Cout] = Fi^T g
        dx = None
        if ctx.needs_input_grad[0]:
            gh_h = gh.conj().t().contiguous()                                       # [r, 2m]
            conj_t = lambda w: torch.view_as_real(torch.view_as_complex(w).conj().transpose(2, 3).contiguous())
            w1h, w2h = conj_t(weight_1.detach()), conj_t(weight_2.detach())         # [m, m, Cout, Cin, 2]
            if cin <= 64:
                dyp = spectral_modes_middle(dup, ghi_h, gh_h, w1h, w2h)             # [N, 2m, r, Cin]
            else:  # the middle kernel writes at most 64 channels per call
                dyp = torch.cat([spectral_modes_middle(dup, ghi_h, gh_h, w1h[:, :, :, c0:c0 + 64].contiguous(),
                                                       w2h[:, :, :, c0:c0 + 64].contiguous())
                                 for c0 in range(0, cin, 64)], dim=3)
            dx = truncated_dft_rows_inverse(dyp, fw, planar=True)                   # [N, r, r, Cin]
            g2, w = g.view(-1, cout), lin_weight.detach()
            if linear_supported(cout, cin):
                dx = fused_linear(g2, w.contiguous(), None, "none", dx.view(-1, cin)).view(N, r, r, cin)
            else:
                dx = dx + torch.matmul(g2, w).view(N, r, r, cin)
        dw_lin = db = dw1 = dw2 = None
        if ctx.needs_input_grad[3] or (ctx.has_bias and ctx.needs_input_grad[4]):
            dw_kn, db = linear_weight_grad(x.view(-1, cin), g.view(-1, cout))
            dw_lin = dw_kn.t()
            if not ctx.has_bias:
                db = None
        if ctx.needs_input_grad[1] or ctx.needs_input_grad[2]:
            yc = torch.complex(yp[:, 0::2], yp[:, 1::2])                            # [N, kw, h, Cin]
            z = torch.einsum("kh,nwhc->nkwc", gh, yc)                               # [N, 2m, kw, Cin]
            duc = torch.complex(dup[:, 0::2], dup[:, 1::2])                         # [N, kw, h, Cout]
            do = torch.einsum("kh,nwho->nkwo", ghi_h, duc)                          # [N, 2m, kw, Cout]
            dw = torch.view_as_real(torch.einsum("nkwc,nkwo->kwco", z.conj(), do))  # [2m, kw, Cin, Cout, 2]
            dw1, dw2 = dw[:m], dw[m:]
        return dx, dw1, dw2, dw_lin, db, None, None


def spectral_linear_trainable(r: int, cin: int, cout: int, m: int) -> bool:
    """True when spectral_linear_train serves this shape: the three-launch route forward, and for the backward a
    row-transform variant for both widths and a weight-gradient row length that is a multiple of 4."""
    return (fused_tail_supported(r, cin, cout, m) and truncated_dft_rows_supported(r, cout, m) and
            spectral_modes_middle_supported(r, cout, min(cin, 64), m) and cout % 4 == 0)


def spectral_linear_train(x: Tensor, weight_1: Tensor, weight_2: Tensor, m: int, lin_weight: Tensor, lin_bias,
                          lin_weight_kn: Tensor) -> Tensor:
    """x @ lin_weight^T + lin_bias + irfft2(W . truncate(rfft2(x))) for x [N, r, r, Cin], with an autograd graph
    (see _SpectralLinearFunction); requires spectral_linear_trainable."""
    return _SpectralLinearFunction.apply(x, weight_1, weight_2, lin_weight, lin_bias, lin_weight_kn, m)


def spectral_modes_apply(x: Tensor, weight_1: Tensor, weight_2: Tensor, m: int) -> Tensor:
    """x [N, r, r, Cin] -> irfft2(W . truncate(rfft2(x))) as [N, r, r, Cout] (norm='ortho')."""
    N, r, _, cin = x.shape
    cout = weight_1.shape[3]
    fw, gh, ghi, fwi = dft_tables(r, m, x.device)
    rows_kernel = truncated_dft_rows_supported(r, cin, m) and truncated_dft_rows_supported(r, cout, m)
    if rows_kernel and spectral_modes_middle_supported(r, cin, cout, m):
        # three launches: DFT along w, everything on the retained modes, inverse DFT along w
        yp = truncated_dft_rows_forward(x, fw, planar=True)                               # [N, 2m, r, Cin]
        up = spectral_modes_middle(yp, gh, ghi, weight_1, weight_2)                       # [N, 2m, r, Cout]
        return truncated_dft_rows_inverse(up, fwi, planar=True)                           # [N, r, r, Cout]
    if rows_kernel:
        y = truncated_dft_rows_forward(x.reshape(N * r, r, cin), fw)                     # [N r, Cin, 2m]
    else:
        y = torch.matmul(x.reshape(N * r, r, cin).transpose(1, 2), fw)
    yc = torch.view_as_complex(y.view(N, r, cin, m, 2)).reshape(N, r, cin * m)
    z = torch.matmul(gh, yc).view(N, 2 * m, cin, m)                                      # [N, 2m, Cin, m]
    o = spectral_modes_compact(z, weight_1, weight_2)                                    # [N, 2m, Cout, m]
    u = torch.matmul(ghi, o.view(N, 2 * m, cout * m))                                    # [N, r, Cout m]
    ur = torch.view_as_real(u).view(N * r, cout, 2 * m)
    if rows_kernel:
        return truncated_dft_rows_inverse(ur, fwi).view(N, r, r, cout)
    return torch.matmul(fwi, ur.transpose(1, 2)).view(N, r, r, cout)
