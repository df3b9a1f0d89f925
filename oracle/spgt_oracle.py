"""CPU oracle for the SpGT hot path.  TEST INFRASTRUCTURE ONLY.

This module restates, with plain torch/numpy library operations on the CPU,
what the reference's unaccelerated PyTorch path computes.  It exists so that
the HIP kernels can be checked against something independent of them.  Only
tests/, __graft_entry__.smoke() and bench.py's cpu_baseline leg may import it;
nothing under spgt_amd/ does.

Every function is written for any floating dtype, so the same code gives the
fp32 result (what the reference produces) and an fp64 result (for error
budgets).  Parameters are passed as dicts keyed like the reference modules'
state_dict entries, so a reference checkpoint's tensors can be used as is.

Reference lines followed (paths relative to the reference checkout):
  project_heads ................ network/layer.py:95-112
  project_layernorm_heads ...... network/layer.py:114-141
  galerkin_attention ........... network/layer.py:143-152
  attention_module ............. network/layer.py:67-93
  attention_core_token_major ... network/layer.py:108-111, 128-140, 149-151, 89
  feed_forward ................. network/layer.py:165-174
  encoder_layer ................ network/layer.py:190-200
  complex_mode_product ......... network/layer.py:249-261
  spectral_conv2d .............. network/layer.py:220-247
  conv_block ................... network/layer.py:16-24
  down_scaler / up_scaler ...... network/model.py:23-39 / 53-65
  encoder_mixer ................ network/model.py:82-95
  decoder_regressor ............ network/model.py:112-123
  galerkin_transformer_2d ...... network/model.py:150-172
  gauss_inverse_transform ...... dataset/darcy_dataset.py:30-31
  resolution_sizes ............. common/trivial.py:78-96
Operator-level layouts (what the reference's CUDA extension returns):
  op_projection_rrc ............ extension/bind/galerkin_attention.cu:9-24 and
                                 extension/native/multihead_dim32.cu:343-344 (x @ W, not x @ W^T)
  op_projection_layernorm_rrc .. extension/bind/galerkin_attention.cu:50-68
  op_attention_cccr ............ extension/bind/galerkin_attention.cu:104-124
  op_batched_transpose ......... extension/bind/datamove.cu:8-23
  op_transpose_gather_dual ..... extension/bind/datamove.cu:25-44
  op_transpose_scatter_dual .... extension/bind/datamove.cu:46-64
  op_spectral_conv2d_sp ........ network/sp_layer.py:125-156

Pinning status: every function here has a CPU-side check in tests/ that does not retype its formula.
  * golden vectors written from the reference's own network/layer.py and network/model.py by
    tests/golden/make_golden.py (tests/test_oracle_golden.py): project_heads, project_layernorm_heads,
    galerkin_attention (the attention's three static pieces), attention_module, encoder_layer (and through it
    feed_forward, _act), spectral_conv2d, op_spectral_conv2d_sp, down_scaler, up_scaler (and through them conv_block,
    _interp), galerkin_transformer_2d (and through it encoder_mixer, decoder_regressor, _with_position);
  * closed forms, brute-force loops on tiny inputs and library identities (tests/test_oracle_closed_forms.py):
    galerkin_attention, project_heads, project_layernorm_heads, complex_mode_product, spectral_conv2d,
    bilinear_align_corners, resolution_sizes and every op_* layout function;
  * tests/test_oracle_pins.py: attention_core_token_major and attention_ktv (reference golden vectors and a
    three-loop product), the invsigma orientation of op_projection_layernorm_rrc with a non-symmetric weight,
    gauss_inverse_transform by hand, galerkin_transformer_2d with a normalizer's mean and std.
  The library routines below torch (FFT, GEMM, convolution) are taken as given: they are the routines the
  reference itself calls.
"""
import math

import numpy as np
import torch
import torch.nn.functional as F

# --------------------------------------------------------------------------- #
# attention
# --------------------------------------------------------------------------- #


def _with_position(heads, position, num_head):
    """heads [B, H, S, dh], position [B, S, dp] -> [B, H, S, dp+dh], position first."""
    pos = position[:, None, :, :].expand(-1, num_head, -1, -1)
    return torch.cat([pos, heads], dim=-1)


def project_heads(x, weight, bias, position, num_head, dim_head):
    """Linear (x W^T + b), split into heads, position channels prepended."""
    B, S, _ = x.shape
    y = F.linear(x, weight, bias).reshape(B, S, num_head, dim_head).permute(0, 2, 1, 3)
    return _with_position(y, position, num_head)


def project_layernorm_heads(x, weight, bias, ln_weight, ln_bias, position, eps, num_head, dim_head):
    """As project_heads, with each head LayerNorm'ed over its dim_head features
    (biased variance, eps under the root, affine [num_head, dim_head])."""
    B, S, _ = x.shape
    y = F.linear(x, weight, bias).reshape(B, S, num_head, dim_head).permute(0, 2, 1, 3)
    normed = [
        F.layer_norm(y[:, h], (dim_head,), ln_weight[h], ln_bias[h], eps) for h in range(num_head)
    ]
    return _with_position(torch.stack(normed, dim=1), position, num_head)


def galerkin_attention(Q, K, V):
    """Q, K, V [B, H, S, d] -> Q (K^T V / S); attention dropout is the identity at p = 0."""
    S = Q.shape[-2]
    return Q @ ((K.transpose(-2, -1) @ V) / S)


def attention_ktv(K, V):
    """The d x d matrices K^T V / S, [B, H, d, d]."""
    return (K.transpose(-2, -1) @ V) / K.shape[-2]


def attention_core_token_major(q, k, v, position, ln_weight_K, ln_bias_K, ln_weight_V, ln_bias_V, eps, num_head):
    """The part of GalerkinAttention.forward between the three Linear projections
    and fc_layer (network/layer.py:108-111, 128-140, 149-151, 89), on projected
    q, k, v [B, S, H*32]: split heads, per-head LayerNorm of k and v, position
    channels first, Q (K^T V / S), heads merged back to [B, S, H*(dp+32)]."""
    B, S, C = q.shape
    dh = C // num_head
    heads = lambda t: t.reshape(B, S, num_head, dh).permute(0, 2, 1, 3)
    ln = lambda t, w, b: torch.stack(
        [F.layer_norm(t[:, h], (dh,), w[h], b[h], eps) for h in range(num_head)], dim=1)
    Q = _with_position(heads(q), position, num_head)
    K = _with_position(ln(heads(k), ln_weight_K, ln_bias_K), position, num_head)
    V = _with_position(ln(heads(v), ln_weight_V, ln_bias_V), position, num_head)
    A = galerkin_attention(Q, K, V)
    return A.permute(0, 2, 1, 3).contiguous().reshape(B, S, -1)


def attention_module(p, xq, xk, xv, position, num_head, eps, prefix=""):
    """GalerkinAttention.forward with all drop rates 0."""
    g = lambda k: p[prefix + k]
    dim_head = g("weight_Q").shape[0] // num_head
    B, S, _ = xq.shape
    Q = project_heads(xq, g("weight_Q"), g("bias_Q"), position, num_head, dim_head)
    K = project_layernorm_heads(xk, g("weight_K"), g("bias_K"), g("ln_weight_K"), g("ln_bias_K"), position, eps,
                                num_head, dim_head)
    V = project_layernorm_heads(xv, g("weight_V"), g("bias_V"), g("ln_weight_V"), g("ln_bias_V"), position, eps,
                                num_head, dim_head)
    A = galerkin_attention(Q, K, V)
    A = A.permute(0, 2, 1, 3).reshape(B, S, -1)
    return F.linear(A, g("fc_layer.weight"), g("fc_layer.bias"))


def _act(name):
    return F.silu if name == "silu" else F.relu


def feed_forward(p, x, activation, prefix=""):
    h = _act(activation)(F.linear(x, p[prefix + "layer1.weight"], p[prefix + "layer1.bias"]))
    return F.linear(h, p[prefix + "layer2.weight"], p[prefix + "layer2.bias"])


def encoder_layer(p, x, position, num_head, eps, ffn_activation, prefix=""):
    x = x + attention_module(p, x, x, x, position, num_head, eps, prefix + "attention_layer.")
    return x + feed_forward(p, x, ffn_activation, prefix + "ffn_layer.")


def encoder_mixer(p, x, position, num_layer, num_head, eps, ffn_activation, prefix=""):
    B, r, _, C = x.shape
    x = x.reshape(B, r * r, C)
    position = position.reshape(B, r * r, position.shape[-1])
    for i in range(num_layer):
        x = encoder_layer(p, x, position, num_head, eps, ffn_activation, f"{prefix}layers.{i}.")
    return x.reshape(B, r, r, C)


# --------------------------------------------------------------------------- #
# spectral convolution
# --------------------------------------------------------------------------- #


def complex_mode_product(x_ri, w_ri):
    """x [N, I, h, w, 2], w [I, O, h, w, 2] (re, im) -> [N, O, h, w, 2]: per-mode
    complex contraction over the input channel."""
    xr, xi = x_ri[..., 0], x_ri[..., 1]
    wr, wi = w_ri[..., 0], w_ri[..., 1]
    mix = lambda a, b: torch.einsum("nihw,iohw->nohw", a, b)
    return torch.stack([mix(xr, wr) - mix(xi, wi), mix(xi, wr) + mix(xr, wi)], dim=-1)


def spectral_conv2d(p, x, mode, activation, prefix="", weight_layout="gt"):
    """SpectralConv2D.forward with drop rate 0.  x [N, r, r, Cin] -> [N, r, r, Cout].

    weight_layout 'gt': fourier_weight.k is [Cin, Cout, m, m, 2] (network/layer.py:214-216);
    'sp': [m, m, Cin, Cout, 2] (network/sp_layer.py:119-121)."""
    N, r, _, _ = x.shape
    m = mode
    res = F.linear(x, p[prefix + "residual_layer.weight"], p[prefix + "residual_layer.bias"])
    w0, w1 = p[prefix + "fourier_weight.0"], p[prefix + "fourier_weight.1"]
    if weight_layout == "sp":
        w0, w1 = w0.permute(2, 3, 0, 1, 4), w1.permute(2, 3, 0, 1, 4)
    out_dim = w0.shape[1]
    xf = torch.fft.rfft2(x.permute(0, 3, 1, 2), s=(r, r), norm="ortho")
    xf = torch.view_as_real(xf)
    of = torch.zeros((N, out_dim, r, r // 2 + 1, 2), dtype=x.dtype, device=x.device)
    of[:, :, :m, :m] = complex_mode_product(xf[:, :, :m, :m], w0)
    of[:, :, r - m:, :m] = complex_mode_product(xf[:, :, r - m:, :m], w1)
    y = torch.fft.irfft2(torch.view_as_complex(of.contiguous()), s=(r, r), norm="ortho")
    return _act(activation)(y.permute(0, 2, 3, 1) + res)


# --------------------------------------------------------------------------- #
# scalers, decoder, full model
# --------------------------------------------------------------------------- #


def bilinear_align_corners(x, size):
    """[N, C, Hin, Win] -> [N, C, Hout, Wout] by the explicit align_corners=True rule:
    source coordinate = dst * (in-1)/(out-1), 4-tap linear blend."""
    Hin, Win = x.shape[-2:]
    Hout, Wout = size

    def taps(n_in, n_out):
        if n_out == 1:
            src = torch.zeros(1, dtype=x.dtype)
        else:
            src = torch.arange(n_out, dtype=x.dtype) * ((n_in - 1) / (n_out - 1))
        i0 = src.floor().long().clamp(0, n_in - 1)
        i1 = (i0 + 1).clamp(max=n_in - 1)
        frac = src - i0.to(x.dtype)
        return i0, i1, frac

    h0, h1, fh = taps(Hin, Hout)
    w0, w1, fw = taps(Win, Wout)
    top = x[..., h0, :][..., :, w0] * (1 - fw) + x[..., h0, :][..., :, w1] * fw
    bot = x[..., h1, :][..., :, w0] * (1 - fw) + x[..., h1, :][..., :, w1] * fw
    return top * (1 - fh)[:, None] + bot * fh[:, None]


def _interp(x, size):
    return F.interpolate(x, size=tuple(size), mode="bilinear", align_corners=True)


def conv_block(p, x, activation, prefix):
    y = F.conv2d(x, p[prefix + "conv_layer.weight"], p[prefix + "conv_layer.bias"], padding=1)
    return _act(activation)(y)


def down_scaler(p, x, resolution_size, activation, prefix=""):
    """x [N, r, r, Cin] -> [N, r_attn, r_attn, Cout]."""
    act = _act(activation)
    x = conv_block(p, x.permute(0, 3, 1, 2), activation, prefix + "conv0.")
    x = act(_interp(x, resolution_size[1]))
    x1 = conv_block(p, x, activation, prefix + "conv1.")
    x2 = conv_block(p, x1, activation, prefix + "conv2.")
    x3 = conv_block(p, x2, activation, prefix + "conv3.")
    x = act(_interp(torch.cat([x1, x2, x3], dim=1), resolution_size[2]))
    return x.permute(0, 2, 3, 1)


def up_scaler(p, x, resolution_size, activation, prefix=""):
    """x [N, r_attn, r_attn, C] -> [N, r, r, C]."""
    x = _interp(x.permute(0, 3, 1, 2), resolution_size[3])
    # the conv block ends with the activation and the scaler applies it once more
    x = _act(activation)(conv_block(p, x, activation, prefix + "conv."))
    x = _interp(x, resolution_size[4])
    return x.permute(0, 2, 3, 1)


def decoder_regressor(p, x, grid, num_layer, mode, activation, prefix="", weight_layout="gt"):
    x = torch.cat([x, grid], dim=-1)
    x = F.linear(x, p[prefix + "spatial_fc_layer.weight"], p[prefix + "spatial_fc_layer.bias"])
    for i in range(num_layer):
        x = spectral_conv2d(p, x, mode, activation, f"{prefix}layers.{i}.", weight_layout)
    return feed_forward(p, x, activation, prefix + "ffn_layer.")


def gauss_inverse_transform(x, mean=0.0, std=1.0, eps=1e-5):
    return x * (std + eps) + mean


def galerkin_transformer_2d(p, cfg, x, position, grid, weight_layout="gt"):
    """Full model forward with every drop rate 0.
    x [N, r, r, dim_node], position [N, ra, ra, dp], grid [N, r, r, dp] -> [N, r, r, dim_target]."""
    rs = cfg["resolution_size"]
    x = down_scaler(p, x, rs, cfg["acti_downscaler"], "down_scaler.")
    x = encoder_mixer(p, x, position, cfg["num_encoder_layer"], cfg["num_head"], cfg["attn_norm_eps"],
                      cfg["acti_encoder_ffn"], "encoder_mixer.")
    x = up_scaler(p, x, rs, cfg["acti_upscaler"], "up_scaler.")
    x = decoder_regressor(p, x, grid, cfg["num_decoder_layer"], cfg["num_frequence_mode"],
                          cfg["acti_decoder_layer"], "decoder_regressor.", weight_layout)
    x = gauss_inverse_transform(x, cfg.get("normalizer_mean", 0.0), cfg.get("normalizer_std", 1.0),
                                cfg.get("normalizer_eps", 1e-5))
    if cfg["boundary_condition"] == "dirichlet":
        x = F.pad(x[:, 1:-1, 1:-1], (0, 0, 1, 1, 1, 1), "constant", 0.0)
    return x


def resolution_sizes(r_large, r_small):
    """The five grid sizes (fine, mid, attention, mid, fine) of the two-step
    down/up sampling; mid = round(r_large * f) - 1 with f = sqrt(r_small/r_large)
    rounded to 4 decimals and then up to a multiple of 0.005 in the reference's
    particular way (which looks at the last printed digit)."""
    # np.sqrt returns a numpy scalar, whose round() is numpy's (scale, round half to even, unscale), not Python's
    factor = np.sqrt(r_small / r_large).round(4)
    last_digit = float(repr(float(factor))[-1])
    factor = float(factor.round(3))
    if last_digit < 5:
        factor += 5.0e-3
    factor = int(factor / 5.0e-3 + 0.5) * 5.0e-3
    r_mid = round(r_large * factor) - 1
    return ((r_large, r_large), (r_mid, r_mid), (r_small, r_small), (r_mid, r_mid), (r_large, r_large))


# --------------------------------------------------------------------------- #
# operator-level layouts of the reference's extension
# --------------------------------------------------------------------------- #


def op_projection_rrc(x, weight, bias, position, num_head, dim_head):
    """[B, H, dp+dh, S]; the extension multiplies by W as stored (x @ W)."""
    return project_heads(x, weight.t(), bias, position, num_head, dim_head).transpose(-2, -1).contiguous()


def op_projection_layernorm_rrc(x, weight, bias, ln_weight, ln_bias, position, eps, num_head, dim_head):
    """([B, H, dp+dh, S], invsigma [B, H, S])."""
    B, S, _ = x.shape
    y = project_layernorm_heads(x, weight.t(), bias, ln_weight, ln_bias, position, eps, num_head, dim_head)
    raw = (x @ weight + bias).reshape(B, S, num_head, dim_head).permute(0, 2, 1, 3)
    invsigma = 1.0 / torch.sqrt(raw.var(dim=-1, unbiased=False) + eps)
    return y.transpose(-2, -1).contiguous(), invsigma


def op_attention_cccr(Q, K, V):
    """Q, K, V [B, H, d, S] -> [B, H, S, d]."""
    t = lambda a: a.transpose(-2, -1)
    return galerkin_attention(t(Q), t(K), t(V)).contiguous()


def op_batched_skinny_gemm(A, B, alpha=1.0):
    return (A @ B) * alpha


def op_batched_transpose(x, batch_list, m_list, n_list):
    b, m, n = math.prod(batch_list), math.prod(m_list), math.prod(n_list)
    y = x.reshape(b, m, n).transpose(1, 2).contiguous()
    return y.reshape(*batch_list, *n_list, *m_list)


def op_transpose_gather_dual(src, dim_list, H_all, W_all, H_low, W_low, hb1, wb1, hb2, wb2):
    """src [*dim_list, H_all, W_all] -> two [H_low, W_low, *dim_list] windows."""
    nd = len(dim_list)
    perm = (nd, nd + 1) + tuple(range(nd))

    def win(hb, wb):
        return src[..., hb:hb + H_low, wb:wb + W_low].permute(*perm).contiguous()

    return win(hb1, wb1), win(hb2, wb2)


def op_transpose_scatter_dual(src1, src2, dim_list, H_all, W_all, H_low, W_low, hb1, wb1, hb2, wb2):
    """Inverse of the gather into a zero-filled [*dim_list, H_all, W_all]."""
    nd = len(dim_list)
    perm = tuple(range(2, 2 + nd)) + (0, 1)
    out = torch.zeros((*dim_list, H_all, W_all), dtype=src1.dtype, device=src1.device)
    out[..., hb1:hb1 + H_low, wb1:wb1 + W_low] = src1.permute(*perm)
    out[..., hb2:hb2 + H_low, wb2:wb2 + W_low] = src2.permute(*perm)
    return out


def op_spectral_conv2d_sp(p, x, mode, activation, prefix=""):
    """Sp_SpectralConv2D.forward as a sequence of the operator-level pieces
    (weights in the 'sp' layout [m, m, Cin, Cout, 2])."""
    N, r, _, cin = x.shape
    m = mode
    res = F.linear(x, p[prefix + "residual_layer.weight"], p[prefix + "residual_layer.bias"])
    w0 = torch.view_as_complex(p[prefix + "fourier_weight.0"].contiguous())
    w1 = torch.view_as_complex(p[prefix + "fourier_weight.1"].contiguous())
    cout = w0.shape[-1]
    xt = op_batched_transpose(x, [N], [r, r], [cin])
    xf = torch.fft.rfft2(xt, s=(r, r), norm="ortho")
    g0, g1 = op_transpose_gather_dual(xf, [N, cin], r, r // 2 + 1, m, m, 0, 0, r - m, 0)
    of = op_transpose_scatter_dual(g0 @ w0, g1 @ w1, [N, cout], r, r // 2 + 1, m, m, 0, 0, r - m, 0)
    y = torch.fft.irfft2(of, s=(r, r), norm="ortho")
    y = op_batched_transpose(y, [N], [cout], [r, r])
    return _act(activation)(y + res)
