"""Accelerated layers: Galerkin attention, encoder layer, FNO spectral
convolution.  Class names, constructor arguments, parameter names and shapes
follow the reference's network/sp_layer.py (Sp_GalerkinAttention :12-78,
Sp_EncoderLayer :81-104, Sp_SpectralConv2D :107-156), so a checkpoint of the
reference's accelerated model loads unchanged and gives the same outputs.

Two conventions of the reference are kept on purpose:
  * the projections multiply by the weight as stored, x @ W + b (its CUDA
    kernel, extension/native/multihead_dim32.cu:343-344), whereas the plain
    PyTorch model computes x @ W^T + b; `convert_gt_state_dict` maps a
    checkpoint of the plain model onto these modules;
  * F.dropout runs with training=True whenever a drop rate is non-zero.

Without autograd (inference) the layers take the fused kernels: one GEMM for
the three projections, then LayerNorm + K^T V / S + Q (K^T V / S) in one call
on token-major data; the spectral layer contracts the retained modes straight
out of and into the full spectrum.  With autograd they run the reference's
operator sequence.
"""
import math
from typing import Dict

import torch
import torch.nn.functional as F
from torch import Tensor, nn

from ..extension.bind.datamove import (batched_transpose, spectral_mode_contract, transpose_gather_dual,
                                       transpose_scatter_dual)
from ..extension.bind.galerkin_attention import (fold_ktv_into_fc, galerkin_attention_fused, galerkin_attention_ktv,
                                                 multihead_galerkin_attention_cccr_cuda,
                                                 multihead_projection_layernorm_with_position_rrc_cuda,
                                                 multihead_projection_with_position_rrc_cuda)
from . import truncated_dft
from ..extension.bind.linear import (encoder_tail_supported, fused_encoder_tail, fused_encoder_tail_folded,
                                     fused_linear, linear_supported, linear_weight_grad_batched)
from .derived import derived, refreshes_derived
from .layer import (FeedForward, activation_name, always_dropout, always_dropout_add, fused_linear_usable, gpu_inference,
                    linear_train, linear_trainable, linear_weight_kn, make_activation)


class _PackedProjectionFunction(torch.autograd.Function):
    """x -> (x W_Q + b_Q, x W_K + b_K, x W_V + b_V) as three contiguous planes: one launch of the fused linear
    kernel over [W_Q | W_K | W_V] forward; backward dX by three chained launches of the same kernel on the
    transposed weights and (dW, db) of all three by one pass over x and the three gradient planes."""

    @staticmethod
    def forward(ctx, x, wq, wk, wv, bq, bk, bv, packed_w, packed_b):
        N, S, C = x.shape
        ctx.save_for_backward(x, wq, wk, wv)
        out = fused_linear(x.reshape(N * S, C), packed_w, packed_b, planes=3).view(3, N, S, C)
        # the fourth result is x itself: a caller that also adds x as a residual takes it from here, so that the
        # residual's gradient arrives in this backward and rides in the dX product instead of a separate add
        return out[0], out[1], out[2], x.view_as(x)

    @staticmethod
    def backward(ctx, dq, dk, dv, dres):
        x, wq, wk, wv = ctx.saved_tensors
        N, S, C = x.shape
        planes = (dq, dk, dv)
        same_buffer = (all(t.is_contiguous() and t.dtype == torch.float32 for t in planes) and
                       len({t.untyped_storage().data_ptr() for t in planes}) == 1 and
                       dk.data_ptr() - dq.data_ptr() == 4 * dq.numel() == dv.data_ptr() - dk.data_ptr())
        if same_buffer:
            # the attention backward hands over the three planes of one buffer: no copy
            grads = torch.as_strided(dq, (3, N * S, C), (N * S * C, C, 1))
        else:
            grads = torch.stack([dq.reshape(N * S, C), dk.reshape(N * S, C), dv.reshape(N * S, C)])
        dx = None
        if ctx.needs_input_grad[0]:
            dx = None if dres is None else dres.reshape(N * S, C).contiguous()
            for g, w in zip(grads, (wq, wk, wv)):
                dx = fused_linear(g, w.t().contiguous(), None, "none", dx)  # dx += g @ w^T
            dx = dx.view(N, S, C)
        dW, db = linear_weight_grad_batched(x.reshape(N * S, C), grads)
        return dx, dW[0], dW[1], dW[2], db[0], db[1], db[2], None, None


class Sp_GalerkinAttention(nn.Module):
    # under autograd: the fused token-major core with its own backward (True) or the reference's sequence of three
    # feature-major operators (False)
    fused_training = True

    def __init__(self, dim_hidden, num_head, dim_position, norm_eps, attn_droprate, fc_droprate, xavier, diagonal,
                 symmetric) -> None:
        super().__init__()
        assert dim_hidden % 128 == 0 and dim_hidden // num_head == 32
        if dim_position not in (0, 2):
            # the reference's position kernel is written for two coordinates and skips the case of none
            # (extension/native/multihead_dim32.cu:6-22, 593-598); any other value corrupts memory there
            raise ValueError(f"dim_position must be 0 or 2 (got {dim_position})")
        self.dim_hidden = dim_hidden
        self.num_head = num_head
        self.dim_head = dim_hidden // num_head
        self.dim_position = dim_position
        self.norm_eps = norm_eps
        self.attn_droprate = attn_droprate  # accepted and, as in the reference's accelerated layer, unused
        self.fc_droprate = fc_droprate
        for n in "QKV":
            setattr(self, f"weight_{n}", nn.Parameter(torch.empty(dim_hidden, dim_hidden)))
        for n in "QKV":
            setattr(self, f"bias_{n}", nn.Parameter(torch.empty(dim_hidden)))
        for kind in ("weight", "bias"):
            for n in "KV":
                setattr(self, f"ln_{kind}_{n}", nn.Parameter(torch.empty(num_head, self.dim_head)))
        self.fc_layer = nn.Linear(dim_hidden + dim_position * num_head, dim_hidden)
        self._reset_parameters(xavier, diagonal, symmetric)

    def _reset_parameters(self, xavier, diagonal, symmetric) -> None:
        with torch.no_grad():
            for w in (self.weight_Q, self.weight_K, self.weight_V):
                nn.init.xavier_uniform_(w, gain=xavier)
                if diagonal > 0:
                    w += diagonal * torch.eye(w.size(-1))
                if symmetric:
                    w += w.T.clone()
            for b in (self.bias_Q, self.bias_K, self.bias_V, self.ln_bias_K, self.ln_bias_V):
                b.zero_()
            for g in (self.ln_weight_K, self.ln_weight_V):
                g.fill_(1.0)

    def _packed_qkv(self):
        """[W_Q | W_K | W_V] (dim_hidden x 3 dim_hidden) and the packed bias: derived tensors, rewritten from the
        six parameters at the start of every inference forward."""
        C = self.dim_hidden

        def weight_spec():
            ws = (self.weight_Q, self.weight_K, self.weight_V)
            return (C, 3 * C), [(w, 0, (1, C, C), (0, w.stride(0), w.stride(1)), j * C, (0, 3 * C, 1))
                                for j, w in enumerate(ws)]

        def bias_spec():
            bs = (self.bias_Q, self.bias_K, self.bias_V)
            return (3 * C,), [(b, 0, (1, 1, C), (0, 0, b.stride(0)), j * C, (0, 0, 1)) for j, b in enumerate(bs)]

        return derived(self, "qkv_weight", weight_spec), derived(self, "qkv_bias", bias_spec)

    def _needs_graph(self, *tensors) -> bool:
        return torch.is_grad_enabled() and (any(t.requires_grad for t in tensors) or
                                            any(p.requires_grad for p in self.parameters()))

    @refreshes_derived
    def forward(self, Q: Tensor, K: Tensor, V: Tensor, position: Tensor, residual: Tensor = None) -> Tensor:
        """Q, K, V [N, seqlen, dim_hidden], position [N, seqlen, dim_position] -> [N, seqlen, dim_hidden];
        with `residual` the result is residual + attention(Q, K, V)."""
        X, identity = self._attend(Q, K, V, position)
        if identity is not None and residual is Q:
            residual = identity  # Q as the packed projection's autograd function handed it on (see there)
        return self.project(X, residual)

    def attend(self, Q: Tensor, K: Tensor, V: Tensor, position: Tensor) -> Tensor:
        """The attention core before fc_layer: [N, seqlen, num_head * (dim_position + dim_head)]."""
        return self._attend(Q, K, V, position)[0]

    def _attend(self, Q: Tensor, K: Tensor, V: Tensor, position: Tensor):
        """(attend(...), Q as an output of the training route's packed projection or None)."""
        identity = None
        N, seqlen, C = Q.size()
        H, dp = self.num_head, self.dim_position
        if self._needs_graph(Q, K, V) and C > 512:
            # wider than the projection operators serve (they keep a head's weight columns in registers, up to
            # dim_hidden 512): library GEMM and LayerNorm under autograd, laid out as the attention operator reads
            def wide(x, w, b, ln_w=None, ln_b=None):
                y = torch.addmm(b, x.reshape(N * seqlen, C), w).view(N, seqlen, H, self.dim_head)
                if ln_w is not None:
                    y = F.layer_norm(y, [self.dim_head], None, None, self.norm_eps) * ln_w + ln_b
                if dp:
                    y = torch.cat([position.unsqueeze(2).expand(N, seqlen, H, dp), y], dim=-1)
                return y.permute(0, 2, 3, 1).contiguous()  # [N, H, dp + dim_head, seqlen]

            X = multihead_galerkin_attention_cccr_cuda(
                wide(Q, self.weight_Q, self.bias_Q), wide(K, self.weight_K, self.bias_K, self.ln_weight_K, self.ln_bias_K),
                wide(V, self.weight_V, self.bias_V, self.ln_weight_V, self.ln_bias_V))
            X = X.transpose(1, 2).contiguous().view(N, seqlen, H * (dp + self.dim_head))
        elif self._needs_graph(Q, K, V) and self.fused_training and Q is K and K is V and linear_supported(C, 3 * C) \
                and linear_supported(C, C) and Q.is_cuda and Q.dtype == torch.float32:
            # training on the token-major path: packed projection, then the fused core, both with their own backward
            w, b = self._packed_qkv()
            q, k, v, ident = _PackedProjectionFunction.apply(Q.contiguous(), self.weight_Q, self.weight_K,
                                                             self.weight_V, self.bias_Q, self.bias_K, self.bias_V, w, b)
            if Q.is_contiguous():
                identity = ident
            pos = position.contiguous() if dp else None
            X = galerkin_attention_fused(q, k, v, pos, self.ln_weight_K, self.ln_bias_K, self.ln_weight_V,
                                         self.ln_bias_V, self.norm_eps, H, dp)
        elif self._needs_graph(Q, K, V):
            q = multihead_projection_with_position_rrc_cuda(Q, self.weight_Q, self.bias_Q, position, H, self.dim_head, dp)
            k = multihead_projection_layernorm_with_position_rrc_cuda(
                K, self.weight_K, self.bias_K, self.ln_weight_K, self.ln_bias_K, position, self.norm_eps, H,
                self.dim_head, dp)
            v = multihead_projection_layernorm_with_position_rrc_cuda(
                V, self.weight_V, self.bias_V, self.ln_weight_V, self.ln_bias_V, position, self.norm_eps, H,
                self.dim_head, dp)
            X = multihead_galerkin_attention_cccr_cuda(q, k, v)
            X = X.transpose(1, 2).contiguous().view(N, seqlen, H * (dp + self.dim_head))
        else:
            if Q is K and K is V and linear_supported(C, 3 * C):
                # one launch over [W_Q | W_K | W_V] with the bias in its epilogue; the three projections land
                # in contiguous planes (the attention passes run 15 % faster on unit-stride rows)
                w, b = self._packed_qkv()
                q, k, v = fused_linear(Q.reshape(N * seqlen, C), w, b, planes=3).view(3, N, seqlen, C).unbind(0)
            else:
                if linear_supported(C, C):
                    proj = lambda x, w, b: fused_linear(x.reshape(N * seqlen, C), w.detach(), b.detach()).view(N, seqlen, C)
                else:  # wider models than the fused linear kernel serves: the library GEMM, then the fused core
                    proj = lambda x, w, b: torch.addmm(b.detach(), x.reshape(N * seqlen, C), w.detach()).view(N, seqlen, C)
                q, k, v = (proj(Q, self.weight_Q, self.bias_Q), proj(K, self.weight_K, self.bias_K),
                           proj(V, self.weight_V, self.bias_V))
            pos = position.contiguous() if dp else None
            X = galerkin_attention_fused(q, k, v, pos, self.ln_weight_K.detach(), self.ln_bias_K.detach(),
                                         self.ln_weight_V.detach(), self.ln_bias_V.detach(), self.norm_eps, H, dp)
        return X, identity

    def folded_projection(self, X: Tensor, position: Tensor):
        """(q, position, folded_fc, folded_pos) for fused_encoder_tail_folded: self-attention on X whose last
        product is folded into fc_layer.  Q~ (K~^T V~ / S) Wfc = Q~ ((K~^T V~ / S) Wfc): instead of a pass over Q
        that writes the attention output for fc_layer to read, the small per-head matrices are multiplied into
        fc_layer's weight, once per sequence, and the projected Q meets the result in the encoder tail."""
        N, seqlen, C = X.size()
        H, dp = self.num_head, self.dim_position
        w, b = self._packed_qkv()
        q, k, v = fused_linear(X.reshape(N * seqlen, C), w, b, planes=3).view(3, N, seqlen, C).unbind(0)
        pos = position.contiguous() if dp else None
        ktv = galerkin_attention_ktv(k, v, pos, self.ln_weight_K.detach(), self.ln_bias_K.detach(),
                                     self.ln_weight_V.detach(), self.ln_bias_V.detach(), self.norm_eps, H, dp)
        folded_fc, folded_pos = fold_ktv_into_fc(ktv, linear_weight_kn(self.fc_layer), dp)
        return q, pos, folded_fc, folded_pos

    def project(self, X: Tensor, residual: Tensor = None) -> Tensor:
        """fc_layer (+ dropout) on the attention core's output, plus the residual when given."""
        if fused_linear_usable(X, self.fc_layer) and (residual is None or self.fc_droprate == 0):
            Y = fused_linear(X, linear_weight_kn(self.fc_layer), self.fc_layer.bias, "none", residual)
            return always_dropout(Y, self.fc_droprate)
        if linear_trainable(X, self.fc_layer):
            if self.fc_droprate == 0:
                return linear_train(X, self.fc_layer, residual)
            return always_dropout_add(linear_train(X, self.fc_layer), residual, self.fc_droprate)
        Y = always_dropout(self.fc_layer(X), self.fc_droprate)
        return Y if residual is None else residual + Y


class Sp_EncoderLayer(nn.Module):
    """x + attention(x); then x + ffn(x).  No normalisation on the residual stream."""

    # inference path: fold the attention's last product into fc_layer's weight (see folded_projection).  The fold
    # costs a fixed 5 us per layer plus 2 us in the tail, the pass over Q it replaces 7.6 us at 20k tokens (a whole
    # Darcy forward measures 0.883-0.888 ms folded against 0.890-0.895 ms) and 31 us at 159k: None folds from
    # fold_attention_min_tokens tokens on, True / False force the choice.
    fold_attention = None
    fold_attention_min_tokens = 16384

    def __init__(self, dim_hidden, num_head, dim_position, norm_eps, attn_droprate, fc_droprate, xavier, diagonal,
                 symmetric, ffn_dim_hidden, ffn_droprate, ffn_activation) -> None:
        super().__init__()
        self.attention_layer = Sp_GalerkinAttention(dim_hidden, num_head, dim_position, norm_eps, attn_droprate,
                                                    fc_droprate, xavier, diagonal, symmetric)
        self.ffn_layer = FeedForward(dim_hidden, dim_hidden, ffn_dim_hidden, ffn_droprate, ffn_activation)

    @refreshes_derived
    def forward(self, X: Tensor, position: Tensor) -> Tensor:
        att, ffn = self.attention_layer, self.ffn_layer
        if (0 <= att.fc_droprate < 1 and 0 <= ffn.droprate < 1 and gpu_inference(X, self) and
                encoder_tail_supported(att.fc_layer.in_features, att.fc_layer.out_features, ffn.layer1.out_features)
                and ffn.layer2.out_features == att.fc_layer.out_features):
            # output projection, both residual adds and the feed-forward net in one launch; the layer's two
            # dropouts (always on in the reference, network/sp_layer.py:76 and network/layer.py:173) are applied
            # inside it when their rates are not zero
            drop = dict(fc_droprate=att.fc_droprate, ffn_droprate=ffn.droprate)
            fold = (X.numel() // X.size(-1) >= self.fold_attention_min_tokens if self.fold_attention is None
                    else self.fold_attention)
            if fold and att.dim_head == 32 and att.num_head * 32 == X.size(-1) == 128 and X.dim() == 3:
                # ... and the attention's Q.(K^T V) product folded into that projection's weight
                q, pos, folded_fc, folded_pos = att.folded_projection(X, position)
                return fused_encoder_tail_folded(q, pos, X.contiguous(), folded_fc, folded_pos, att.fc_layer.bias,
                                                 linear_weight_kn(ffn.layer1), ffn.layer1.bias,
                                                 linear_weight_kn(ffn.layer2), ffn.layer2.bias,
                                                 activation_name(ffn.activation_layer), **drop)
            A = att.attend(X, X, X, position)
            return fused_encoder_tail(A, X.contiguous(), linear_weight_kn(att.fc_layer), att.fc_layer.bias,
                                      linear_weight_kn(ffn.layer1), ffn.layer1.bias, linear_weight_kn(ffn.layer2),
                                      ffn.layer2.bias, activation_name(ffn.activation_layer), **drop)
        X = self.attention_layer(X, X, X, position, residual=X)
        return self.ffn_layer(X, residual=X)


class Sp_SpectralConv2D(nn.Module):
    # inference path: truncated DFTs as matrix products instead of rfft2 / irfft2 (see truncated_dft.py)
    use_truncated_dft = True

    def __init__(self, in_dim, out_dim, mode, droprate, activation) -> None:
        super().__init__()
        self.in_dim, self.out_dim, self.mode, self.droprate = in_dim, out_dim, mode, droprate
        self.activation_layer = make_activation(activation)
        self.residual_layer = nn.Linear(in_dim, out_dim)
        # real pairs rather than complex64 (the reference's choice: its collective backend lacks complex types)
        self.fourier_weight = nn.ParameterList(
            [nn.Parameter(torch.empty(mode, mode, in_dim, out_dim, 2)) for _ in range(2)])
        for w in self.fourier_weight:
            nn.init.xavier_normal_(w, gain=1.0 / (in_dim * out_dim) * math.sqrt(in_dim + out_dim))

    @refreshes_derived
    def forward(self, X: Tensor) -> Tensor:
        """[N, r, r, in_dim] -> [N, r, r, out_dim]."""
        N, r, _, cin = X.size()
        m, cout = self.mode, self.out_dim
        needs_graph = torch.is_grad_enabled() and (X.requires_grad or self.fourier_weight[0].requires_grad)
        truncated = self.use_truncated_dft and not needs_graph and truncated_dft.supported(r, m)
        if (truncated and self.droprate == 0 and truncated_dft.fused_tail_supported(r, cin, cout, m) and
                gpu_inference(X, self.residual_layer)):
            # only the retained modes are ever computed: no FFT, no transposes, no full-size spectrum; the
            # inverse transform along w, the residual Linear, the add and the activation are one kernel
            return truncated_dft.spectral_modes_apply_linear(
                X.contiguous(), self.fourier_weight[0], self.fourier_weight[1], m,
                linear_weight_kn(self.residual_layer), self.residual_layer.bias,
                activation_name(self.activation_layer))
        if truncated and fused_linear_usable(X, self.residual_layer):
            X0 = X.contiguous()
            Y = truncated_dft.spectral_modes_apply(always_dropout(X0, self.droprate), self.fourier_weight[0],
                                                   self.fourier_weight[1], m)
            return fused_linear(X0, linear_weight_kn(self.residual_layer), self.residual_layer.bias,
                                activation_name(self.activation_layer), Y)
        if (needs_graph and self.use_truncated_dft and self.droprate == 0 and X.is_cuda and X.dtype == torch.float32
                and truncated_dft.supported(r, m) and truncated_dft.spectral_linear_trainable(r, cin, cout, m)):
            # training on the truncated-DFT route: the layer's linear part (residual Linear + spectral term) is one
            # autograd function whose backward runs the adjoint stages on the same kernels
            lin = self.residual_layer
            pre = truncated_dft.spectral_linear_train(X.contiguous(), self.fourier_weight[0], self.fourier_weight[1], m,
                                                      lin.weight, lin.bias, linear_weight_kn(lin))
            return self.activation_layer(pre)
        res = self.residual_layer(X)
        X = always_dropout(X, self.droprate)
        if truncated:
            Y = truncated_dft.spectral_modes_apply(X.contiguous(), self.fourier_weight[0], self.fourier_weight[1], m)
            return self.activation_layer(Y + res)
        X = batched_transpose(X, [N], [r, r], [cin])  # -> [N, in_dim, r, r]
        X_ft = torch.fft.rfft2(X, s=(r, r), norm="ortho")
        w_all = r // 2 + 1
        if needs_graph:
            g0, g1 = transpose_gather_dual(X_ft, [N, cin], r, w_all, m, m, 0, 0, r - m, 0)
            o0 = g0 @ torch.view_as_complex(self.fourier_weight[0])
            o1 = g1 @ torch.view_as_complex(self.fourier_weight[1])
            Out_ft = transpose_scatter_dual(o0, o1, [N, cout], r, w_all, m, m, 0, 0, r - m, 0)
        else:
            Out_ft = spectral_mode_contract(X_ft, self.fourier_weight[0], self.fourier_weight[1], m, m, 0, 0, r - m, 0)
        X = torch.fft.irfft2(Out_ft, s=(r, r), norm="ortho")
        X = batched_transpose(X, [N], [cout], [r, r])  # -> [N, r, r, out_dim]
        return self.activation_layer(X + res)


def convert_gt_state_dict(state_dict: Dict[str, Tensor]) -> Dict[str, Tensor]:
    """Maps a state_dict of the reference's plain-PyTorch model (or of any of its sub-modules) onto the
    accelerated modules: projection weights are transposed (x @ W^T there, x @ W here) and Fourier weights
    go from [Cin, Cout, m, m, 2] (network/layer.py:214-216) to [m, m, Cin, Cout, 2] (network/sp_layer.py:119-121)."""
    out = {}
    for k, v in state_dict.items():
        leaf = k.rsplit(".", 1)[-1]
        if leaf in ("weight_Q", "weight_K", "weight_V"):
            v = v.t().contiguous()
        elif ".fourier_weight." in "." + k and v.dim() == 5:
            v = v.permute(2, 3, 0, 1, 4).contiguous()
        out[k] = v
    return out
