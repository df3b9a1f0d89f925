"""Down- and up-scalers around the encoder: 3x3 convolutions with bilinear
align_corners resampling.  Inference fuses them into this package's kernels
where it can (the down-scaler's three middle convolutions stay with the
library); under autograd the resamplings, the down-scaler's first stage and
the up-scaler's convolution (as a Linear on the low-resolution tokens plus a
gather) run on this package's kernels forward and backward.  Structure,
parameter names and shapes follow the reference's network/model.py:7-39
(DownScaler2D) and :42-65 (UpScaler2D).
"""
import torch
import torch.nn.functional as F
from torch import Tensor, nn

from ..extension.bind.datamove import (bilinear_align_corners, bilinear_align_corners_nhwc, bilinear_nhwc_affine,
                                       bilinear_nhwc_train, bilinear_to_nhwc_train, bilinear_train,
                                       bilinear_resample, bilinear_resample_concat, conv3x3_resample,
                                       conv3x3_resample_train,
                                       conv3x3_resample_supported, upsample_conv3x3_gather,
                                       upsample_conv3x3_gather_train)
from ..extension.bind.linear import fused_linear, linear_supported
from .derived import derived, refreshes_derived
from .layer import ConvResBlock2D, _LinearFunction, activation_name, always_dropout, gpu_inference, make_activation


def get_resolution_size(r_large: int, r_small: int):
    """The five grid sizes (fine, mid, attention, mid, fine) of the two down- and two up-sampling steps
    around the encoder, as the reference derives them (common/trivial.py:78-96): the side ratio of one step,
    sqrt(r_small / r_large), is rounded to four decimals and then to a multiple of 0.005, upwards when the last
    digit the rounded number prints with is below 5 (whatever decimal place that digit stands in: the reference
    reads it off the printed number, and configurations depend on that), and r_mid = round(r_large * ratio) - 1.
    (211, 71) -> 122, (141, 71) -> 99, (421, 71) -> 172, (512, 256) -> 363."""
    import numpy as np
    # The reference rounds numpy scalars (np.sqrt's result), and round() of a numpy scalar scales, rounds half to
    # even and unscales, which differs from Python's exactly-rounded round() on ties such as 0.5825 and 0.4975
    # ((56, 19) -> 31, (198, 49) -> 98): numpy's rounding is used here for that reason.
    step = 5.0e-3
    ratio = np.round(np.sqrt(r_small / r_large), 4)
    last_printed_digit = int(repr(float(ratio))[-1])
    coarse = float(np.round(ratio, 3)) + (step if last_printed_digit < 5 else 0.0)
    r_mid = round(r_large * (int(coarse / step + 0.5) * step)) - 1
    fine, mid, small = (r_large, r_large), (r_mid, r_mid), (r_small, r_small)
    return (fine, mid, small, mid, fine)


def _channels_last_memory(X: Tensor) -> bool:
    """True for an [N, C, H, W] tensor that is a permuted view of a contiguous [N, H, W, C] one."""
    return X.dim() == 4 and not X.is_contiguous() and X.permute(0, 2, 3, 1).is_contiguous()


def resample(X: Tensor, size) -> Tensor:
    """Bilinear, align_corners=True, on [N, C, H, W].  A channels-last input gives a channels-last result, as
    F.interpolate does."""
    if torch.is_grad_enabled() and X.requires_grad:
        if not (X.is_cuda and X.dtype == torch.float32 and X.dim() == 4):
            return F.interpolate(X, size=tuple(size), mode="bilinear", align_corners=True)
        if _channels_last_memory(X) and X.size(1) % 4 == 0:
            return bilinear_nhwc_train(X.permute(0, 2, 3, 1), tuple(size)).permute(0, 3, 1, 2)
        return bilinear_train(X, tuple(size))
    return bilinear_align_corners(X.contiguous(), tuple(size))


def resample_to_nhwc(X: Tensor, size) -> Tensor:
    """Bilinear, align_corners=True, [N, C, H, W] -> [N, H', W', C] (contiguous)."""
    if torch.is_grad_enabled() and X.requires_grad:
        if not (X.is_cuda and X.dtype == torch.float32 and X.dim() == 4):
            return F.interpolate(X, size=tuple(size), mode="bilinear", align_corners=True).permute(0, 2, 3, 1)
        if X.size(1) % 4 != 0:
            return bilinear_train(X, tuple(size)).permute(0, 2, 3, 1)
        if _channels_last_memory(X):
            return bilinear_nhwc_train(X.permute(0, 2, 3, 1), tuple(size))
        return bilinear_to_nhwc_train(X, tuple(size))
    return bilinear_align_corners_nhwc(X.contiguous(), tuple(size))


def nhwc_to_nchw(X: Tensor) -> Tensor:
    """[N, H, W, C] -> [N, C, H, W] with plain row-major strides.  For C == 1 the permuted view is already
    dense but its strides look channels-last, which makes the convolution library answer in channels-last."""
    N, H, W, C = X.shape
    X = X.permute(0, 3, 1, 2).contiguous()
    return X.as_strided((N, C, H, W), (C * H * W, H * W, W, 1))


class DownScaler2D(nn.Module):
    """[N, r, r, in_dim] -> [N, r_attn, r_attn, out_dim] in two resampling steps; the three
    stacked convolutions after the first step are concatenated along channels."""

    def __init__(self, resolution_size, in_dim, out_dim, droprate, activation) -> None:
        super().__init__()
        self.resolution_size = resolution_size
        d1 = d2 = out_dim // 3
        d3 = out_dim - d1 - d2
        self.conv0 = ConvResBlock2D(in_dim, out_dim, 3, 1, droprate, activation)
        self.conv1 = ConvResBlock2D(out_dim, d1, 3, 1, droprate, activation)
        self.conv2 = ConvResBlock2D(d1, d2, 3, 1, droprate, activation)
        self.conv3 = ConvResBlock2D(d2, d3, 3, 1, droprate, activation)
        self.activation_layer = make_activation(activation)

    def forward(self, X: Tensor) -> Tensor:
        fused = gpu_inference(X, self)
        act = activation_name(self.activation_layer)
        c0 = self.conv0.conv_layer
        if (fused and self.conv0.fusable(X) and conv3x3_resample_supported(X.size(-1)) and c0.kernel_size == (3, 3) and
                c0.padding == (1, 1) and c0.stride == (1, 1) and c0.dilation == (1, 1) and c0.groups == 1):
            # few input channels: convolution, bias, activation, resampling and the scaler's activation in one
            # pass straight from the channels-last input; the full-resolution convolution output is never stored
            X = conv3x3_resample(X.contiguous(), c0.weight, c0.bias, self.resolution_size[1],
                                 pre_activation=activation_name(self.conv0.activation_layer), post_activation=act,
                                 droprate=self.conv0.droprate)
        elif fused and self.conv0.fusable(X) and self.conv0.droprate == 0:
            X = nhwc_to_nchw(X)
            # conv0's bias and activation, the resampling and the scaler's activation in one pass
            X = bilinear_resample(self.conv0.conv_raw(X), self.resolution_size[1], pre_bias=self.conv0.conv_layer.bias,
                                  pre_activation=activation_name(self.conv0.activation_layer), post_activation=act)
        elif (torch.is_grad_enabled() and not X.requires_grad and X.is_cuda and X.dtype == torch.float32 and
                X.dim() == 4 and c0.weight.dtype == torch.float32 and conv3x3_resample_supported(X.size(-1)) and
                c0.kernel_size == (3, 3) and c0.padding == (1, 1) and c0.stride == (1, 1) and c0.dilation == (1, 1) and
                c0.groups == 1 and c0.padding_mode == "zeros" and 0 <= self.conv0.droprate < 1):
            # training on the model's input field: the same single pass forward, and a backward that forms the
            # full-resolution convolution, dropout and activation again instead of storing them
            X = self.activation_layer(conv3x3_resample_train(
                X, c0.weight, c0.bias, self.resolution_size[1], activation_name(self.conv0.activation_layer),
                self.conv0.droprate))
        else:
            X = self.activation_layer(resample(self.conv0(nhwc_to_nchw(X)), self.resolution_size[1]))
        X1 = self.conv1(X)
        X2 = self.conv2(X1)
        if fused and self.conv3.fusable(X2) and (X1.size(1) + X2.size(1) + self.conv3.conv_layer.out_channels) % 4 == 0:
            # the second resampling reads the three blocks where they are (no concatenated tensor), gives the last
            # one its bias and activation on the way, and writes channels-last: the scaler's activation commutes
            # with the permute
            return bilinear_resample_concat(
                [X1, X2, self.conv3.conv_raw(X2)], self.resolution_size[2],
                pre_biases=[None, None, self.conv3.conv_layer.bias], pre_flags=[0, 0, 1],
                pre_activation=activation_name(self.conv3.activation_layer), post_activation=act,
                pre_droprate=self.conv3.droprate)
        X3 = self.conv3(X2)
        X = torch.cat([X1, X2, X3], dim=1)
        # the activation commutes with the permute, so the second resampling can write channels-last directly
        if fused:
            return bilinear_resample(X, self.resolution_size[2], dst_nhwc=True, post_activation=act)
        return self.activation_layer(resample_to_nhwc(X, self.resolution_size[2]))


class UpScaler2D(nn.Module):
    """[N, r_attn, r_attn, in_dim] -> [N, r, r, out_dim]: resample, conv block, activation (again), resample."""

    def __init__(self, resolution_size, in_dim, out_dim, droprate, activation) -> None:
        super().__init__()
        self.resolution_size = resolution_size
        self.droprate = droprate
        self.conv = ConvResBlock2D(in_dim, out_dim, 3, 1, droprate, activation)
        self.activation_layer = make_activation(activation)

    def can_defer_last_resample(self, X: Tensor) -> bool:
        """True when forward(X, defer_last_resample=True) is available: fused inference with one kind of activation."""
        return (gpu_inference(X, self) and self.droprate == 0 and self.conv.droprate == 0 and
                self.conv.fusable(X) and type(self.conv.activation_layer) is type(self.activation_layer))

    def _tap_weight_kn(self) -> Tensor:
        """The convolution's weight as [Cin, 9 * Cout], column (3 ky + kx) * Cout + co: the nine per-tap 1x1
        products as one GEMM operand; a derived tensor, rewritten from the parameter at the start of every
        inference forward."""
        w = self.conv.conv_layer.weight
        if w.stride(2) != 3 * w.stride(3):  # the nine taps are walked as one axis
            return w.detach().permute(1, 2, 3, 0).reshape(w.size(1), 9 * w.size(0)).contiguous()
        conv = self.conv.conv_layer

        def spec():  # looks the weight up on every call: the parameter may be replaced
            w = conv.weight
            cout, cin = w.size(0), w.size(1)
            return (cin, 9 * cout), [(w, 0, (cin, 9, cout), (w.stride(1), w.stride(3), w.stride(0)), 0,
                                      (9 * cout, cout, 1))]

        return derived(self, "tap_weight_kn", spec)

    def _mixes_before_resampling(self, X: Tensor) -> bool:
        """True when interpolate -> conv3x3 -> activations is computed as GEMM at the low resolution + gather:
        fused inference, a plain 3x3 convolution, one kind of activation, and enough up-sampling to pay."""
        c = self.conv.conv_layer
        size = self.resolution_size[3]
        size = (size, size) if isinstance(size, int) else size
        return (self.can_defer_last_resample(X) and c.kernel_size == (3, 3) and c.padding == (1, 1) and
                c.stride == (1, 1) and c.dilation == (1, 1) and c.groups == 1 and c.padding_mode == "zeros" and
                c.out_channels % 4 == 0 and linear_supported(c.in_channels, 9 * c.out_channels) and
                size[0] * size[1] >= 2 * X.size(1) * X.size(2))

    def _trains_mixing_before_resampling(self, X: Tensor) -> bool:
        """True when the training route can take interpolate -> conv3x3 as Linear + gather (see forward)."""
        c = self.conv.conv_layer
        size = self.resolution_size[3]
        size = (size, size) if isinstance(size, int) else tuple(size)
        return (torch.is_grad_enabled() and X.is_cuda and X.dtype == torch.float32 and X.dim() == 4 and
                c.weight.dtype == torch.float32 and c.kernel_size == (3, 3) and c.padding == (1, 1) and
                c.stride == (1, 1) and c.dilation == (1, 1) and c.groups == 1 and c.padding_mode == "zeros" and
                c.out_channels % 4 == 0 and linear_supported(c.in_channels, 9 * c.out_channels) and
                size[0] * size[1] >= 2 * X.size(1) * X.size(2) and
                # the adjoint walks the outputs around a source pixel: bounded up-sampling only
                size[0] <= 3 * X.size(1) and size[1] <= 3 * X.size(2))

    def _mid_resolution_nhwc(self, X: Tensor) -> Tensor:
        """interpolate -> conv -> activation -> activation as [N, r_mid, r_mid, out_dim] channels-last."""
        N, H, W, C = X.shape
        c = self.conv.conv_layer
        # conv(interp(X)) = sum over the taps of shifted interp(X . W_tap): the channel mixing runs on the
        # low-resolution tokens, (r_mid / r_attn)^2 times fewer than the convolution would see
        Z = fused_linear(X.reshape(N * H * W, C), self._tap_weight_kn())
        return upsample_conv3x3_gather(Z.view(N, H, W, 9, c.out_channels), c.bias, self.resolution_size[3],
                                       activation_name(self.activation_layer), 2)

    @refreshes_derived
    def forward(self, X: Tensor, defer_last_resample: bool = False) -> Tensor:
        """With defer_last_resample (see can_defer_last_resample) the result is the channels-last tensor at
        resolution_size[3], [N, r_mid, r_mid, out_dim], and the caller owes the interpolation to resolution_size[4]:
        a Linear over the channels commutes with it and is cheaper at the lower resolution."""
        if self._mixes_before_resampling(X):
            X = self._mid_resolution_nhwc(X.contiguous())
            return X if defer_last_resample else bilinear_nhwc_affine(X, self.resolution_size[4])
        if defer_last_resample:
            X = bilinear_resample(X.contiguous(), self.resolution_size[3], src_nhwc=True)
            # the block's bias, its activation and the scaler's own on the way to channels-last: a resampling to
            # the same size has weights (1, 0) and copies the samples exactly
            Y = self.conv.conv_raw(X)
            return bilinear_resample(Y, tuple(Y.shape[-2:]), dst_nhwc=True, pre_bias=self.conv.conv_layer.bias,
                                     pre_activation=activation_name(self.activation_layer), pre_count=2)
        if gpu_inference(X, self) and self.droprate == 0:
            # channels-last in, NCHW out for the convolution; the block's bias and activation and the
            # scaler's own activation are one in-place pass (an upsampling reads every source sample
            # several times, so they are not applied inside it); the second resampling writes channels-last
            X = bilinear_resample(X.contiguous(), self.resolution_size[3], src_nhwc=True)
            if type(self.conv.activation_layer) is type(self.activation_layer):
                X = self.conv(X, extra_activations=1)
            else:
                X = self.activation_layer(self.conv(X))
            return bilinear_resample(X, self.resolution_size[4], dst_nhwc=True)
        if self._trains_mixing_before_resampling(X):
            # under autograd the same reordering: the convolution's channel mixing as a Linear on the low-resolution
            # tokens (forward, dX and dW on this package's kernels), then the nine-tap gather, whose backward is
            # its adjoint; the library convolution (forward, data and weight gradient) and the first
            # interpolation do not run
            N, H, W, C = X.shape
            c = self.conv.conv_layer
            w_taps = c.weight.permute(2, 3, 0, 1).reshape(9 * c.out_channels, c.in_channels)  # rows (ky, kx, co)
            Z = _LinearFunction.apply(X.reshape(N * H * W, C), w_taps, None, self._tap_weight_kn(), None)
            Y = upsample_conv3x3_gather_train(Z.view(N, H, W, 9, c.out_channels), c.bias, self.resolution_size[3])
            Y = self.conv.activation_layer(always_dropout(Y, self.conv.droprate))
            Y = self.activation_layer(always_dropout(Y, self.droprate))
            return bilinear_nhwc_train(Y, tuple(self.resolution_size[4]))
        X = resample(X.permute(0, 3, 1, 2), self.resolution_size[3])
        X = self.activation_layer(always_dropout(self.conv(X), self.droprate))
        return resample_to_nhwc(X, self.resolution_size[4])
