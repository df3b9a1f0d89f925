"""Plain-torch building blocks shared by the accelerated model: the 3x3
convolution block and the two-layer feed-forward net.  Parameter names and
shapes match the reference's network/layer.py:7-24 (ConvResBlock2D) and
:155-174 (FeedForward) so that its checkpoints load unchanged.

As in the reference, dropout is applied whenever the drop rate is non-zero,
also under model.eval() (the reference calls `F.dropout` with its default
training=True); run with drop rates of 0 for deterministic inference.  On the
GPU the fused kernels apply it themselves, with the library's own masks.
"""
import torch
import torch.nn.functional as F
from torch import Tensor, nn

from ..extension.bind.datamove import bias_activation_nchw_
from .._lib import dropout_seed
from ..extension.bind.linear import (dropout_add, ffn_scalar_supported, fused_ffn_scalar, fused_linear, linear_supported,
                                     linear_weight_grad)
from .derived import derived, refreshes_derived, transposed_2d


def make_activation(name: str) -> nn.Module:
    return nn.SiLU() if name == "silu" else nn.ReLU()


def activation_name(module: nn.Module) -> str:
    return "silu" if isinstance(module, nn.SiLU) else "relu"


def linear_weight_kn(lin: nn.Linear) -> Tensor:
    """lin.weight transposed to [in_features, out_features], contiguous: a derived tensor, rewritten from the
    parameter at the start of every inference forward (see derived.py)."""
    return derived(lin, "weight_kn", lambda: transposed_2d(lin.weight))


def _any_requires_grad(sources) -> bool:
    for src in sources:
        if src is None:
            continue
        if isinstance(src, Tensor):
            if src.requires_grad:
                return True
        elif isinstance(src, nn.Module):
            if any(p.requires_grad for p in src.parameters()):
                return True
        elif _any_requires_grad(src):
            return True
    return False


def gpu_inference(X: Tensor, *sources) -> bool:
    """fp32 on a GPU with nothing to differentiate: the case the fused inference kernels serve.  sources: tensors,
    modules (their parameters) or sequences of those; they are only looked at while gradients are enabled, so that
    a forward under torch.no_grad() does not walk the module tree."""
    if not X.is_cuda or X.dtype != torch.float32:
        return False
    return not (torch.is_grad_enabled() and (X.requires_grad or _any_requires_grad(sources)))


def fused_linear_usable(X: Tensor, *linears: nn.Linear) -> bool:
    """gpu_inference, and the fused linear kernel has a variant for every layer's shape."""
    return gpu_inference(X, *linears) and all(linear_supported(l.in_features, l.out_features) for l in linears)


def _weight_and_bias_grad(x: Tensor, g: Tensor, has_bias: bool):
    """(dW [out, in], db [out] or None) of y = x @ W^T + b from g = dL/dy: one pass over x and g with a fixed
    summation order.  The pass writes rows of out features, which must be a multiple of 4; a Linear with a narrow
    output (the regression head's 128 -> 1) is served with the roles swapped, dW = g^T x."""
    out_f, in_f = g.shape[-1], x.shape[-1]
    if out_f % 4 == 0:
        dw_kn, db = linear_weight_grad(x, g)
        return dw_kn.t(), (db if has_bias else None)
    dw, _ = linear_weight_grad(g, x)  # [out, in]
    return dw, (g.reshape(-1, out_f).sum(0) if has_bias else None)


class _LinearFunction(torch.autograd.Function):
    """x @ W^T + b (+ residual) for an nn.Linear's parameters, forward and backward on this package's kernels:
    the fused linear kernel forward and for dX = g @ W where it has a variant for the shape (the library's GEMM
    otherwise), and one pass over x and g for dW = g^T x and db (the library's GEMM for that product, whose
    contraction runs over all tokens, takes 250 us at 65k tokens).
    relu: the result is relu(x @ W^T + b), formed in the forward kernel's epilogue; the backward masks the incoming
    gradient with the saved result.  with_identity: x is handed on as a second result, for a caller that also adds
    it as a residual further on: that residual's gradient then arrives here and rides in the dX product."""

    @staticmethod
    def forward(ctx, x, weight, bias, weight_kn, residual, relu=False, with_identity=False):
        ctx.has_bias, ctx.has_residual, ctx.relu, ctx.with_identity = bias is not None, residual is not None, relu, with_identity
        if weight_kn is not None:
            y = fused_linear(x, weight_kn, bias, "relu" if relu else "none", residual)
        else:
            y = F.linear(x, weight, bias)
            if residual is not None:
                y = y + residual
            if relu:
                y = torch.relu_(y)
        ctx.save_for_backward(x, weight, *([y] if relu else []))
        return (y, x.view_as(x)) if with_identity else y

    @staticmethod
    def backward(ctx, g, g_identity=None):
        x, weight = ctx.saved_tensors[:2]
        g = g.contiguous()
        if ctx.relu:
            g = torch.ops.aten.threshold_backward(g, ctx.saved_tensors[2], 0)
        dx = None
        if ctx.needs_input_grad[0]:
            w = weight.detach()
            gi = None if g_identity is None else g_identity.reshape(-1, x.shape[-1]).contiguous()
            # g @ W: the fused kernel where it has a variant for [out -> in], else the library's GEMM
            if linear_supported(w.shape[0], w.shape[1]):
                dx = fused_linear(g.reshape(-1, w.shape[0]), w.contiguous(), None, "none", gi).view(x.shape)
            else:
                dx = torch.matmul(g, w)
                if gi is not None:
                    dx = dx + gi.view(x.shape)
        elif g_identity is not None:
            dx = g_identity
        dw = db = None
        if ctx.needs_input_grad[1] or (ctx.has_bias and ctx.needs_input_grad[2]):
            dw, db = _weight_and_bias_grad(x, g, ctx.has_bias)
        return dx, dw, db, None, (g if ctx.has_residual else None), None, None


def linear_trainable(X: Tensor, lin: nn.Linear) -> bool:
    """True when linear_train serves lin(X): fp32 on a GPU and a row length the weight-gradient pass can write
    (out_features, or else in_features, a multiple of 4)."""
    return (X.is_cuda and X.dtype == torch.float32 and lin.weight.dtype == torch.float32 and
            (lin.out_features % 4 == 0 or lin.in_features % 4 == 0))


def linear_train(X: Tensor, lin: nn.Linear, residual: Tensor = None, relu: bool = False, with_identity: bool = False):
    """lin(X) (+ residual), or relu of it, with an autograd graph, on this package's kernels (see _LinearFunction);
    with_identity: (result, X handed on for use as a residual further on)."""
    kn = linear_weight_kn(lin) if linear_supported(lin.in_features, lin.out_features) else None
    return _LinearFunction.apply(X, lin.weight, lin.bias, kn, residual, relu, with_identity)


class _SplitLinearFunction(torch.autograd.Function):
    """Linear(cat([x, extra], -1)) without the concatenation, for up to four extra columns (the decoder's input
    layer on hidden features and grid coordinates): forward = the fused linear kernel with the extra columns as a
    rank-r update in its epilogue; backward: dX = g @ W[:, :in_x] by the library's GEMM, the two column blocks of
    dW and db by this package's pass over the tokens."""

    @staticmethod
    def forward(ctx, x, extra, weight, bias, weight_x_kn, weight_extra_kn):
        ctx.save_for_backward(x, extra, weight)
        ctx.has_bias = bias is not None
        return fused_linear(x, weight_x_kn, bias, "none", x_extra=extra, weight_extra_kn=weight_extra_kn)

    @staticmethod
    def backward(ctx, g):
        x, extra, weight = ctx.saved_tensors
        g = g.contiguous()
        in_x = x.shape[-1]
        w = weight.detach()
        dx = torch.matmul(g, w[:, :in_x]) if ctx.needs_input_grad[0] else None
        dextra = torch.matmul(g, w[:, in_x:]) if ctx.needs_input_grad[1] else None
        dw = db = None
        if ctx.needs_input_grad[2] or (ctx.has_bias and ctx.needs_input_grad[3]):
            dwx, db = _weight_and_bias_grad(x, g, ctx.has_bias)
            dwe, _ = _weight_and_bias_grad(extra, g, False)
            dw = torch.cat([dwx, dwe], dim=1)
        return dx, dextra, dw, db, None, None


def always_dropout(X: Tensor, p: float) -> Tensor:
    return F.dropout(X, p=p) if p > 0 else X


class _DropoutAddFunction(torch.autograd.Function):
    """residual + dropout(y) in one pass; the backward regenerates the mask from the saved seed words."""

    @staticmethod
    def forward(ctx, y, residual, p):
        seed = dropout_seed(y.device)
        ctx.seed, ctx.p, ctx.has_residual = seed, p, residual is not None
        return dropout_add(y.contiguous(), None if residual is None else residual.contiguous(), p, seed)

    @staticmethod
    def backward(ctx, g):
        dy = dropout_add(g.contiguous(), None, ctx.p, ctx.seed) if ctx.needs_input_grad[0] else None
        return dy, (g if ctx.has_residual else None), None


def always_dropout_add(Y: Tensor, residual: Tensor, p: float) -> Tensor:
    """residual + F.dropout(Y, p) (the dropout always on, as in the reference), or the dropout alone without a
    residual.  On the GPU in fp32 it is one kernel with the library's own masks, forward and backward."""
    if p > 0 and Y.is_cuda and Y.dtype == torch.float32 and Y.shape[-1] % 4 == 0 and 0 < p < 1 and (
            residual is None or (residual.is_cuda and residual.dtype == torch.float32 and residual.shape == Y.shape)):
        return _DropoutAddFunction.apply(Y, residual, p)
    Y = always_dropout(Y, p)
    return Y if residual is None else residual + Y


class ConvResBlock2D(nn.Module):
    """conv3x3 -> dropout -> activation on [N, C, H, W]."""

    def __init__(self, in_dim, out_dim, kernel_size, padding, droprate, activation) -> None:
        super().__init__()
        self.droprate = droprate
        self.conv_layer = nn.Conv2d(in_dim, out_dim, kernel_size=kernel_size, padding=padding)
        self.activation_layer = make_activation(activation)

    def fusable(self, X: Tensor) -> bool:
        """Inference: the bias, the dropout (the reference's F.dropout, on by default in inference too) and the
        activation can ride in the caller's next kernel."""
        return 0 <= self.droprate < 1 and gpu_inference(X, self)

    def conv_raw(self, X: Tensor) -> Tensor:
        """The convolution without its bias (to be added by the kernel that consumes the result)."""
        c = self.conv_layer
        Y = F.conv2d(X, c.weight, None, c.stride, c.padding, c.dilation, c.groups)
        return Y if Y.is_contiguous() else Y.contiguous()

    def forward(self, X: Tensor, extra_activations: int = 0) -> Tensor:
        """conv -> dropout -> activation, the activation applied 1 + extra_activations times."""
        if self.fusable(X):
            return bias_activation_nchw_(self.conv_raw(X), self.conv_layer.bias, activation_name(self.activation_layer),
                                         1 + extra_activations, droprate=self.droprate)
        X = self.activation_layer(always_dropout(self.conv_layer(X), self.droprate))
        for _ in range(extra_activations):
            X = self.activation_layer(X)
        return X


class FeedForward(nn.Module):
    """Linear -> activation -> Linear -> dropout on [N, seqlen, in_dim]."""

    def __init__(self, in_dim, out_dim, dim_hidden, droprate, activation) -> None:
        super().__init__()
        self.droprate = droprate
        self.layer1 = nn.Linear(in_dim, dim_hidden)
        self.layer2 = nn.Linear(dim_hidden, out_dim)
        self.activation_layer = make_activation(activation)

    @refreshes_derived
    def forward(self, X: Tensor, residual: Tensor = None) -> Tensor:
        """ffn(X), or residual + ffn(X) when a residual is given."""
        if (self.layer2.out_features == 1 and residual is None and
                gpu_inference(X, self) and
                ffn_scalar_supported(self.layer1.in_features, self.layer1.out_features)):
            # single output feature: both layers in one kernel, the hidden activations stay in registers
            Y = fused_ffn_scalar(X, linear_weight_kn(self.layer1), self.layer1.bias, self.layer2.weight.detach(),
                                 self.layer2.bias, activation_name(self.activation_layer))
            return always_dropout(Y, self.droprate)
        if fused_linear_usable(X, self.layer1, self.layer2) and (residual is None or self.droprate == 0):
            # inference: bias + activation and bias + residual ride in the two GEMMs' epilogues
            H = fused_linear(X, linear_weight_kn(self.layer1), self.layer1.bias, activation_name(self.activation_layer))
            Y = fused_linear(H, linear_weight_kn(self.layer2), self.layer2.bias, "none", residual)
            return always_dropout(Y, self.droprate)
        if linear_trainable(X, self.layer1) and linear_trainable(X, self.layer2):
            # under autograd: the same kernels, with the weight gradients by this package's pass over the tokens
            relu = isinstance(self.activation_layer, nn.ReLU)
            identity = residual is X and X.is_contiguous()
            Hd = linear_train(X, self.layer1, None, relu, identity)
            if identity:
                Hd, residual = Hd
            if not relu:
                Hd = self.activation_layer(Hd)
            if self.droprate == 0:
                return linear_train(Hd, self.layer2, residual)
            return always_dropout_add(linear_train(Hd, self.layer2), residual, self.droprate)
        Y = always_dropout(self.layer2(self.activation_layer(self.layer1(X))), self.droprate)
        return Y if residual is None else residual + Y
