"""Plain-torch building blocks shared by the accelerated model: the 3x3
convolution block and the two-layer feed-forward net.  Parameter names and
shapes match the reference's network/layer.py:7-24 (ConvResBlock2D) and
:155-174 (FeedForward) so that its checkpoints load unchanged.

As in the reference, `F.dropout` is applied with its default training=True
whenever the drop rate is non-zero, also under model.eval(); run with drop
rates of 0 for deterministic inference.
"""
import torch
import torch.nn.functional as F
from torch import Tensor, nn


def make_activation(name: str) -> nn.Module:
    return nn.SiLU() if name == "silu" else nn.ReLU()


def always_dropout(X: Tensor, p: float) -> Tensor:
    return F.dropout(X, p=p) if p > 0 else X


class ConvResBlock2D(nn.Module):
    """conv3x3 -> dropout -> activation on [N, C, H, W]."""

    def __init__(self, in_dim, out_dim, kernel_size, padding, droprate, activation) -> None:
        super().__init__()
        self.droprate = droprate
        self.conv_layer = nn.Conv2d(in_dim, out_dim, kernel_size=kernel_size, padding=padding)
        self.activation_layer = make_activation(activation)

    def forward(self, X: Tensor) -> Tensor:
        return self.activation_layer(always_dropout(self.conv_layer(X), self.droprate))


class FeedForward(nn.Module):
    """Linear -> activation -> Linear -> dropout on [N, seqlen, in_dim]."""

    def __init__(self, in_dim, out_dim, dim_hidden, droprate, activation) -> None:
        super().__init__()
        self.droprate = droprate
        self.layer1 = nn.Linear(in_dim, dim_hidden)
        self.layer2 = nn.Linear(dim_hidden, out_dim)
        self.activation_layer = make_activation(activation)

    def forward(self, X: Tensor) -> Tensor:
        return always_dropout(self.layer2(self.activation_layer(self.layer1(X))), self.droprate)
