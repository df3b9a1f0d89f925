"""Accelerated Galerkin Transformer for 2-D problems: DownScaler2D ->
Sp_EncoderMixer -> UpScaler2D -> Sp_DecoderRegressor.  Class names,
constructor arguments and parameter names follow the reference's
network/sp_model.py (Sp_EncoderMixer :9-36, Sp_DecoderRegressor :39-64,
Sp_GalerkinTransformer2D :67-113).
"""
import torch
import torch.nn.functional as F
from torch import Tensor, nn

from ..extension.bind.datamove import bilinear_nhwc_affine, denormalize_boundary
from ..extension.bind.linear import fused_linear, linear_supported
from .derived import derived, refreshes_derived, transposed_2d
from .layer import FeedForward, _SplitLinearFunction, always_dropout, gpu_inference
from .model import DownScaler2D, UpScaler2D
from .sp_layer import Sp_EncoderLayer, Sp_SpectralConv2D


class UnitNormalizer:
    """The reference's GaussNormalizer fitted on nothing (dataset/darcy_dataset.py:12-31): mean 0, std 1, eps 1e-5."""

    def __init__(self, mean=0.0, std=1.0, eps=1.0e-5) -> None:
        self.mean, self.std, self.eps = mean, std, eps

    def transform(self, X):
        return (X - self.mean) / (self.std + self.eps)

    def inverse_transform(self, X):
        return X * (self.std + self.eps) + self.mean


class Sp_EncoderMixer(nn.Module):
    def __init__(self, num_layer, dim_hidden, num_head, dim_position, norm_eps, attn_droprate, fc_droprate, xavier,
                 diagonal, symmetric, ffn_dim_hidden, ffn_droprate, ffn_activation) -> None:
        super().__init__()
        self.layers = nn.ModuleList([
            Sp_EncoderLayer(dim_hidden, num_head, dim_position, norm_eps, attn_droprate, fc_droprate, xavier, diagonal,
                            symmetric, ffn_dim_hidden, ffn_droprate, ffn_activation) for _ in range(num_layer)])

    @refreshes_derived
    def forward(self, X: Tensor, position: Tensor) -> Tensor:
        """X [N, ra, ra, dim_hidden], position [N, ra, ra, dim_position] -> [N, ra, ra, dim_hidden]."""
        N, ra, _, C = X.size()
        X = X.reshape(N, ra * ra, C).contiguous()  # a strided residual stream would be re-copied by every Linear
        position = position.reshape(N, ra * ra, position.size(-1))
        for layer in self.layers:
            X = layer(X, position)
        return X.view(N, ra, ra, C)


class Sp_DecoderRegressor(nn.Module):
    def __init__(self, num_layer, in_dim, out_dim, dim_position, dim_spatial_hidden, mode, droprate,
                 activation) -> None:
        super().__init__()
        self.spatial_fc_layer = nn.Linear(in_dim + dim_position, dim_spatial_hidden)
        self.layers = nn.ModuleList([
            Sp_SpectralConv2D(dim_spatial_hidden, dim_spatial_hidden, mode, droprate, activation)
            for _ in range(num_layer)])
        self.ffn_layer = FeedForward(dim_spatial_hidden, out_dim, 2 * dim_position * dim_spatial_hidden, droprate,
                                     activation)

    def _split_weight_kn(self, dim_x: int):
        """spatial_fc_layer.weight as ([dim_x, C], [dim_position, C]): the hidden-feature and the grid columns,
        transposed; derived tensors, rewritten from the parameter at the start of every inference forward."""
        lin = self.spatial_fc_layer  # the specs look the weight up on every call: the parameter may be replaced
        return (derived(self, f"fc_hidden_kn_{dim_x}", lambda: transposed_2d(lin.weight, slice(0, dim_x))),
                derived(self, f"fc_grid_kn_{dim_x}",
                        lambda: transposed_2d(lin.weight, slice(dim_x, lin.weight.size(1)))))

    def accepts_low_resolution(self, X: Tensor, grid: Tensor) -> bool:
        """True when forward(X, grid, resample_to=size) is available for a channels-last X."""
        W, dim_x = self.spatial_fc_layer.weight, X.size(-1)
        return (grid is not None and grid.is_cuda and grid.dtype == torch.float32 and
                gpu_inference(X, grid, W, self.spatial_fc_layer.bias) and linear_supported(dim_x, W.size(0)) and
                W.size(0) % 4 == 0 and 0 < W.size(1) - dim_x <= 4 and grid.size(-1) == W.size(1) - dim_x)

    @refreshes_derived
    def forward(self, X: Tensor, grid: Tensor = None, resample_to=None) -> Tensor:
        """X [N, r, r, dim_hidden], grid [N, r, r, dim_position] -> [N, r, r, dim_target].
        With resample_to = (r, r) (see accepts_low_resolution), X is [N, r_low, r_low, dim_hidden] and stands for
        its bilinear (align_corners) interpolation to r x r: the input layer runs on the low-resolution X, which
        gives the same result up to rounding because the layer is linear and interpolation weights sum to 1, and
        the interpolation then moves dim_spatial_hidden channels instead of dim_hidden."""
        # Linear(cat([X, grid])) without materialising the concatenation: W = [W_x | W_grid]
        W, dim_x = self.spatial_fc_layer.weight, X.size(-1)
        if resample_to is not None:
            w_x, w_grid = self._split_weight_kn(dim_x)
            X = fused_linear(X, w_x, self.spatial_fc_layer.bias, "none")
            # the grid columns are a rank-2 update at the full resolution, applied by the resampling kernel
            X = bilinear_nhwc_affine(X, resample_to, grid.contiguous(), w_grid)
        elif (gpu_inference(X, W, self.spatial_fc_layer.bias) and linear_supported(dim_x, W.size(0)) and
                W.size(1) - dim_x <= 4):
            # the GEMM runs over the hidden features; the grid columns are a rank-2 update in its epilogue
            w_x, w_grid = self._split_weight_kn(dim_x)
            X = fused_linear(X, w_x, self.spatial_fc_layer.bias, "none", x_extra=grid, weight_extra_kn=w_grid)
        elif (X.is_cuda and X.dtype == torch.float32 and grid is not None and grid.is_cuda and
                grid.dtype == torch.float32 and W.dtype == torch.float32 and linear_supported(dim_x, W.size(0)) and
                0 < W.size(1) - dim_x <= 4 and grid.size(-1) == W.size(1) - dim_x and W.size(0) % 4 == 0):
            # under autograd: the same kernel forward, weight gradients by this package's pass over the tokens
            w_x, w_grid = self._split_weight_kn(dim_x)
            X = _SplitLinearFunction.apply(X.contiguous(), grid.contiguous(), W, self.spatial_fc_layer.bias, w_x, w_grid)
        else:
            X = F.linear(X, W[:, :dim_x], self.spatial_fc_layer.bias) + F.linear(grid, W[:, dim_x:])
        for layer in self.layers:
            X = layer(X)
        return self.ffn_layer(X)


class Sp_GalerkinTransformer2D(nn.Module):
    def __init__(self, cfg) -> None:
        super().__init__()
        self.droprate = cfg["drop_module"]
        self.boundary_condition = cfg["boundary_condition"]
        self.normalizer = cfg["target_normalizer"]
        self.down_scaler = DownScaler2D(cfg["resolution_size"], cfg["dim_node"], cfg["dim_hidden"],
                                        cfg["drop_downscaler"], cfg["acti_downscaler"])
        self.encoder_mixer = Sp_EncoderMixer(
            cfg["num_encoder_layer"], cfg["dim_hidden"], cfg["num_head"], cfg["dim_position"], cfg["attn_norm_eps"],
            cfg["drop_encoder_attn"], cfg["drop_encoder_attn_fc"], cfg["attn_xavier"], cfg["attn_diagonal"],
            cfg["attn_symmetric"], cfg["dim_encoder_ffn"], cfg["drop_encoder_ffn"], cfg["acti_encoder_ffn"])
        self.up_scaler = UpScaler2D(cfg["resolution_size"], cfg["dim_hidden"], cfg["dim_hidden"], cfg["drop_upscaler"],
                                    cfg["acti_upscaler"])
        self.decoder_regressor = Sp_DecoderRegressor(
            cfg["num_decoder_layer"], cfg["dim_hidden"], cfg["dim_target"], cfg["dim_position"],
            cfg["dim_spatial_hidden"], cfg["num_frequence_mode"], cfg["drop_decoder_layer"], cfg["acti_decoder_layer"])

    @refreshes_derived
    def forward(self, X: Tensor, position: Tensor, grid: Tensor) -> Tensor:
        """X [N, r, r, dim_node], position [N, ra, ra, dim_position], grid [N, r, r, dim_position]
        -> [N, r, r, dim_target] (de-normalised; zero on the boundary for the Dirichlet condition)."""
        X = always_dropout(self.down_scaler(X), self.droprate)
        X = self.encoder_mixer(X, position)
        if (self.droprate == 0 and self.up_scaler.can_defer_last_resample(X) and
                self.decoder_regressor.accepts_low_resolution(X, grid)):
            # the decoder's input layer moves in front of the up-scaler's last interpolation
            X = self.decoder_regressor(self.up_scaler(X, defer_last_resample=True), grid,
                                       resample_to=self.up_scaler.resolution_size[4])
        else:
            X = always_dropout(self.up_scaler(X), self.droprate)
            X = self.decoder_regressor(X, grid)
        dirichlet = self.boundary_condition == "dirichlet"
        # (a grid with fewer than two rows or columns has no interior: the padded result would change shape)
        affine = self._normalizer_affine(X) if gpu_inference(X) and min(X.shape[1:3]) >= 2 else None
        if affine is not None:
            # de-normalisation and the zero boundary in one pass
            return denormalize_boundary(X, affine[0], affine[1], dirichlet)
        X = self.normalizer.inverse_transform(X)
        if dirichlet:
            X = F.pad(X[:, 1:-1, 1:-1], (0, 0, 1, 1, 1, 1), "constant", 0.0)
        return X

    def _normalizer_affine(self, X: Tensor):
        """(std + eps, mean) of the target normalizer as device tensors of one value or of one value per grid
        point and channel, or None when the normalizer is of another kind.  Cached per device."""
        nz = self.normalizer
        if not all(hasattr(nz, k) for k in ("mean", "std", "eps")):
            return None
        key = (id(nz.mean), id(nz.std), getattr(nz.mean, "_version", None), getattr(nz.std, "_version", None), nz.eps,
               X.device, tuple(X.shape[1:]))
        cache = getattr(self, "_spgt_affine", None)
        if cache is not None and cache[0] == key:
            return cache[1]
        mean, std = nz.mean, nz.std
        if isinstance(mean, Tensor) != isinstance(std, Tensor):
            return None
        if isinstance(mean, Tensor):
            if mean.dtype != torch.float32 or std.dtype != torch.float32:
                return None
            scale = (std + nz.eps).to(X.device)
            shift = mean.to(X.device)
            if scale.numel() != 1 or shift.numel() != 1:
                try:
                    scale = scale.expand(X.shape[1:]).contiguous()
                    shift = shift.expand(X.shape[1:]).contiguous()
                except RuntimeError:
                    return None
            else:
                scale, shift = scale.reshape(1).contiguous(), shift.reshape(1).contiguous()
        else:
            # python numbers: torch multiplies a float32 tensor by float32(std + eps)
            scale = torch.tensor([float(std) + float(nz.eps)], dtype=torch.float32, device=X.device)
            shift = torch.tensor([float(mean)], dtype=torch.float32, device=X.device)
        self._spgt_affine = (key, (scale, shift))
        return scale, shift
