"""Writes tests/golden/*.npz from the reference's own plain-PyTorch modules.

Run in the development container only (it needs the reference checkout, by
default /root/reference, which is never shipped):

    python tests/golden/make_golden.py [--reference /root/reference]

It imports network/layer.py and network/model.py of the reference (pure torch,
CPU), builds each module at a small size with every drop rate 0 and a fixed
seed, and stores the module's parameters, inputs and output.  The fixtures pin
how the pieces are composed (concat orders, channel splits, head merge,
boundary handling) - the part of the oracle that closed forms cannot pin.
Only data is written: tensors as float32 arrays plus a few integers.
"""
import argparse
import os
import sys
import tempfile

import numpy as np
import torch

HERE = os.path.dirname(os.path.abspath(__file__))


def import_reference(ref_root):
    """Makes the checkout importable under the package name its files use."""
    tmp = tempfile.mkdtemp(prefix="spgt_ref_")
    os.symlink(ref_root, os.path.join(tmp, "SpGT"))
    sys.path.insert(0, tmp)
    import SpGT.network.layer as layer  # noqa: E402
    import SpGT.network.model as model  # noqa: E402
    return layer, model


def randomize(module, gen):
    """Replaces every parameter by N(0, 0.3^2) noise around its initial value so
    that biases, LayerNorm affines and Fourier weights are all non-trivial."""
    with torch.no_grad():
        for prm in module.parameters():
            prm.add_(0.3 * torch.randn(prm.shape, generator=gen))


def save(name, module, inputs, output, **meta):
    arrays = {}
    if module is not None:
        arrays.update({f"param/{k}": v.detach().numpy() for k, v in module.state_dict().items()})
    arrays.update({f"in/{k}": v.detach().numpy() for k, v in inputs.items()})
    arrays["out"] = output.detach().numpy()
    arrays.update({f"meta/{k}": np.asarray(v) for k, v in meta.items()})
    path = os.path.join(HERE, name + ".npz")
    np.savez_compressed(path, **arrays)
    print(f"{path}: {os.path.getsize(path) / 1024:.1f} KiB")


class UnitNormalizer:
    """GaussNormalizer() with no data: mean 0, std 1, eps 1e-5 (dataset/darcy_dataset.py:12-31)."""

    def inverse_transform(self, X):
        return X * (1.0 + 1.0e-5) + 0.0


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--reference", default="/root/reference")
    args = ap.parse_args()
    layer, model = import_reference(args.reference)
    torch.manual_seed(20240607)
    gen = torch.Generator().manual_seed(1234)
    rn = lambda *shape: torch.randn(*shape, generator=gen)

    with torch.no_grad():
        # GalerkinAttention, dim_position 0 and 2
        for dp in (0, 2):
            B, S = 2, 50 if dp == 0 else 77
            m = layer.GalerkinAttention(128, 4, dp, 1e-6, 0.0, 0.0, 1.0, 0.01, False)
            randomize(m, gen)
            x, pos = rn(B, S, 128), torch.rand(B, S, dp, generator=gen)
            save(f"attention_dp{dp}", m, {"x": x, "position": pos}, m(x, x, x, pos),
                 num_head=4, dim_position=dp, norm_eps=1e-6)
            # the three static pieces, for operator-level checks (parameters: attention_dp*.npz)
            Q = m.multihead_projection_with_position(x, m.weight_Q, m.bias_Q, pos, 4, 32, dp)
            K = m.multihead_projection_layernorm_with_position(
                x, m.weight_K, m.bias_K, m.ln_weight_K, m.ln_bias_K, pos, 1e-6, 4, 32, dp)
            V = m.multihead_projection_layernorm_with_position(
                x, m.weight_V, m.bias_V, m.ln_weight_V, m.ln_bias_V, pos, 1e-6, 4, 32, dp)
            A = m.multihead_galerkin_attention(Q, K, V, 0.0)
            save(f"attention_pieces_dp{dp}", None, {"x": x, "position": pos, "Q": Q, "K": K, "V": V}, A,
                 num_head=4, dim_position=dp, norm_eps=1e-6)

        # EncoderLayer (dp 2, silu)
        m = layer.EncoderLayer(128, 4, 2, 1e-6, 0.0, 0.0, 0.01, 0.01, False, 256, 0.0, "silu")
        randomize(m, gen)
        x, pos = rn(2, 45, 128), torch.rand(2, 45, 2, generator=gen)
        save("encoder_layer", m, {"x": x, "position": pos}, m(x, pos),
             num_head=4, dim_position=2, norm_eps=1e-6, activation="silu")

        # SpectralConv2D, odd grid, Cin != Cout
        m = layer.SpectralConv2D(6, 4, 3, 0.0, "silu")
        randomize(m, gen)
        x = rn(2, 9, 9, 6)
        save("spectral_conv2d", m, {"x": x}, m(x), mode=3, activation="silu")

        # DownScaler2D / UpScaler2D
        rs = ((21, 21), (15, 15), (11, 11), (15, 15), (21, 21))
        m = model.DownScaler2D(rs, 1, 128, 0.0, "relu")
        randomize(m, gen)
        x = rn(2, 21, 21, 1)
        save("down_scaler", m, {"x": x}, m(x), resolution_size=np.asarray(rs), activation="relu")
        m = model.UpScaler2D(rs, 128, 128, 0.0, "silu")
        randomize(m, gen)
        x = rn(2, 11, 11, 128)
        save("up_scaler", m, {"x": x}, m(x), resolution_size=np.asarray(rs), activation="silu")

        # full model
        cfg = dict(
            drop_module=0.0, boundary_condition="dirichlet", target_normalizer=UnitNormalizer(),
            resolution_size=rs, dim_node=1, dim_hidden=128, drop_downscaler=0.0, acti_downscaler="relu",
            num_encoder_layer=2, num_head=4, dim_position=2, attn_norm_eps=1e-6, drop_encoder_attn=0.0,
            drop_encoder_attn_fc=0.0, attn_xavier=0.01, attn_diagonal=0.01, attn_symmetric=False,
            dim_encoder_ffn=256, drop_encoder_ffn=0.0, acti_encoder_ffn="relu", drop_upscaler=0.0,
            acti_upscaler="silu", num_decoder_layer=2, dim_target=1, dim_spatial_hidden=32,
            num_frequence_mode=4, drop_decoder_layer=0.0, acti_decoder_layer="silu",
        )
        m = model.GalerkinTransformer2D(cfg)
        randomize(m, torch.Generator().manual_seed(99))  # smaller perturbation would also do
        lin = lambda n: torch.linspace(0, 1, n)
        mesh = lambda n: torch.stack(torch.meshgrid(lin(n), lin(n), indexing="ij"), dim=-1)[None].repeat(2, 1, 1, 1)
        x, pos, grid = rn(2, 21, 21, 1), mesh(11), mesh(21)
        meta = {k: v for k, v in cfg.items() if isinstance(v, (int, float, str, bool))}
        save("galerkin_transformer_2d", m, {"x": x, "position": pos, "grid": grid}, m(x, pos, grid),
             resolution_size=np.asarray(rs), **meta)


if __name__ == "__main__":
    main()
