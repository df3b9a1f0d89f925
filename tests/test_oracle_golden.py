"""The oracle against vectors written from the reference's own PyTorch modules
(tests/golden/make_golden.py).  Same library, same machine: differences are a
few ulps, so the bound is tight enough to catch any composition mistake."""
import pytest
import torch

from conftest import load_golden, max_rel
from oracle import spgt_oracle as O

TOL = 2e-6


@pytest.mark.parametrize("dp", [0, 2])
def test_attention_module(dp):
    p, i, out, meta = load_golden(f"attention_dp{dp}")
    got = O.attention_module(p, i["x"], i["x"], i["x"], i["position"], meta["num_head"], meta["norm_eps"])
    assert got.shape == out.shape
    assert max_rel(got, out) < TOL


@pytest.mark.parametrize("dp", [0, 2])
def test_attention_pieces(dp):
    p, _, _, meta = load_golden(f"attention_dp{dp}")
    _, i, out, _ = load_golden(f"attention_pieces_dp{dp}")
    H, eps = meta["num_head"], meta["norm_eps"]
    Q = O.project_heads(i["x"], p["weight_Q"], p["bias_Q"], i["position"], H, 32)
    K = O.project_layernorm_heads(i["x"], p["weight_K"], p["bias_K"], p["ln_weight_K"], p["ln_bias_K"],
                                  i["position"], eps, H, 32)
    V = O.project_layernorm_heads(i["x"], p["weight_V"], p["bias_V"], p["ln_weight_V"], p["ln_bias_V"],
                                  i["position"], eps, H, 32)
    for got, want in ((Q, i["Q"]), (K, i["K"]), (V, i["V"])):
        assert got.shape == want.shape
        assert max_rel(got, want) < TOL
    assert max_rel(O.galerkin_attention(i["Q"], i["K"], i["V"]), out) < TOL


def test_encoder_layer():
    p, i, out, meta = load_golden("encoder_layer")
    got = O.encoder_layer(p, i["x"], i["position"], meta["num_head"], meta["norm_eps"], meta["activation"])
    assert max_rel(got, out) < TOL


def test_spectral_conv2d():
    p, i, out, meta = load_golden("spectral_conv2d")
    got = O.spectral_conv2d(p, i["x"], meta["mode"], meta["activation"])
    assert max_rel(got, out) < TOL
    # the accelerated module's weight layout and operator sequence give the same result
    psp = dict(p)
    for k in ("fourier_weight.0", "fourier_weight.1"):
        psp[k] = p[k].permute(2, 3, 0, 1, 4).contiguous()
    assert max_rel(O.spectral_conv2d(psp, i["x"], meta["mode"], meta["activation"], weight_layout="sp"), out) < TOL
    assert max_rel(O.op_spectral_conv2d_sp(psp, i["x"], meta["mode"], meta["activation"]), out) < 1e-5


def test_down_scaler():
    p, i, out, meta = load_golden("down_scaler")
    got = O.down_scaler(p, i["x"], meta["resolution_size"].tolist(), meta["activation"])
    assert got.shape == out.shape
    assert max_rel(got, out) < TOL


def test_up_scaler():
    p, i, out, meta = load_golden("up_scaler")
    got = O.up_scaler(p, i["x"], meta["resolution_size"].tolist(), meta["activation"])
    assert got.shape == out.shape
    assert max_rel(got, out) < TOL


def test_full_model():
    p, i, out, meta = load_golden("galerkin_transformer_2d")
    cfg = dict(meta)
    cfg["resolution_size"] = meta["resolution_size"].tolist()
    got = O.galerkin_transformer_2d(p, cfg, i["x"], i["position"], i["grid"])
    assert torch.isfinite(out).all()
    assert got.shape == out.shape
    assert (got[:, 0] == 0).all() and (got[:, :, -1] == 0).all()
    assert max_rel(got, out) < 1e-5
