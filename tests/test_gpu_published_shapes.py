"""Parity at the shapes of the reference's own published timings (evaluate/sp_all.py:8-19: sp_galerkin.py:20-72 and
:130-229, sp_fno2d.py:10-26, sp_darcy_breakdown.py:69-101, sp_darcy_ablation.py:23-70), so that every row of
bench.py's `reference_published_shapes` has a gate at its shape.  Inputs are torch.rand as in those scripts.
The spectral layer's 128 -> 32 shapes are in tests/test_gpu_modules.py
(test_spectral_conv_unequal_widths_take_the_fused_route)."""
import math

import pytest
import torch

from conftest import max_rel, rel_l2
from oracle import spgt_oracle as O
from spgt_amd.extension.bind import galerkin_attention as ga
from spgt_amd.network import model as M
from spgt_amd.network import sp_layer as L
from spgt_amd.network import sp_model as SM

pytestmark = pytest.mark.gpu
TOL = 1e-4


def urand(*shape, seed):
    return torch.rand(*shape, generator=torch.Generator().manual_seed(seed))


@pytest.mark.parametrize("S", [65536, 262144])
def test_skinny_gemm_at_the_published_shapes(gpu, S):
    """[16, 32, S] x [16, S, 32] (time_skinny_gemm_wrt_resolution, resolutions 256 and 512) against a float64
    product on the host; two runs give the same bits."""
    A, B = urand(16, 32, S, seed=1), urand(16, S, 32, seed=2)
    want = torch.matmul(A.double(), B.double())
    Ad, Bd = A.to(gpu), B.to(gpu)
    got = ga.batched_skinny_gemm(Ad, Bd)
    assert max_rel(got.cpu().double(), want) < 1e-5
    assert torch.equal(got, ga.batched_skinny_gemm(Ad, Bd))


def test_projection_operators_at_the_published_shape(gpu):
    """projection + position and projection + LayerNorm + position at B=16, S=65536, 4 heads of 32, dp=2,
    norm_eps 1e-5, uniform inputs and parameters (time_projpos_lnorm_wrt_resolution, resolution 256): two batch
    entries against the oracle in float64, all sixteen against float64 torch operations on the GPU."""
    Bn, S, H, dp = 16, 65536, 4, 2
    x, W, b = urand(Bn, S, 128, seed=3), urand(128, 128, seed=4), urand(128, seed=5)
    pos, lw, lb = urand(Bn, S, dp, seed=6), urand(H, 32, seed=7), urand(H, 32, seed=8)
    d = lambda t: t.to(gpu)
    got_p = ga.multihead_projection_with_position_rrc_cuda(d(x), d(W), d(b), d(pos), H, 32, dp)
    got_l = ga.multihead_projection_layernorm_with_position_rrc_cuda(d(x), d(W), d(b), d(lw), d(lb), d(pos), 1e-5, H, 32, dp)
    assert got_p.shape == got_l.shape == (Bn, H, dp + 32, S)
    for e in (0, Bn - 1):
        sl = slice(e, e + 1)
        want_p = O.op_projection_rrc(x[sl].double(), W.double(), b.double(), pos[sl].double(), H, 32)
        want_l, _ = O.op_projection_layernorm_rrc(x[sl].double(), W.double(), b.double(), lw.double(), lb.double(),
                                                  pos[sl].double(), 1e-5, H, 32)
        assert max_rel(got_p[sl].cpu().double(), want_p) < TOL
        assert max_rel(got_l[sl].cpu().double(), want_l) < TOL
    y = (d(x).double() @ d(W).double() + d(b).double()).view(Bn, S, H, 32)
    yl = torch.nn.functional.layer_norm(y, [32], None, None, 1e-5) * d(lw).double() + d(lb).double()
    posr = d(pos).double().unsqueeze(2).expand(Bn, S, H, dp)
    for got, feat in ((got_p, y), (got_l, yl)):
        want = torch.cat([posr, feat], -1).permute(0, 2, 3, 1)
        assert max_rel(got.double(), want) < TOL
        assert torch.equal(got[:, :, :dp], want[:, :, :dp].float())  # position rows are copies


def yaml_cfg(R, drops=0.0):
    """config/darcy_config.yaml as the reference's timing scripts set it up (sp_darcy_ablation.py:23-45):
    subsample_node 1, subsample_attn 2, modes ceil(sqrt(r))."""
    ra = int((R - 1) / 2 + 1)
    return dict(
        drop_module=0.0, boundary_condition="dirichlet", target_normalizer=SM.UnitNormalizer(),
        resolution_size=M.get_resolution_size(R, ra), dim_node=1, dim_hidden=128, drop_downscaler=drops,
        acti_downscaler="relu", num_encoder_layer=6, num_head=4, dim_position=2, attn_norm_eps=1e-6,
        drop_encoder_attn=0.0, drop_encoder_attn_fc=drops, attn_xavier=0.01, attn_diagonal=0.01, attn_symmetric=False,
        dim_encoder_ffn=256, drop_encoder_ffn=drops, acti_encoder_ffn="relu", drop_upscaler=0.0, acti_upscaler="silu",
        num_decoder_layer=2, dim_target=1, dim_spatial_hidden=32, num_frequence_mode=math.ceil(math.sqrt(R)),
        drop_decoder_layer=0.0, acti_decoder_layer="silu"), ra


def oracle_params(sd, dtype):
    return {k: (v.t() if k.rsplit(".", 1)[-1] in ("weight_Q", "weight_K", "weight_V") else v).to(dtype)
            for k, v in sd.items()}


def test_six_encoder_layers_at_the_published_shape(gpu):
    """Six yaml-default encoder layers on [4, 128 * 128, 128] with two position channels (gen_encoder_layers,
    resolution 256), drop rates 0: the inference path and the path under autograd against the oracle in float64."""
    cfg, ra = yaml_cfg(256)
    torch.manual_seed(0)
    layers = [L.Sp_EncoderLayer(128, 4, 2, 1e-6, 0.0, 0.0, 0.01, 0.01, False, 256, 0.0, "relu") for _ in range(6)]
    sds = [{k: v.clone() for k, v in layer.state_dict().items()} for layer in layers]
    x, pos = urand(4, ra * ra, 128, seed=9), urand(4, ra * ra, 2, seed=10)
    want = x.double()
    for sd in sds:
        want = O.encoder_layer(oracle_params(sd, torch.float64), want, pos.double(), 4, 1e-6, "relu")
    mods = [layer.to(gpu).eval() for layer in layers]
    with torch.no_grad():
        y = x.to(gpu)
        for m in mods:
            y = m(y, pos.to(gpu))
    assert max_rel(y.cpu().double(), want) < TOL
    yg = x.to(gpu).requires_grad_(True)
    out = yg
    for m in mods:
        out = m(out, pos.to(gpu))
    assert max_rel(out.detach().cpu().double(), want) < TOL


def test_yaml_default_model_at_resolution_256(gpu):
    """The whole yaml-default model as the reference's ablation script builds it at resolution 256 (r_attn 128,
    r_mid from get_resolution_size, 16 modes, spectral width 32), drop rates 0, two samples, against the oracle in
    float64: relative L2 <= 1e-4."""
    cfg, ra = yaml_cfg(256)
    assert cfg["resolution_size"][1] == (181, 181)
    torch.manual_seed(1)
    model = SM.Sp_GalerkinTransformer2D(cfg)
    sd = {k: v.clone() for k, v in model.state_dict().items()}
    node, pos, grid = urand(2, 256, 256, 1, seed=11), urand(2, ra, ra, 2, seed=12), urand(2, 256, 256, 2, seed=13)
    want = O.galerkin_transformer_2d(oracle_params(sd, torch.float64), cfg, node.double(), pos.double(), grid.double(),
                                     weight_layout="sp")
    model = model.to(gpu).eval()
    with torch.no_grad():
        got = model(node.to(gpu), pos.to(gpu), grid.to(gpu))
    assert got.shape == want.shape
    assert rel_l2(got.cpu().double(), want) < TOL
