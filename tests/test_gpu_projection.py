"""Parity of the multi-head projection operators (x @ W + b, optional LayerNorm, position rows,
feature-major output) with the CPU oracle."""
import pytest
import torch

from conftest import load_golden, max_rel
from oracle import spgt_oracle as O
from spgt_amd import _lib
from spgt_amd.extension.bind import galerkin_attention as ga

pytestmark = pytest.mark.gpu
TOL = 1e-4


def rnd(*shape, seed=0):
    return torch.randn(*shape, generator=torch.Generator().manual_seed(seed), dtype=torch.float32)


@pytest.mark.parametrize("dp", [0, 2])
@pytest.mark.parametrize("B,S,Dm", [(1, 1, 128), (2, 50, 128), (1, 777, 128), (3, 4099, 128), (2, 130, 256),
                                    (2, 97, 384), (1, 333, 512),
                                    # long inputs: ragged last tiles, many short sequences, one long sequence
                                    (3, 30011, 128), (1024, 65, 128), (1100, 64, 128), (1, 65537, 128)])
def test_projection_vs_oracle(gpu, dp, B, S, Dm):
    H = Dm // 32
    x, W, b = rnd(B, S, Dm, seed=1), rnd(Dm, Dm, seed=2) / Dm ** 0.5, rnd(Dm, seed=3)
    pos = torch.rand(B, S, dp, generator=torch.Generator().manual_seed(4))
    want = O.op_projection_rrc(x.double(), W.double(), b.double(), pos.double(), H, 32)
    got = ga.multihead_projection_with_position_rrc_cuda(x.to(gpu), W.to(gpu), b.to(gpu), pos.to(gpu), H, 32, dp)
    assert got.shape == (B, H, dp + 32, S)
    assert max_rel(got.cpu().double(), want) < TOL
    if dp:
        for h in range(H):
            assert torch.equal(got[:, h, :dp].cpu(), pos.transpose(1, 2))  # position rows copied bit-exactly


@pytest.mark.parametrize("dp", [0, 2])
@pytest.mark.parametrize("B,S,Dm", [(1, 1, 128), (2, 50, 128), (1, 777, 128), (3, 4099, 128), (2, 130, 256),
                                    (2, 97, 384), (1, 333, 512),
                                    # long inputs: ragged last tiles, many short sequences, one long sequence
                                    (3, 30011, 128), (1024, 65, 128), (1100, 64, 128), (1, 65537, 128)])
def test_projection_layernorm_vs_oracle(gpu, dp, B, S, Dm):
    H = Dm // 32
    x, W, b = rnd(B, S, Dm, seed=5), rnd(Dm, Dm, seed=6) / Dm ** 0.5, rnd(Dm, seed=7)
    g, be = 1 + 0.3 * rnd(H, 32, seed=8), 0.2 * rnd(H, 32, seed=9)
    pos = torch.rand(B, S, dp, generator=torch.Generator().manual_seed(10))
    eps = 1e-6
    want, want_inv = O.op_projection_layernorm_rrc(x.double(), W.double(), b.double(), g.double(), be.double(),
                                                   pos.double(), eps, H, 32)
    d = lambda t: t.to(gpu)
    got, inv = ga.gexts.multihead_projection_layernorm_with_position_rrc_forward(
        d(x), d(W), d(b), d(g), d(be), eps, d(pos), S, Dm, H, 32, dp, B)
    assert got.shape == (B, H, dp + 32, S) and inv.shape == (B, H, S)
    assert max_rel(got.cpu().double(), want) < TOL
    assert max_rel(inv.cpu().double(), want_inv) < TOL
    via_python_surface = ga.multihead_projection_layernorm_with_position_rrc_cuda(d(x), d(W), d(b), d(g), d(be),
                                                                                  d(pos), eps, H, 32, dp)
    assert torch.equal(via_python_surface, got)


def test_projection_identity_weight_is_exact(gpu):
    B, S, Dm, H = 2, 333, 128, 4
    x = rnd(B, S, Dm, seed=11)
    got = ga.multihead_projection_with_position_rrc_cuda(
        x.to(gpu), torch.eye(Dm, device=gpu), torch.zeros(Dm, device=gpu), torch.zeros(B, S, 0, device=gpu), H, 32, 0)
    assert torch.equal(got.cpu(), x.view(B, S, H, 32).permute(0, 2, 3, 1))


def test_projection_identity_weight_is_exact_on_long_inputs(gpu):
    B, S, Dm, H = 5, 20001, 128, 4
    x = rnd(B, S, Dm, seed=14)
    pos = torch.rand(B, S, 2, generator=torch.Generator().manual_seed(15))
    got = ga.multihead_projection_with_position_rrc_cuda(
        x.to(gpu), torch.eye(Dm, device=gpu), torch.zeros(Dm, device=gpu), pos.to(gpu), H, 32, 2)
    assert torch.equal(got[:, :, 2:].cpu(), x.view(B, S, H, 32).permute(0, 2, 3, 1))
    assert torch.equal(got[:, :, :2].cpu(), pos.transpose(1, 2)[:, None].expand(B, H, 2, S))


def test_layernorm_constant_rows_give_bias(gpu):
    B, S, Dm, H = 1, 70, 128, 4
    x = torch.full((B, S, Dm), 3.0, device=gpu)
    g, be = (1 + 0.3 * rnd(H, 32, seed=12)).to(gpu), (0.2 * rnd(H, 32, seed=13)).to(gpu)
    got = ga.multihead_projection_layernorm_with_position_rrc_cuda(
        x, torch.eye(Dm, device=gpu), torch.zeros(Dm, device=gpu), g, be, torch.zeros(B, S, 0, device=gpu), 1e-6, H,
        32, 0)
    assert torch.allclose(got, be[None, :, :, None].expand(B, H, 32, S), atol=1e-6, rtol=0)


@pytest.mark.parametrize("dp", [0, 2])
def test_operator_chain_golden(gpu, dp):
    """The reference module's own Q, K, V and attention output, reproduced by the three drop-in operators.
    The reference's plain model multiplies by W^T, the operators by W, hence the transposed weights."""
    p, i, _, meta = load_golden(f"attention_dp{dp}")
    _, pieces, want, _ = load_golden(f"attention_pieces_dp{dp}")
    H, eps = int(meta["num_head"]), float(meta["norm_eps"])
    d = lambda t: t.to(gpu).contiguous()
    x, pos = d(i["x"]), d(i["position"])
    Q = ga.multihead_projection_with_position_rrc_cuda(x, d(p["weight_Q"].t()), d(p["bias_Q"]), pos, H, 32, dp)
    K = ga.multihead_projection_layernorm_with_position_rrc_cuda(
        x, d(p["weight_K"].t()), d(p["bias_K"]), d(p["ln_weight_K"]), d(p["ln_bias_K"]), pos, eps, H, 32, dp)
    V = ga.multihead_projection_layernorm_with_position_rrc_cuda(
        x, d(p["weight_V"].t()), d(p["bias_V"]), d(p["ln_weight_V"]), d(p["ln_bias_V"]), pos, eps, H, 32, dp)
    for got, name in ((Q, "Q"), (K, "K"), (V, "V")):
        assert max_rel(got.cpu(), pieces[name].transpose(-2, -1)) < TOL, name
    A = ga.multihead_galerkin_attention_cccr_cuda(Q, K, V)
    assert max_rel(A.cpu(), want) < TOL


def test_projection_argument_validation(gpu):
    x = torch.zeros(1, 8, 64, device=gpu)
    with pytest.raises(_lib.SpgtError):  # dim_hidden 64 is not supported
        ga.multihead_projection_with_position_rrc_cuda(x, torch.zeros(64, 64, device=gpu), torch.zeros(64, device=gpu),
                                                       torch.zeros(1, 8, 0, device=gpu), 2, 32, 0)
    x = torch.zeros(1, 8, 128, device=gpu)
    with pytest.raises(_lib.SpgtError):  # dim_position 1
        ga.multihead_projection_with_position_rrc_cuda(x, torch.zeros(128, 128, device=gpu),
                                                       torch.zeros(128, device=gpu), torch.zeros(1, 8, 1, device=gpu),
                                                       4, 32, 1)
