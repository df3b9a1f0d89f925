"""Backward of the attention operators against autograd through the CPU oracle in fp64."""
import pytest
import torch

from conftest import max_rel
from oracle import spgt_oracle as O
from spgt_amd.extension.bind import galerkin_attention as ga
from spgt_amd.network import sp_layer as L

pytestmark = pytest.mark.gpu
TOL = 1e-4


def rnd(*shape, seed=0):
    return torch.randn(*shape, generator=torch.Generator().manual_seed(seed), dtype=torch.float32)


@pytest.mark.parametrize("d", [32, 34])
@pytest.mark.parametrize("B,H,S", [(1, 1, 1), (2, 4, 50), (1, 3, 777), (2, 2, 4099),
                                   # chunks of several 128-token blocks per wave, ragged tails: (8, 4, 20011) gives a
                                   # wave two blocks, the benchmark shape four
                                   (8, 4, 20011), (8, 4, 44521)])
def test_attention_backward(gpu, d, B, H, S):
    Q, K, V, G = rnd(B, H, d, S, seed=1), rnd(B, H, d, S, seed=2), rnd(B, H, d, S, seed=3), rnd(B, H, S, d, seed=4)
    q, k, v = (t.double().requires_grad_(True) for t in (Q, K, V))
    O.op_attention_cccr(q, k, v).backward(G.double())
    qg, kg, vg = (t.to(gpu).requires_grad_(True) for t in (Q, K, V))
    ga.multihead_galerkin_attention_cccr_cuda(qg, kg, vg).backward(G.to(gpu))
    for got, want, name in ((qg.grad, q.grad, "dQ"), (kg.grad, k.grad, "dK"), (vg.grad, v.grad, "dV")):
        assert got.shape == want.shape
        assert max_rel(got.cpu().double(), want) < TOL, name


@pytest.mark.parametrize("dp", [0, 2])
@pytest.mark.parametrize("B,S", [(1, 1), (2, 50), (1, 777), (2, 1031)])
def test_projection_backward(gpu, dp, B, S):
    Dm, H = 128, 4
    X, W, b = rnd(B, S, Dm, seed=5), rnd(Dm, Dm, seed=6) / Dm ** 0.5, rnd(Dm, seed=7)
    pos = torch.rand(B, S, dp, generator=torch.Generator().manual_seed(8))
    G = rnd(B, H, dp + 32, S, seed=9)
    x, w, bb = (t.double().requires_grad_(True) for t in (X, W, b))
    O.op_projection_rrc(x, w, bb, pos.double(), H, 32).backward(G.double())
    xg, wg, bg = (t.to(gpu).requires_grad_(True) for t in (X, W, b))
    ga.multihead_projection_with_position_rrc_cuda(xg, wg, bg, pos.to(gpu), H, 32, dp).backward(G.to(gpu))
    for got, want, name in ((xg.grad, x.grad, "dX"), (wg.grad, w.grad, "dW"), (bg.grad, bb.grad, "db")):
        assert max_rel(got.cpu().double(), want) < TOL, name


@pytest.mark.parametrize("dp", [0, 2])
@pytest.mark.parametrize("B,S", [(1, 1), (2, 50), (1, 777), (2, 1031)])
def test_projection_layernorm_backward(gpu, dp, B, S):
    Dm, H = 128, 4
    X, W, b = rnd(B, S, Dm, seed=10), rnd(Dm, Dm, seed=11) / Dm ** 0.5, rnd(Dm, seed=12)
    g, be = 1 + 0.3 * rnd(H, 32, seed=13), 0.2 * rnd(H, 32, seed=14)
    g[1, 5] = 0.0  # a zero LayerNorm weight must not poison the gradients
    pos = torch.rand(B, S, dp, generator=torch.Generator().manual_seed(15))
    G = rnd(B, H, dp + 32, S, seed=16)
    leaves = [t.double().requires_grad_(True) for t in (X, W, b, g, be)]
    y, _ = O.op_projection_layernorm_rrc(*leaves, pos.double(), 1e-6, H, 32)
    y.backward(G.double())
    gl = [t.to(gpu).requires_grad_(True) for t in (X, W, b, g, be)]
    ga.multihead_projection_layernorm_with_position_rrc_cuda(*gl, pos.to(gpu), 1e-6, H, 32, dp).backward(G.to(gpu))
    for got, want, name in zip(gl, leaves, ("dX", "dW", "db", "dgamma", "dbeta")):
        assert torch.isfinite(got.grad).all(), name
        assert max_rel(got.grad.cpu().double(), want.grad) < TOL, name


@pytest.mark.parametrize("dp", [0, 2])
def test_projection_layernorm_backward_with_the_reference_arguments(gpu, dp):
    """The pybind-level backward as the reference declares it (extension/bind/galerkin_attention.cu:70-102):
    (grad_ln, input, weight, hat_ln, invsigma, lnw, lnb, ints...) -> (dX, dW, db, dgamma, dbeta), with hat_ln and
    invsigma as the forward operator returned them; against autograd through the oracle in float64."""
    B, S, Dm, H = 2, 333, 128, 4
    X, W, b = rnd(B, S, Dm, seed=30), rnd(Dm, Dm, seed=31) / Dm ** 0.5, rnd(Dm, seed=32)
    g, be = 1 + 0.3 * rnd(H, 32, seed=33), 0.2 * rnd(H, 32, seed=34)
    pos = torch.rand(B, S, dp, generator=torch.Generator().manual_seed(35))
    G = rnd(B, H, dp + 32, S, seed=36)
    leaves = [t.double().requires_grad_(True) for t in (X, W, b, g, be)]
    y, _ = O.op_projection_layernorm_rrc(*leaves, pos.double(), 1e-6, H, 32)
    y.backward(G.double())
    d = lambda t: t.to(gpu)
    hat_ln, invsigma = ga.gexts.multihead_projection_layernorm_with_position_rrc_forward(
        d(X), d(W), d(b), d(g), d(be), 1e-6, d(pos), S, Dm, H, 32, dp, B)
    grads = ga.gexts.multihead_projection_layernorm_with_position_rrc_backward(
        d(G), d(X), d(W), hat_ln, invsigma, d(g), d(be), S, Dm, H, 32, dp, B)
    assert len(grads) == 5
    for got, want, name in zip(grads, leaves, ("dX", "dW", "db", "dgamma", "dbeta")):
        assert got.shape == want.shape, name
        assert max_rel(got.cpu().double(), want.grad) < TOL, name


def test_heads_feature_to_token_major(gpu):
    B, H, dp, S = 2, 4, 2, 333
    src = rnd(B, H, dp + 32, S, seed=17)
    got = ga.gexts.heads_feature_to_token_major(src.to(gpu), B, H, dp, 32, S)
    want = src[:, :, dp:, :].permute(0, 3, 1, 2).reshape(B, S, H * 32)
    assert torch.equal(got.cpu(), want)


@pytest.mark.parametrize("dp", [0, 2])
def test_attention_module_trains_like_the_oracle(gpu, dp):
    """Sp_GalerkinAttention under autograd (operator sequence + the three backwards) against autograd
    through the oracle's plain-PyTorch restatement, for the input and every parameter."""
    torch.manual_seed(5)
    B, S, H = 2, 150, 4
    m = L.Sp_GalerkinAttention(128, H, dp, 1e-6, 0.0, 0.0, 0.7, 0.01, False)
    with torch.no_grad():
        for prm in m.parameters():
            prm.add_(0.1 * torch.randn_like(prm))
    x = rnd(B, S, 128, seed=18)
    pos = torch.rand(B, S, dp, generator=torch.Generator().manual_seed(19))
    G = rnd(B, S, 128, seed=20)
    po = {k: v.detach().double().clone().requires_grad_(True) for k, v in m.state_dict().items()}
    xo = x.double().requires_grad_(True)
    transposed = {k: (v.t() if k in ("weight_Q", "weight_K", "weight_V") else v) for k, v in po.items()}
    O.attention_module(transposed, xo, xo, xo, pos.double(), H, 1e-6).backward(G.double())
    m = m.to(gpu)
    xg = x.to(gpu).requires_grad_(True)
    m(xg, xg, xg, pos.to(gpu)).backward(G.to(gpu))
    assert max_rel(xg.grad.cpu().double(), xo.grad) < TOL
    for name, prm in m.named_parameters():
        assert max_rel(prm.grad.cpu().double(), po[name].grad) < TOL, name
