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
@pytest.mark.parametrize("fused", [True, False])
@pytest.mark.parametrize("B,S", [(2, 150), (3, 2501)])
def test_attention_module_trains_like_the_oracle(gpu, dp, fused, B, S):
    """Sp_GalerkinAttention under autograd, on the fused token-major path (packed projection + fused core, each
    with its own backward) and on the reference's operator sequence with its three backwards, against autograd
    through the oracle's plain-PyTorch restatement, for the input and every parameter."""
    torch.manual_seed(5)
    H = 4
    m = L.Sp_GalerkinAttention(128, H, dp, 1e-6, 0.0, 0.0, 0.7, 0.01, False)
    m.fused_training = fused
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


@pytest.mark.parametrize("dp", [0, 2])
@pytest.mark.parametrize("B,H,S", [(1, 4, 1), (2, 4, 50), (1, 8, 777), (2, 4, 4099), (3, 4, 20011), (8, 4, 44521)])
def test_fused_attention_backward(gpu, dp, B, H, S):
    """galerkin_attention_fused under autograd (token-major forward + its two-pass backward) against autograd
    through the oracle's attention core in float64: gradients of the plain projections q, k, v and of the four
    LayerNorm parameters, one of them zero; ragged sequence lengths up to the benchmark shape."""
    q, k, v = rnd(B, S, H * 32, seed=21), rnd(B, S, H * 32, seed=22) * 1.3 + 0.2, rnd(B, S, H * 32, seed=23)
    pos = torch.rand(B, S, dp, generator=torch.Generator().manual_seed(24))
    aff = [1 + 0.3 * rnd(H, 32, seed=25), 0.2 * rnd(H, 32, seed=26), 1 + 0.3 * rnd(H, 32, seed=27), 0.2 * rnd(H, 32, seed=28)]
    aff[0][1, 5] = 0.0
    G = rnd(B, S, H * (dp + 32), seed=29)
    if S > 10000:  # the float64 oracle on one batch entry, the kernel on all of them
        sl = slice(B - 1, B)
    else:
        sl = slice(0, B)
    leaves = [t[sl].double().requires_grad_(True) for t in (q, k, v)] + [t.double().requires_grad_(True) for t in aff]
    O.attention_core_token_major(leaves[0], leaves[1], leaves[2], pos[sl].double(), *leaves[3:], 1e-6, H).backward(G[sl].double())
    dl = [t.to(gpu).requires_grad_(True) for t in (q, k, v)] + [t.to(gpu).requires_grad_(True) for t in aff]
    out = ga.galerkin_attention_fused(dl[0], dl[1], dl[2], pos.to(gpu) if dp else None, *dl[3:], 1e-6, H, dp)
    out.backward(G.to(gpu))
    for i, name in enumerate(("dq", "dk", "dv")):
        assert max_rel(dl[i].grad[sl].cpu().double(), leaves[i].grad) < TOL, name
    if sl == slice(0, B):
        for i, name in zip(range(3, 7), ("dgammaK", "dbetaK", "dgammaV", "dbetaV")):
            assert dl[i].grad.shape == (H, 32)
            assert max_rel(dl[i].grad.cpu().double(), leaves[i].grad) < TOL, name
    # a second run gives the same bits (fixed summation order)
    grads1 = [t.grad.clone() for t in dl]
    for t in dl:
        t.grad = None
    ga.galerkin_attention_fused(dl[0], dl[1], dl[2], pos.to(gpu) if dp else None, *dl[3:], 1e-6, H, dp).backward(G.to(gpu))
    assert all(torch.equal(a, t.grad) for a, t in zip(grads1, dl))


def test_fused_attention_backward_layernorm_parameters_at_full_size(gpu):
    """d gamma / d beta at B=8, S=44521 against float64 sums formed on the GPU from the same definitions
    (dy * x_hat and dy summed over all tokens), where the float64 CPU oracle would take minutes."""
    B, S, H, dp = 8, 44521, 4, 2
    q, k, v = rnd(B, S, H * 32, seed=31).to(gpu), (rnd(B, S, H * 32, seed=32) * 1.3 + 0.2).to(gpu), rnd(B, S, H * 32, seed=33).to(gpu)
    pos = torch.rand(B, S, dp, generator=torch.Generator().manual_seed(34)).to(gpu)
    aff = [(1 + 0.3 * rnd(H, 32, seed=35)).to(gpu), (0.2 * rnd(H, 32, seed=36)).to(gpu),
           (1 + 0.3 * rnd(H, 32, seed=37)).to(gpu), (0.2 * rnd(H, 32, seed=38)).to(gpu)]
    G = rnd(B, S, H * (dp + 32), seed=39).to(gpu)
    dl = [t.clone().requires_grad_(True) for t in (q, k, v)] + [t.clone().requires_grad_(True) for t in aff]
    ga.galerkin_attention_fused(dl[0], dl[1], dl[2], pos, *dl[3:], 1e-6, H, dp).backward(G)
    # the same function in float64 torch ops on the GPU, differentiated by autograd
    ref = [t.double().requires_grad_(True) for t in (q, k, v)] + [t.double().requires_grad_(True) for t in aff]

    def heads(x, gamma=None, beta=None):
        x = x.view(B, S, H, 32)
        if gamma is not None:
            x = torch.nn.functional.layer_norm(x, [32], None, None, 1e-6) * gamma + beta
        return torch.cat([pos.double().unsqueeze(2).expand(B, S, H, dp), x], -1).transpose(1, 2)  # [B, H, S, D]
    Qh, Kh, Vh = heads(ref[0]), heads(ref[1], ref[3], ref[4]), heads(ref[2], ref[5], ref[6])
    out = Qh @ (Kh.transpose(-2, -1) @ Vh / S)
    out.transpose(1, 2).reshape(B, S, H * (dp + 32)).backward(G.double())
    for i, name in enumerate(("dq", "dk", "dv", "dgammaK", "dbetaK", "dgammaV", "dbetaV")):
        assert max_rel(dl[i].grad.double(), ref[i].grad) < TOL, name


@pytest.mark.parametrize("dp,act", [(0, "silu"), (2, "relu")])
def test_encoder_layer_trains_like_the_oracle(gpu, dp, act):
    """A whole Sp_EncoderLayer under autograd (packed projection, fused attention core, output projection and
    feed-forward net, each with this package's backward) against autograd through the oracle in float64: the
    gradient of the input and of every parameter."""
    torch.manual_seed(7)
    B, S, H = 2, 1333, 4
    m = L.Sp_EncoderLayer(128, H, dp, 1e-6, 0.0, 0.0, 0.7, 0.01, False, 256, 0.0, act)
    with torch.no_grad():
        for prm in m.parameters():
            prm.add_(0.05 * torch.randn_like(prm))
    x = rnd(B, S, 128, seed=41)
    pos = torch.rand(B, S, dp, generator=torch.Generator().manual_seed(42))
    G = rnd(B, S, 128, seed=43)
    po = {k: v.detach().double().clone().requires_grad_(True) for k, v in m.state_dict().items()}
    xo = x.double().requires_grad_(True)
    transposed = {k: (v.t() if k.rsplit(".", 1)[-1] in ("weight_Q", "weight_K", "weight_V") else v) for k, v in po.items()}
    O.encoder_layer(transposed, xo, pos.double(), H, 1e-6, act).backward(G.double())
    m = m.to(gpu)
    xg = x.to(gpu).requires_grad_(True)
    out = m(xg, pos.to(gpu))
    out.backward(G.to(gpu))
    with torch.no_grad():
        assert max_rel(out.detach().cpu().double(), O.encoder_layer(transposed, xo, pos.double(), H, 1e-6, act).detach()) < TOL
    assert max_rel(xg.grad.cpu().double(), xo.grad) < TOL
    for name, prm in m.named_parameters():
        assert prm.grad is not None, name
        assert max_rel(prm.grad.cpu().double(), po[name].grad) < TOL, name


@pytest.mark.parametrize("N,r,cin,cout,m,act", [(2, 33, 64, 64, 5, "silu"), (2, 40, 128, 32, 6, "silu"),
                                                (1, 64, 32, 32, 8, "relu"), (2, 21, 128, 64, 4, "silu"),
                                                (1, 141, 64, 32, 12, "silu")])
def test_spectral_conv_trains_like_the_oracle(gpu, N, r, cin, cout, m, act):
    """Sp_SpectralConv2D under autograd on the truncated-DFT route (forward and adjoint stages on the same kernels)
    against autograd through the oracle's rfft2 / irfft2 restatement in float64: the gradient of the input, of
    both Fourier weights and of the residual Linear."""
    from spgt_amd.network import truncated_dft
    torch.manual_seed(23)
    layer = L.Sp_SpectralConv2D(cin, cout, m, 0.0, act)
    with torch.no_grad():
        for w in layer.fourier_weight:
            w.copy_(torch.randn(w.shape) / cin)
    x = rnd(N, r, r, cin, seed=51)
    G = rnd(N, r, r, cout, seed=52)
    po = {k: v.detach().double().clone().requires_grad_(True) for k, v in layer.state_dict().items()}
    xo = x.double().requires_grad_(True)
    want = O.spectral_conv2d(po, xo, m, act, weight_layout="sp")
    want.backward(G.double())
    assert truncated_dft.spectral_linear_trainable(r, cin, cout, m)
    layer = layer.to(gpu)
    xg = x.to(gpu).requires_grad_(True)
    got = layer(xg)
    got.backward(G.to(gpu))
    assert max_rel(got.detach().cpu().double(), want.detach()) < TOL
    assert max_rel(xg.grad.cpu().double(), xo.grad) < TOL
    for name, prm in layer.named_parameters():
        assert prm.grad is not None, name
        assert max_rel(prm.grad.cpu().double(), po[name].grad) < TOL, name


@pytest.mark.parametrize("N,r,dim_x,hidden,m", [(2, 33, 128, 32, 5), (1, 40, 64, 64, 6)])
def test_decoder_regressor_trains_like_the_oracle(gpu, N, r, dim_x, hidden, m):
    """Sp_DecoderRegressor under autograd (input layer on hidden features and grid columns without a concatenation,
    spectral layers on the truncated-DFT route, regression head with one output feature) against autograd through
    the oracle in float64: output, gradient of the hidden features and of every parameter."""
    from spgt_amd.network import sp_model as M
    torch.manual_seed(29)
    dec = M.Sp_DecoderRegressor(2, dim_x, 1, 2, hidden, m, 0.0, "silu")
    with torch.no_grad():
        for layer in dec.layers:
            for w in layer.fourier_weight:
                w.copy_(torch.randn(w.shape) / hidden)
    x = rnd(N, r, r, dim_x, seed=61)
    grid = rnd(N, r, r, 2, seed=62)
    G = rnd(N, r, r, 1, seed=63)
    po = {k: v.detach().double().clone().requires_grad_(True) for k, v in dec.state_dict().items()}
    xo = x.double().requires_grad_(True)
    want = O.decoder_regressor(po, xo, grid.double(), 2, m, "silu", weight_layout="sp")
    want.backward(G.double())
    dec = dec.to(gpu)
    xg = x.to(gpu).requires_grad_(True)
    got = dec(xg, grid.to(gpu))
    got.backward(G.to(gpu))
    assert max_rel(got.detach().cpu().double(), want.detach()) < TOL
    assert max_rel(xg.grad.cpu().double(), xo.grad) < TOL
    for name, prm in dec.named_parameters():
        assert prm.grad is not None, name
        assert max_rel(prm.grad.cpu().double(), po[name].grad) < TOL, name


@pytest.mark.parametrize("r,r_attn,dim", [(41, 21, 32), (64, 32, 48), (41, 21, 128)])
def test_scalers_train_like_the_oracle(gpu, r, r_attn, dim):
    """DownScaler2D and UpScaler2D under autograd (resamplings forward and backward on this package's kernels, in
    the planes and the channels-last layouts; at 128 channels the up-scaler's interpolate -> conv3x3 as a Linear on the
    low-resolution tokens plus the nine-tap gather and its adjoint) against autograd through the oracle in float64."""
    from spgt_amd.network import model as M
    torch.manual_seed(37)
    sizes = M.get_resolution_size(r, r_attn)
    for kind in ("down", "up"):
        if kind == "down":
            mod = M.DownScaler2D(sizes, 1, dim, 0.0, "relu")
            x = rnd(2, r, r, 1, seed=81)
            fn = O.down_scaler
            G = rnd(2, r_attn, r_attn, dim, seed=82)
        else:
            mod = M.UpScaler2D(sizes, dim, dim, 0.0, "silu")
            x = rnd(2, r_attn, r_attn, dim, seed=83)
            fn = O.up_scaler
            G = rnd(2, r, r, dim, seed=84)
        po = {k: v.detach().double().clone().requires_grad_(True) for k, v in mod.state_dict().items()}
        xo = x.double().requires_grad_(True)
        want = fn(po, xo, sizes, "relu" if kind == "down" else "silu")
        want.backward(G.double())
        mod = mod.to(gpu)
        xg = x.to(gpu).requires_grad_(True)
        got = mod(xg)
        got.backward(G.to(gpu))
        assert max_rel(got.detach().cpu().double(), want.detach()) < TOL, kind
        assert max_rel(xg.grad.cpu().double(), xo.grad) < TOL, kind
        for name, prm in mod.named_parameters():
            assert max_rel(prm.grad.cpu().double(), po[name].grad) < TOL, (kind, name)


@pytest.mark.parametrize("in_f,hid,out_f", [(32, 128, 1), (128, 256, 128), (36, 40, 3)])
def test_feed_forward_trains_like_the_oracle(gpu, in_f, hid, out_f):
    """FeedForward under autograd, including a head with one output feature (weight gradient with the roles of
    input and gradient swapped) and widths no kernel here serves (torch throughout)."""
    from spgt_amd.network.layer import FeedForward
    torch.manual_seed(31)
    ffn = FeedForward(in_f, out_f, hid, 0.0, "silu")
    x = rnd(3, 1201, in_f, seed=71)
    G = rnd(3, 1201, out_f, seed=72)
    po = {k: v.detach().double().clone().requires_grad_(True) for k, v in ffn.state_dict().items()}
    xo = x.double().requires_grad_(True)
    want = O.feed_forward(po, xo, "silu")
    want.backward(G.double())
    ffn = ffn.to(gpu)
    xg = x.to(gpu).requires_grad_(True)
    got = ffn(xg)
    got.backward(G.to(gpu))
    assert max_rel(got.detach().cpu().double(), want.detach()) < TOL
    assert max_rel(xg.grad.cpu().double(), xo.grad) < TOL
    for name, prm in ffn.named_parameters():
        assert max_rel(prm.grad.cpu().double(), po[name].grad) < TOL, name


def test_packed_projection_function_with_separate_gradient_tensors(gpu):
    """The packed Q | K | V projection's backward when its three gradients are separate allocations (the attention
    backward hands it three planes of one buffer, which takes the no-copy branch): against torch's own autograd."""
    from spgt_amd.network.sp_layer import _PackedProjectionFunction
    torch.manual_seed(3)
    N, S, C = 2, 777, 128
    x = torch.randn(N, S, C, device=gpu, requires_grad=True)
    ws = [(torch.randn(C, C, device=gpu) / C ** 0.5).requires_grad_(True) for _ in range(3)]
    bs = [torch.randn(C, device=gpu).requires_grad_(True) for _ in range(3)]
    packed_w = torch.cat([w.detach() for w in ws], dim=1).contiguous()
    packed_b = torch.cat([b.detach() for b in bs]).contiguous()
    outs = _PackedProjectionFunction.apply(x, *ws, *bs, packed_w, packed_b)
    assert len(outs) == 4 and torch.equal(outs[3], x)  # the input handed on for a residual add further on
    gs = [torch.randn(N, S, C, device=gpu) for _ in range(4)]
    got = torch.autograd.grad(outs, [x, *ws, *bs], gs)
    x2 = x.detach().double().requires_grad_(True)
    ws2 = [w.detach().double().requires_grad_(True) for w in ws]
    bs2 = [b.detach().double().requires_grad_(True) for b in bs]
    ref_outs = [x2 @ w + b for w, b in zip(ws2, bs2)] + [x2 * 1.0]
    want = torch.autograd.grad(ref_outs, [x2, *ws2, *bs2], [g.double() for g in gs])
    for o, r in zip(outs, ref_outs):
        assert max_rel(o.detach().double().cpu(), r.detach().cpu()) < TOL
    for g, w in zip(got, want):
        assert max_rel(g.double().cpu(), w.cpu()) < TOL
