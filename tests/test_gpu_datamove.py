"""Bit-exact parity of the data-movement kernels, and tolerance parity of the
spectral contraction and bilinear resampling, against the CPU oracle."""
import pytest
import torch
import torch.nn.functional as F

from conftest import load_golden, max_rel
from oracle import spgt_oracle as O
from spgt_amd import _lib
from spgt_amd.extension.bind import datamove as dm

pytestmark = pytest.mark.gpu


def rnd(*shape, seed=0):
    return torch.randn(*shape, generator=torch.Generator().manual_seed(seed), dtype=torch.float32)


def bits_equal(a, b):
    ia = torch.view_as_real(a).contiguous().view(torch.int32) if a.is_complex() else a.contiguous().view(torch.int32)
    ib = torch.view_as_real(b).contiguous().view(torch.int32) if b.is_complex() else b.contiguous().view(torch.int32)
    return a.shape == b.shape and torch.equal(ia, ib)


def special_values(x):
    """Sprinkles NaN payloads, infinities, -0.0 and denormals into a float tensor."""
    flat = x.view(-1).view(torch.int32)
    # quiet NaN with payload, signalling-range NaN, -inf, -0.0, smallest denormal, +inf
    pats = torch.tensor([0x7FC00001, 0x7FA00000, -0x800000, -0x80000000, 0x00000001, 0x7F800000],
                        dtype=torch.int64).to(torch.int32)
    idx = torch.arange(0, flat.numel(), max(1, flat.numel() // 97))
    flat[idx] = pats[torch.arange(idx.numel()) % pats.numel()]
    return x


@pytest.mark.parametrize("batch,M,N", [([1], [1], [1]), ([2], [3, 5], [7]), ([3], [64], [64]), ([2], [65], [63]),
                                       ([2, 2], [9, 9], [6]), ([1], [141, 141], [64]), ([4], [64], [71, 71]),
                                       ([1], [1], [1000]), ([1], [1000], [1])])
def test_batched_transpose_bit_exact(gpu, batch, M, N):
    x = special_values(rnd(*batch, *M, *N, seed=1))
    want = O.op_batched_transpose(x, batch, M, N)
    got = dm.batched_transpose(x.to(gpu), batch, M, N)
    assert bits_equal(got.cpu(), want)
    back = dm.batched_transpose(got, batch, N, M)
    assert bits_equal(back.cpu(), x)


GATHER_CASES = [
    # dim_list, H_all, W_all, H_low, W_low, hb1, wb1, hb2, wb2
    ([1], 1, 1, 1, 1, 0, 0, 0, 0),
    ([2, 3], 6, 4, 2, 3, 0, 0, 4, 1),
    ([2, 6], 9, 5, 3, 3, 0, 0, 6, 0),
    ([8, 64], 141, 71, 12, 12, 0, 0, 129, 0),
    ([3, 65], 20, 11, 5, 7, 2, 1, 15, 4),
    ([4, 32], 8, 5, 5, 5, 0, 0, 3, 0),  # overlapping windows
    ([2, 70], 12, 160, 3, 100, 0, 2, 9, 60),   # wide windows: more than 64 KiB of LDS
    ([1, 5], 7, 157, 2, 157, 0, 0, 5, 0),      # the widest window
]


@pytest.mark.parametrize("case", GATHER_CASES)
def test_gather_scatter_bit_exact(gpu, case):
    dim_list, H_all, W_all, H_low, W_low, hb1, wb1, hb2, wb2 = case
    src = torch.view_as_complex(special_values(rnd(*dim_list, H_all, W_all, 2, seed=2)))
    w1, w2 = O.op_transpose_gather_dual(src, dim_list, H_all, W_all, H_low, W_low, hb1, wb1, hb2, wb2)
    g1, g2 = dm.transpose_gather_dual(src.to(gpu), dim_list, H_all, W_all, H_low, W_low, hb1, wb1, hb2, wb2)
    assert bits_equal(g1.cpu(), w1) and bits_equal(g2.cpu(), w2)
    a = torch.view_as_complex(special_values(rnd(H_low, W_low, *dim_list, 2, seed=3)))
    b = torch.view_as_complex(special_values(rnd(H_low, W_low, *dim_list, 2, seed=4)))
    want = O.op_transpose_scatter_dual(a, b, dim_list, H_all, W_all, H_low, W_low, hb1, wb1, hb2, wb2)
    got = dm.transpose_scatter_dual(a.to(gpu), b.to(gpu), dim_list, H_all, W_all, H_low, W_low, hb1, wb1, hb2, wb2)
    assert bits_equal(got.cpu(), want)


def test_scatter_of_gather_is_masked_identity(gpu):
    N, C, r, m = 8, 64, 141, 12
    src = torch.view_as_complex(rnd(N, C, r, r // 2 + 1, 2, seed=5)).to(gpu)
    g1, g2 = dm.transpose_gather_dual(src, [N, C], r, r // 2 + 1, m, m, 0, 0, r - m, 0)
    back = dm.transpose_scatter_dual(g1, g2, [N, C], r, r // 2 + 1, m, m, 0, 0, r - m, 0)
    mask = torch.zeros(r, r // 2 + 1, dtype=torch.bool, device=gpu)
    mask[:m, :m] = True
    mask[r - m:, :m] = True
    assert torch.equal(torch.view_as_real(back[..., mask]), torch.view_as_real(src[..., mask]))
    assert (torch.view_as_real(back[..., ~mask]) == 0).all()


def test_datamove_autograd(gpu):
    x = rnd(2, 6, 5, seed=6).to(gpu).requires_grad_(True)
    y = dm.batched_transpose(x, [2], [6], [5])
    gy = rnd(2, 5, 6, seed=7).to(gpu)
    y.backward(gy)
    assert torch.equal(x.grad, gy.transpose(1, 2))
    src = torch.view_as_complex(rnd(3, 6, 4, 2, seed=8)).to(gpu).requires_grad_(True)
    a, b = dm.transpose_gather_dual(src, [3], 6, 4, 2, 3, 0, 0, 4, 1)
    ga, gb = torch.view_as_complex(rnd(2, 3, 3, 2, seed=9)).to(gpu), torch.view_as_complex(rnd(2, 3, 3, 2, seed=10)).to(gpu)
    torch.autograd.backward([a, b], [ga, gb])
    want = O.op_transpose_scatter_dual(ga.cpu(), gb.cpu(), [3], 6, 4, 2, 3, 0, 0, 4, 1)
    assert bits_equal(src.grad.cpu(), want)


@pytest.mark.parametrize("N,Cin,Cout,r,m", [(1, 1, 1, 4, 1), (2, 6, 4, 9, 3), (8, 64, 64, 141, 12), (3, 32, 32, 33, 6),
                                             (17, 20, 70, 16, 4), (2, 8, 8, 8, 5)])
def test_spectral_mode_contract_vs_oracle(gpu, N, Cin, Cout, r, m):
    W_all = r // 2 + 1
    xf = torch.view_as_complex(rnd(N, Cin, r, W_all, 2, seed=11))
    w1, w2 = rnd(m, m, Cin, Cout, 2, seed=12) / Cin, rnd(m, m, Cin, Cout, 2, seed=13) / Cin
    # oracle: the reference's gather -> complex matmul -> scatter sequence, in complex128
    g1, g2 = O.op_transpose_gather_dual(xf.to(torch.complex128), [N, Cin], r, W_all, m, m, 0, 0, r - m, 0)
    c = lambda w: torch.view_as_complex(w.double().contiguous())
    want = O.op_transpose_scatter_dual(g1 @ c(w1), g2 @ c(w2), [N, Cout], r, W_all, m, m, 0, 0, r - m, 0)
    got = dm.spectral_mode_contract(xf.to(gpu), w1.to(gpu), w2.to(gpu), m, m, 0, 0, r - m, 0)
    assert got.shape == (N, Cout, r, W_all)
    inside = want != 0
    assert (torch.view_as_real(got.cpu())[~inside] == 0).all()
    assert max_rel(torch.view_as_real(got.cpu()).double(), torch.view_as_real(want)) < 1e-5
    # and the three-operator sequence on the GPU gives the same numbers
    a, b = dm.transpose_gather_dual(xf.to(gpu), [N, Cin], r, W_all, m, m, 0, 0, r - m, 0)
    seq = dm.transpose_scatter_dual(a @ torch.view_as_complex(w1.to(gpu)), b @ torch.view_as_complex(w2.to(gpu)),
                                    [N, Cout], r, W_all, m, m, 0, 0, r - m, 0)
    assert max_rel(torch.view_as_real(seq.cpu()).double(), torch.view_as_real(want)) < 1e-5


@pytest.mark.parametrize("N,Cin,Cout,H,W,mh,mw,hb1,wb1,hb2,wb2", [
    (2, 5, 3, 9, 6, 3, 3, 1, 2, 4, 1),       # windows anywhere, disjoint rows
    (3, 4, 70, 10, 7, 4, 3, 2, 1, 4, 3),     # rows overlap, columns overlap partly: the second window wins
    (1, 3, 2, 6, 5, 3, 2, 0, 0, 0, 0),       # identical windows
    (2, 8, 8, 12, 40, 2, 33, 9, 5, 1, 0),    # wide windows (more than 32 columns), second window first in memory
    (1, 2, 2, 5, 4, 5, 4, 0, 0, 0, 0),       # windows cover everything: nothing to zero
])
def test_spectral_mode_contract_general_windows(gpu, N, Cin, Cout, H, W, mh, mw, hb1, wb1, hb2, wb2):
    """Windows at arbitrary bases, overlapping and not, against the reference's gather -> matmul -> scatter
    sequence (extension/bind/datamove.cu:25-64) in complex128; every element outside the windows must be zero
    even though the output buffer starts out as NaN."""
    xf = torch.view_as_complex(rnd(N, Cin, H, W, 2, seed=31))
    w1, w2 = rnd(mh, mw, Cin, Cout, 2, seed=32), rnd(mh, mw, Cin, Cout, 2, seed=33)
    g1, g2 = O.op_transpose_gather_dual(xf.to(torch.complex128), [N, Cin], H, W, mh, mw, hb1, wb1, hb2, wb2)
    c = lambda w: torch.view_as_complex(w.double().contiguous())
    want = O.op_transpose_scatter_dual(g1 @ c(w1), g2 @ c(w2), [N, Cout], H, W, mh, mw, hb1, wb1, hb2, wb2)
    poison = torch.full((1 << 20,), float("nan"), device=gpu)  # the allocator hands these bytes to the output
    del poison
    got = dm.spectral_mode_contract(xf.to(gpu), w1.to(gpu), w2.to(gpu), mh, mw, hb1, wb1, hb2, wb2)
    assert got.shape == (N, Cout, H, W)
    mask = torch.zeros(H, W, dtype=torch.bool)
    mask[hb1:hb1 + mh, wb1:wb1 + mw] = True
    mask[hb2:hb2 + mh, wb2:wb2 + mw] = True
    gr = torch.view_as_real(got.cpu())
    assert (gr[:, :, ~mask] == 0).all()
    assert max_rel(gr.double(), torch.view_as_real(want)) < 1e-5


def test_spectral_mode_contract_golden(gpu):
    """Reference SpectralConv2D fixture: rfft2 / irfft2 by torch on the GPU, the middle by the fused kernel."""
    p, i, want, meta = load_golden("spectral_conv2d")
    m = int(meta["mode"])
    x = i["x"].to(gpu)
    N, r, _, cin = x.shape
    w = [p[f"fourier_weight.{k}"].permute(2, 3, 0, 1, 4).contiguous().to(gpu) for k in (0, 1)]  # GT -> Sp layout
    res = F.linear(x, p["residual_layer.weight"].to(gpu), p["residual_layer.bias"].to(gpu))
    xt = dm.batched_transpose(x, [N], [r, r], [cin])
    of = dm.spectral_mode_contract(torch.fft.rfft2(xt, s=(r, r), norm="ortho"), w[0], w[1], m, m, 0, 0, r - m, 0)
    y = torch.fft.irfft2(of, s=(r, r), norm="ortho")
    y = dm.batched_transpose(y, [N], [w[0].shape[3]], [r, r])
    got = F.silu(y + res)
    assert max_rel(got.cpu(), want) < 1e-4


@pytest.mark.parametrize("shape,size", [((2, 3, 7, 9), (7, 9)), ((2, 3, 7, 9), (4, 5)), ((2, 3, 7, 9), (13, 17)),
                                        ((1, 1, 5, 5), (1, 1)), ((1, 2, 1, 1), (3, 4)), ((4, 128, 211, 211), (122, 122)),
                                        ((2, 128, 71, 71), (122, 122)), ((1, 3, 2, 300), (5, 301))])
def test_bilinear_vs_oracle(gpu, shape, size):
    x = rnd(*shape, seed=14)
    want = O.bilinear_align_corners(x.double(), size)
    got = dm.bilinear_align_corners(x.to(gpu), size)
    assert got.shape == want.shape
    assert max_rel(got.cpu().double(), want) < 1e-5
    # torch's own fp32 kernel rounds the source coordinates differently; both sit within
    # ~1e-5 of the fp64 result, so they are compared at the path's stated 1e-4 tolerance
    lib = F.interpolate(x, size=size, mode="bilinear", align_corners=True)
    assert max_rel(got.cpu(), lib) < 1e-4


@pytest.mark.parametrize("shape,size", [((2, 4, 7, 9), (7, 9)), ((2, 4, 7, 9), (4, 5)), ((2, 4, 7, 9), (13, 17)),
                                        ((1, 4, 5, 5), (1, 1)), ((1, 8, 1, 1), (3, 4)), ((2, 128, 71, 71), (122, 122)),
                                        ((2, 128, 122, 122), (71, 71)), ((1, 4, 2, 300), (5, 301)),
                                        ((1, 4, 40, 33), (9, 7)), ((1, 12, 9, 7), (40, 33)), ((3, 5, 17, 12), (25, 30))])
def test_bilinear_adjoint_vs_oracle(gpu, shape, size):
    """The resampling's backward (both layouts, and the three autograd functions built on it) against autograd
    through the oracle's restatement in float64; up- and down-sampling, by more than two (sources no output reads),
    single rows and single outputs.  The source coordinates are formed in float32 as in the forward, which
    bounds the agreement with float64 at a few 1e-6 relative to the largest value."""
    x = rnd(*shape, seed=16)
    g = rnd(*shape[:2], *size, seed=17)
    xo = x.double().requires_grad_(True)
    O.bilinear_align_corners(xo, size).backward(g.double())
    want = xo.grad
    got = dm.bilinear_adjoint(g.to(gpu), shape[-2:])
    assert got.shape == want.shape
    assert max_rel(got.cpu().double(), want) < 5e-5
    xg = x.to(gpu).requires_grad_(True)
    dm.bilinear_train(xg, size).backward(g.to(gpu))
    assert max_rel(xg.grad.cpu().double(), want) < 5e-5
    if shape[1] % 4 == 0:
        got = dm.bilinear_adjoint(g.permute(0, 2, 3, 1).contiguous().to(gpu), shape[-2:], nhwc=True)
        assert max_rel(got.permute(0, 3, 1, 2).cpu().double(), want) < 5e-5
        xg = x.to(gpu).requires_grad_(True)
        y = dm.bilinear_to_nhwc_train(xg, size)
        assert max_rel(y.detach().permute(0, 3, 1, 2).cpu().double(), O.bilinear_align_corners(x.double(), size)) < 5e-5
        y.backward(g.permute(0, 2, 3, 1).to(gpu))
        assert max_rel(xg.grad.cpu().double(), want) < 5e-5
        xg = x.permute(0, 2, 3, 1).contiguous().to(gpu).requires_grad_(True)
        y = dm.bilinear_nhwc_train(xg, size)
        assert max_rel(y.detach().permute(0, 3, 1, 2).cpu().double(), O.bilinear_align_corners(x.double(), size)) < 5e-5
        y.backward(g.permute(0, 2, 3, 1).contiguous().to(gpu))
        assert max_rel(xg.grad.permute(0, 3, 1, 2).cpu().double(), want) < 5e-5


@pytest.mark.parametrize("hw,size", [((257, 257), (363, 363)), ((363, 363), (512, 512)), ((512, 512), (363, 363)),
                                      ((363, 363), (257, 257))])
def test_bilinear_adjoint_inner_product_at_the_model_sizes(gpu, hw, size):
    """<A x, g> = <x, A^T g> for the four resamplings of the r = 512 model with 128 channels, both layouts; the
    column sums of A^T g also equal those of g (the weights of an output sum to one)."""
    torch.manual_seed(5)
    x = torch.randn(2, 128, *hw, device=gpu)
    g = torch.randn(2, 128, *size, device=gpu)
    lhs = (dm.bilinear_align_corners(x, size).double() * g.double()).sum().item()
    a = dm.bilinear_adjoint(g, hw)
    assert abs((x.double() * a.double()).sum().item() - lhs) < 1e-6 * x.numel() ** 0.5 * 10
    assert max_rel(a.double().sum((2, 3)).cpu(), g.double().sum((2, 3)).cpu()) < 1e-6
    b = dm.bilinear_adjoint(g.permute(0, 2, 3, 1).contiguous(), hw, nhwc=True)
    assert max_rel(b.permute(0, 3, 1, 2).cpu(), a.cpu()) < 1e-6


def _kept_fraction_ok(keep, p, n_rows_tol=0.04):
    assert keep.float().mean().item() == pytest.approx(1 - p, abs=4e-3)
    flat = keep.reshape(-1, keep.shape[-1])
    assert (flat[:, 1:] & flat[:, :-1]).float().mean().item() == pytest.approx((1 - p) ** 2, abs=6e-3)
    assert (flat[1:] & flat[:-1]).float().mean().item() == pytest.approx((1 - p) ** 2, abs=6e-3)


def test_down_scaler_kernels_with_dropout(gpu):
    """ConvResBlock2D's dropout (conv -> dropout -> activation, network/layer.py:7-24, on in inference too) inside
    the three kernels that consume a convolution's sums.  The masks are the library's own, so the test is of their
    properties: a dropped sum is 0 and a kept one is scaled by 1 / (1 - p); kept fractions and neighbour
    correlations fit independent draws; one seed repeats and another differs; and a resampling reads the same
    decision for a source sample from every output that touches it (the resampled result equals the resampling of
    the same-size result under the same seed)."""
    g = torch.Generator().manual_seed(21)
    p = 0.3
    seed = torch.tensor([77, 99], dtype=torch.int32, device=gpu)
    seed2 = torch.tensor([78, 99], dtype=torch.int32, device=gpu)
    # bias + dropout + activation in place
    x = torch.randn(3, 20, 37, 41, generator=g).to(gpu)
    b = torch.randn(20, generator=g).to(gpu)
    plain = dm.bias_activation_nchw_(x.clone(), b, None)
    d = dm.bias_activation_nchw_(x.clone(), b, None, droprate=p, seed=seed)
    keep = d != 0
    assert torch.equal(d[keep], (plain / (1 - p))[keep]) or max_rel(d[keep].cpu(), (plain / (1 - p))[keep].cpu()) < 1e-6
    _kept_fraction_ok(keep, p)
    assert torch.equal(d, dm.bias_activation_nchw_(x.clone(), b, None, droprate=p, seed=seed))
    other = dm.bias_activation_nchw_(x.clone(), b, None, droprate=p, seed=seed2) != 0
    assert (keep != other).float().mean().item() == pytest.approx(2 * p * (1 - p), abs=6e-3)
    assert torch.equal(dm.bias_activation_nchw_(x.clone(), b, "relu", 2, droprate=p, seed=seed), torch.relu(d))
    assert not torch.equal(dm.bias_activation_nchw_(x.clone(), b, None, droprate=p),
                           dm.bias_activation_nchw_(x.clone(), b, None, droprate=p))
    # conv3x3 + bias + dropout + activation + resampling
    xi = torch.randn(2, 45, 52, 1, generator=g).to(gpu)
    w = torch.randn(24, 1, 3, 3, generator=g).to(gpu)
    cb = torch.randn(24, generator=g).to(gpu)
    same = dm.conv3x3_resample(xi, w, cb, (45, 52))
    same_d = dm.conv3x3_resample(xi, w, cb, (45, 52), droprate=p, seed=seed)
    keep = same_d != 0
    assert max_rel(same_d[keep].cpu(), (same / (1 - p))[keep].cpu()) < 1e-6
    _kept_fraction_ok(keep, p)
    for size in ((31, 29), (70, 81)):
        pre = dm.conv3x3_resample(xi, w, cb, (45, 52), pre_activation="silu", droprate=p, seed=seed)
        got = dm.conv3x3_resample(xi, w, cb, size, pre_activation="silu", post_activation="relu", droprate=p, seed=seed)
        want = torch.relu(dm.bilinear_align_corners(pre, size))
        assert max_rel(got.cpu(), want.cpu()) < 1e-5
    # concatenation whose last source is a convolution's sums without bias, dropout and activation
    x1, x2 = torch.randn(2, 8, 33, 35, generator=g).to(gpu), torch.randn(2, 8, 33, 35, generator=g).to(gpu)
    raw = torch.randn(2, 12, 33, 35, generator=g).to(gpu)
    b3 = torch.randn(12, generator=g).to(gpu)
    kw = dict(pre_biases=[None, None, b3], pre_flags=[0, 0, 1])
    same = dm.bilinear_resample_concat([x1, x2, raw], (33, 35), **kw)
    same_d = dm.bilinear_resample_concat([x1, x2, raw], (33, 35), pre_droprate=p, seed=seed, **kw)
    assert torch.equal(same_d[..., :16], same[..., :16])
    keep = same_d[..., 16:] != 0
    assert max_rel(same_d[..., 16:][keep].cpu(), (same[..., 16:] / (1 - p))[keep].cpu()) < 1e-6
    _kept_fraction_ok(keep.permute(0, 3, 1, 2), p)
    pre = dm.bilinear_resample_concat([x1, x2, raw], (33, 35), pre_activation="silu", pre_droprate=p, seed=seed, **kw)
    got = dm.bilinear_resample_concat([x1, x2, raw], (20, 23), pre_activation="silu", post_activation="relu",
                                      pre_droprate=p, seed=seed, **kw)
    want = torch.relu(dm.bilinear_align_corners(pre.permute(0, 3, 1, 2).contiguous(), (20, 23))).permute(0, 2, 3, 1)
    assert max_rel(got.cpu(), want.cpu()) < 1e-5
    with pytest.raises(Exception):
        dm.bias_activation_nchw_(x.clone(), b, None, droprate=1.5)


@pytest.mark.parametrize("N,hw,size,C", [(2, (9, 7), (13, 11), 8), (1, (21, 21), (29, 29), 128), (2, (5, 6), (5, 6), 4),
                                          (1, (4, 4), (12, 11), 12), (1, (7, 1), (9, 1), 4)])
def test_upsample_conv3x3_gather_adjoint(gpu, N, hw, size, C):
    """The backward of the nine-tap gather (UpScaler2D's interpolate -> conv3x3 as a Linear on the low-resolution
    tokens followed by a gather, network/model.py:59-62): against autograd in float64 through the oracle's
    resampling and torch's convolution on per-tap identity weights, and as an autograd function with its bias."""
    g = torch.Generator().manual_seed(31)
    Z = torch.randn(N, *hw, 9, C, generator=g)
    G = torch.randn(N, *size, C, generator=g)
    bias = torch.randn(C, generator=g)
    # oracle: out[n, y, x, c] = sum over taps of interp(Z_t)[y + ky - 1, x + kx - 1, c] (zero outside) + bias
    Zo = Z.double().requires_grad_(True)
    bo = bias.double().requires_grad_(True)
    up = O.bilinear_align_corners(Zo.permute(0, 3, 4, 1, 2).reshape(N, 9 * C, *hw), size).view(N, 9, C, *size)
    pad = torch.nn.functional.pad(up, (1, 1, 1, 1))
    want = sum(pad[:, 3 * ky + kx, :, ky:ky + size[0], kx:kx + size[1]] for ky in range(3) for kx in range(3))
    want = want.permute(0, 2, 3, 1) + bo
    want.backward(G.double())
    Zg = Z.to(gpu).requires_grad_(True)
    bg = bias.to(gpu).requires_grad_(True)
    got = dm.upsample_conv3x3_gather_train(Zg, bg, size)
    assert max_rel(got.detach().cpu().double(), want.detach()) < 5e-5
    got.backward(G.to(gpu))
    assert max_rel(Zg.grad.cpu().double(), Zo.grad) < 5e-5
    assert max_rel(bg.grad.cpu().double(), bo.grad) < 5e-5
    assert torch.equal(dm.upsample_conv3x3_gather_adjoint(G.to(gpu), hw), Zg.grad)


@pytest.mark.parametrize("Cin,Cout,hw,size,act,p", [(1, 24, (45, 52), (31, 37), "relu", 0.0),
                                                     (1, 128, (41, 41), (29, 29), "relu", 0.25),
                                                     (3, 10, (20, 33), (27, 40), "silu", 0.25),
                                                     (4, 6, (9, 8), (9, 8), None, 0.0), (2, 5, (12, 70), (5, 23), "silu", 0.0)])
def test_conv3x3_resample_backward(gpu, Cin, Cout, hw, size, act, p):
    """Weight and bias gradients of the down-scaler's first stage (conv3x3 -> dropout -> activation -> interpolate,
    network/model.py:30-33 with network/layer.py:7-24) from the kernel that forms the full-resolution chain again,
    against autograd in float64 through torch's convolution, the forward's own dropout mask (read off a same-size
    forward with the same seed) and the oracle's resampling."""
    g = torch.Generator().manual_seed(41)
    N = 2
    x = torch.randn(N, *hw, Cin, generator=g)
    w = torch.randn(Cout, Cin, 3, 3, generator=g) / 3.0
    b = torch.randn(Cout, generator=g)
    G = torch.randn(N, Cout, *size, generator=g)
    seed = torch.tensor([4242, 17], dtype=torch.int32, device=gpu)
    xg, wg, bg = x.to(gpu), w.to(gpu), b.to(gpu)
    wo, bo = w.double().requires_grad_(True), b.double().requires_grad_(True)
    z = torch.nn.functional.conv2d(x.double().permute(0, 3, 1, 2), wo, bo, padding=1)
    if p > 0:
        plain = dm.conv3x3_resample(xg, wg, bg, hw)
        dropped = dm.conv3x3_resample(xg, wg, bg, hw, droprate=p, seed=seed)
        mask = ((dropped != 0) | (plain == 0)).cpu().double()
        assert mask.mean().item() == pytest.approx(1 - p, abs=0.02)
        z = z * mask / (1 - p)
    a = z if act is None else (torch.relu(z) if act == "relu" else torch.nn.functional.silu(z))
    want = O.bilinear_align_corners(a, size)
    want.backward(G.double())
    got = dm.conv3x3_resample(xg, wg, bg, size, pre_activation=act, droprate=p, seed=seed if p > 0 else None)
    assert max_rel(got.cpu().double(), want.detach()) < 5e-5
    dW, db = dm.dexts.conv3x3_resample_backward(xg, wg, bg, G.to(gpu), act, p, seed if p > 0 else None)
    assert max_rel(dW.cpu().double(), wo.grad) < 1e-4
    assert max_rel(db.cpu().double(), bo.grad) < 1e-4
    # the autograd function (its own seed): gradients exist, and without dropout they are the ones above
    wt, bt = wg.clone().requires_grad_(True), bg.clone().requires_grad_(True)
    out = dm.conv3x3_resample_train(xg, wt, bt, size, act, p)
    out.backward(G.to(gpu))
    assert wt.grad.shape == w.shape and bt.grad.shape == b.shape
    if p == 0:
        assert torch.equal(wt.grad, dW) and torch.equal(bt.grad, db)


def test_bilinear_closed_forms(gpu):
    x = rnd(2, 3, 7, 9, seed=15).to(gpu)
    assert torch.equal(dm.bilinear_align_corners(x, (7, 9)), x)  # identity when sizes agree
    y = dm.bilinear_align_corners(x, (13, 17))
    assert torch.equal(y[..., 0, 0], x[..., 0, 0])
    assert torch.allclose(y[..., -1, -1], x[..., -1, -1], rtol=1e-6)


def test_datamove_argument_validation(gpu):
    lib = _lib.load()
    x = torch.zeros(4, 4, device=gpu)
    assert lib.spgt_batched_transpose(_lib.ptr(x), _lib.ptr(x), 1, 4, 4, None) == -1
    c = torch.zeros(2, 4, 4, dtype=torch.complex64, device=gpu)
    with pytest.raises(_lib.SpgtError):
        dm.transpose_gather_dual(c, [2], 4, 4, 3, 3, 0, 0, 2, 0)  # second window leaves the plane
    with pytest.raises(TypeError):
        dm.batched_transpose(x.double(), [1], [4], [4])


@pytest.mark.parametrize("N,Cin,Cout,m", [(1, 1, 1, 1), (2, 6, 4, 3), (8, 64, 64, 12), (17, 20, 70, 4)])
def test_spectral_modes_compact_vs_einsum(gpu, N, Cin, Cout, m):
    z = torch.view_as_complex(rnd(N, 2 * m, Cin, m, 2, seed=21))
    w1, w2 = rnd(m, m, Cin, Cout, 2, seed=22) / Cin, rnd(m, m, Cin, Cout, 2, seed=23) / Cin
    wc = torch.cat([torch.view_as_complex(w1.double()), torch.view_as_complex(w2.double())], 0)  # [2m, m, Cin, Cout]
    want = torch.einsum("nhiw,hwio->nhow", z.to(torch.complex128), wc)
    got = dm.spectral_modes_compact(z.to(gpu), w1.to(gpu), w2.to(gpu))
    assert got.shape == (N, 2 * m, Cout, m)
    assert max_rel(torch.view_as_real(got.cpu()).double(), torch.view_as_real(want)) < 1e-5


@pytest.mark.parametrize("N,r,Cin,Cout,m", [(2, 9, 6, 4, 3), (8, 141, 64, 64, 12), (4, 211, 64, 64, 12), (3, 16, 8, 8, 8),
                                             (2, 30, 5, 7, 15), (1, 421, 32, 32, 21), (1, 512, 32, 32, 23),
                                             (2, 211, 64, 64, 15), (1, 70, 64, 32, 32), (2, 141, 32, 32, 12)])
def test_truncated_dft_spectral_layer_vs_oracle(gpu, N, r, Cin, Cout, m):
    """The DFT-as-matrix-product route of the spectral layer against the oracle's rfft2 / irfft2 route (fp64)."""
    from spgt_amd.network import truncated_dft as T
    x = rnd(N, r, r, Cin, seed=24)
    w1, w2 = rnd(m, m, Cin, Cout, 2, seed=25) / Cin, rnd(m, m, Cin, Cout, 2, seed=26) / Cin
    p = {"residual_layer.weight": torch.zeros(Cout, Cin, dtype=torch.float64),
         "residual_layer.bias": torch.zeros(Cout, dtype=torch.float64),
         "fourier_weight.0": w1.double(), "fourier_weight.1": w2.double()}

    xf = torch.fft.rfft2(x.double().permute(0, 3, 1, 2), s=(r, r), norm="ortho")
    of = torch.zeros(N, Cout, r, r // 2 + 1, dtype=torch.complex128)
    of[:, :, :m, :m] = torch.einsum("nihw,hwio->nohw", xf[:, :, :m, :m], torch.view_as_complex(w1.double()))
    of[:, :, r - m:, :m] = torch.einsum("nihw,hwio->nohw", xf[:, :, r - m:, :m], torch.view_as_complex(w2.double()))
    want = torch.fft.irfft2(of, s=(r, r), norm="ortho").permute(0, 2, 3, 1)
    assert T.supported(r, m)
    got = T.spectral_modes_apply(x.to(gpu), w1.to(gpu), w2.to(gpu), m)
    assert got.shape == (N, r, r, Cout)
    assert max_rel(got.cpu().double(), want) < 1e-5
    # and the oracle's own module function agrees with the hand-written FFT reference above
    relu_want = O.spectral_conv2d(p, x.double(), m, "relu", weight_layout="sp")
    assert max_rel(relu_want, torch.relu(want)) < 1e-10


@pytest.mark.parametrize("shape,size", [((2, 3, 7, 9), (7, 9)), ((2, 3, 7, 9), (4, 5)), ((1, 128, 122, 122), (211, 211)),
                                        ((2, 130, 16, 33), (40, 65)), ((1, 1, 5, 5), (1, 1)), ((3, 40, 9, 9), (9, 70)),
                                        ((2, 132, 16, 33), (40, 65)), ((4, 128, 122, 122), (71, 71))])
def test_bilinear_nhwc_matches_nchw_kernel(gpu, shape, size):
    """The channels-last variant is the planar kernel followed by a permute, value for value."""
    x = rnd(*shape, seed=30).to(gpu)
    want = dm.bilinear_align_corners(x, size).permute(0, 2, 3, 1)
    got = dm.bilinear_align_corners_nhwc(x, size)
    assert got.is_contiguous() and got.shape == want.shape
    assert torch.equal(got, want)


def _act64(x, name, count=1):
    for _ in range(count if name else 0):
        x = torch.relu(x) if name == "relu" else x * torch.sigmoid(x)
    return x


@pytest.mark.parametrize("shape,size", [((2, 3, 7, 9), (4, 5)), ((1, 128, 71, 71), (122, 122)), ((2, 40, 9, 33), (9, 70)),
                                        ((1, 1, 5, 5), (1, 1)), ((2, 260, 6, 7), (11, 37)), ((2, 12, 9, 7), (9, 7))])
@pytest.mark.parametrize("src_nhwc,dst_nhwc", [(False, False), (False, True), (True, False)])
@pytest.mark.parametrize("pre,count,post", [(None, 0, None), ("silu", 1, "silu"), ("relu", 2, None), (None, 0, "relu"),
                                            ("silu", 2, None)])
def test_bilinear_resample_layouts_and_activations(gpu, shape, size, src_nhwc, dst_nhwc, pre, count, post):
    """post(interpolate(pre^count(x))) between layouts, against the float64 oracle resampling
    (network/model.py:30-38, 59-64 with the activations of network/layer.py:7-24 around it)."""
    x = rnd(*shape, seed=41)  # NCHW master copy
    want = _act64(O.bilinear_align_corners(_act64(x.double(), pre, count), size), post)
    src = x.permute(0, 2, 3, 1).contiguous() if src_nhwc else x
    got = dm.bilinear_resample(src.to(gpu), size, src_nhwc=src_nhwc, dst_nhwc=dst_nhwc, pre_activation=pre,
                               pre_count=max(count, 1), post_activation=post)
    assert got.is_contiguous()
    got = got.cpu().double()
    if dst_nhwc:
        got = got.permute(0, 3, 1, 2)
    assert got.shape == want.shape
    assert (got - want).abs().max().item() <= 1e-5 * max(1.0, want.abs().max().item())


@pytest.mark.parametrize("shape,size,E", [((2, 7, 9, 8), (13, 17), 2), ((1, 122, 122, 64), (211, 211), 2),
                                          ((3, 5, 5, 4), (5, 5), 0), ((2, 9, 4, 12), (3, 11), 4),
                                          ((1, 1, 1, 4), (3, 2), 1), ((2, 6, 6, 132), (1, 1), 3)])
def test_bilinear_nhwc_affine(gpu, shape, size, E):
    """Channels-last resampling plus extra @ W (network/model.py:63-64 followed by the grid columns of
    network/sp_model.py:60), against the float64 oracle resampling and a float64 matmul."""
    x = rnd(*shape, seed=71)
    N, _, _, C = shape
    want = O.bilinear_align_corners(x.double().permute(0, 3, 1, 2), size).permute(0, 2, 3, 1)
    extra = w = None
    if E:
        extra, w = rnd(N, size[0], size[1], E, seed=72), rnd(E, C, seed=73)
        want = want + extra.double() @ w.double()
    got = dm.bilinear_nhwc_affine(x.to(gpu), size, None if extra is None else extra.to(gpu),
                                  None if w is None else w.to(gpu))
    assert got.is_contiguous() and got.shape == want.shape
    assert (got.cpu().double() - want).abs().max().item() <= 1e-5 * max(1.0, want.abs().max().item())


@pytest.mark.parametrize("chans,hw,size", [((42, 42, 44), (13, 9), (7, 11)), ((4,), (5, 5), (9, 3)), ((3, 5), (6, 7), (6, 7)),
                                           ((100, 1, 1, 30), (4, 6), (9, 13)), ((42, 42, 44), (122, 122), (71, 71))])
@pytest.mark.parametrize("pre,count,post,flags", [(None, 0, None, None), ("silu", 1, "silu", (0, 0, 1, 1)),
                                                   ("relu", 2, "relu", (1, 0, 1, 0)), (None, 1, "silu", (1, 1, 1, 1))])
def test_bilinear_resample_concat(gpu, chans, hw, size, pre, count, post, flags):
    """cat -> interpolate -> permute -> activation (network/model.py:35-38) from the separate blocks, flagged ones
    still lacking bias and activation (network/layer.py:7-24), against the float64 oracle on the concatenation."""
    n = len(chans)
    xs = [rnd(2, c, hw[0], hw[1], seed=90 + s) for s, c in enumerate(chans)]
    bs = [rnd(c, seed=95 + s) if s % 2 == 0 else None for s, c in enumerate(chans)]
    fl = list(flags[:n]) if flags is not None else None
    parts = []
    for s in range(n):
        x = xs[s].double()
        if fl is not None and fl[s]:
            if bs[s] is not None:
                x = x + bs[s].double().view(1, -1, 1, 1)
            x = _act64(x, pre, count)
        parts.append(x)
    want = _act64(O.bilinear_align_corners(torch.cat(parts, dim=1), size), post).permute(0, 2, 3, 1)
    got = dm.bilinear_resample_concat([x.to(gpu) for x in xs], size,
                                      pre_biases=[None if b is None else b.to(gpu) for b in bs] if fl else None,
                                      pre_flags=fl, pre_activation=pre, pre_count=max(count, 1), post_activation=post)
    assert got.is_contiguous() and got.shape == want.shape
    assert (got.cpu().double() - want).abs().max().item() <= 1e-5 * max(1.0, want.abs().max().item())


def test_bilinear_resample_concat_rejects(gpu):
    x = rnd(1, 3, 4, 4, seed=1).to(gpu)
    with pytest.raises(ValueError):
        dm.bilinear_resample_concat([x, x], (5, 5))  # 6 channels
    with pytest.raises(ValueError):
        dm.bilinear_resample_concat([x] * 5, (5, 5))
    with pytest.raises(ValueError):
        dm.bilinear_resample_concat([x, rnd(1, 1, 4, 5, seed=2).to(gpu)], (5, 5))


@pytest.mark.parametrize("N,hw,size,cin,cout", [(2, (5, 7), (9, 12), 6, 8), (1, (71, 71), (122, 122), 16, 128),
                                                 (2, (4, 4), (4, 4), 3, 4), (1, (3, 5), (1, 2), 5, 12),
                                                 (2, (1, 1), (3, 3), 2, 4)])
@pytest.mark.parametrize("act,count", [(None, 1), ("relu", 1), ("silu", 2)])
def test_upsample_conv3x3_gather(gpu, N, hw, size, cin, cout, act, count):
    """interpolate -> conv3x3(padding 1) -> bias -> activations (network/model.py:59-62) from the per-tap products
    of the low-resolution input, against torch's float64 convolution of the float64 oracle resampling."""
    x = rnd(N, cin, hw[0], hw[1], seed=101).double()
    w = rnd(cout, cin, 3, 3, seed=102).double()
    b = rnd(cout, seed=103).double()
    want = torch.nn.functional.conv2d(O.bilinear_align_corners(x, size), w, b, padding=1)
    want = _act64(want, act, count).permute(0, 2, 3, 1)
    # Z[n, h, w, 3 ky + kx, co] = sum_ci x[n, ci, h, w] * w[co, ci, ky, kx]
    Z = torch.einsum("nchw,ocyx->nhwyxo", x, w).reshape(N, hw[0], hw[1], 9, cout).float().contiguous()
    got = dm.upsample_conv3x3_gather(Z.to(gpu), b.float().to(gpu), size, act, count)
    assert got.is_contiguous() and got.shape == want.shape
    assert (got.cpu().double() - want).abs().max().item() <= 2e-5 * max(1.0, want.abs().max().item())
    no_bias = dm.upsample_conv3x3_gather(Z.to(gpu), None, size, None, 1).cpu().double()
    want0 = torch.nn.functional.conv2d(O.bilinear_align_corners(x, size), w, None, padding=1).permute(0, 2, 3, 1)
    assert (no_bias - want0).abs().max().item() <= 2e-5 * max(1.0, want0.abs().max().item())


def test_upsample_conv3x3_gather_rejects(gpu):
    with pytest.raises(ValueError):
        dm.upsample_conv3x3_gather(rnd(1, 4, 4, 8, 4, seed=1).to(gpu), None, (5, 5))  # 8 taps
    with pytest.raises(ValueError):
        dm.upsample_conv3x3_gather(rnd(1, 4, 4, 9, 6, seed=1).to(gpu), None, (5, 5))  # 6 channels
    with pytest.raises(ValueError):
        dm.upsample_conv3x3_gather(rnd(1, 4, 4, 9, 4, seed=1).to(gpu), rnd(5, seed=2).to(gpu), (5, 5))


def test_bilinear_nhwc_affine_rejects(gpu):
    with pytest.raises(ValueError):
        dm.bilinear_nhwc_affine(rnd(1, 4, 4, 6, seed=1).to(gpu), (5, 5))  # 6 channels: not a multiple of 4
    with pytest.raises(ValueError):
        dm.bilinear_nhwc_affine(rnd(1, 4, 4, 8, seed=1).to(gpu), (5, 5), rnd(1, 5, 5, 5, seed=2).to(gpu),
                                rnd(5, 8, seed=3).to(gpu))  # more than 4 extra columns


def test_resampling_to_the_same_size_copies(gpu):
    """Weights (1, 0): the layout-changing kernels double as bias + activation + permute."""
    x = rnd(2, 12, 9, 7, seed=81).to(gpu)
    assert torch.equal(dm.bilinear_resample(x, (9, 7), dst_nhwc=True), x.permute(0, 2, 3, 1).contiguous())
    assert torch.equal(dm.bilinear_resample(x, (9, 7)), x)


def test_bilinear_resample_rejects(gpu):
    x = rnd(1, 4, 5, 5, seed=1).to(gpu)
    with pytest.raises(ValueError):
        dm.bilinear_resample(x, (3, 3), src_nhwc=True, dst_nhwc=True)
    with pytest.raises(ValueError):
        dm.bilinear_resample(x, (3, 3), pre_activation="tanh")


@pytest.mark.parametrize("shape", [(2, 5, 7, 9), (4, 42, 122, 122), (1, 3, 1), (2, 128, 33, 31)])
@pytest.mark.parametrize("act,count", [(None, 1), ("relu", 1), ("silu", 1), ("silu", 2), ("relu", 2)])
@pytest.mark.parametrize("with_bias", [True, False])
def test_bias_activation_nchw(gpu, shape, act, count, with_bias):
    """In-place bias + activation(s) after a bias-free convolution (network/layer.py:7-24), against float64."""
    x = rnd(*shape, seed=51)
    b = rnd(shape[1], seed=52) if with_bias else None
    want = x.double()
    if with_bias:
        want = want + b.double().view(1, -1, *([1] * (len(shape) - 2)))
    want = _act64(want, act, count)
    xd = x.to(gpu)
    got = dm.bias_activation_nchw_(xd, b.to(gpu) if with_bias else None, act, count)
    assert got.data_ptr() == xd.data_ptr()
    assert (got.cpu().double() - want).abs().max().item() <= 1e-5 * max(1.0, want.abs().max().item())


@pytest.mark.parametrize("src_nhwc,dst_nhwc", [(False, False), (False, True), (True, False)])
def test_bilinear_resample_pre_bias(gpu, src_nhwc, dst_nhwc):
    """The bias of a bias-free convolution added to the source samples before the activation."""
    x = rnd(2, 40, 9, 33, seed=61)
    b = rnd(40, seed=62)
    want = O.bilinear_align_corners(_act64(x.double() + b.double().view(1, -1, 1, 1), "silu"), (13, 20))
    src = x.permute(0, 2, 3, 1).contiguous() if src_nhwc else x
    got = dm.bilinear_resample(src.to(gpu), (13, 20), src_nhwc=src_nhwc, dst_nhwc=dst_nhwc, pre_activation="silu",
                               pre_bias=b.to(gpu)).cpu().double()
    if dst_nhwc:
        got = got.permute(0, 3, 1, 2)
    assert (got - want).abs().max().item() <= 1e-5 * max(1.0, want.abs().max().item())


@pytest.mark.parametrize("rows,r,C,m", [(3, 211, 64, 12), (5, 16, 32, 8), (2, 33, 96, 16), (1, 7, 32, 3), (844, 211, 64, 12),
                                        (3, 421, 32, 21), (2, 512, 64, 23), (2, 65, 96, 32), (5, 35, 32, 17),
                                        (2, 511, 32, 24), (2, 100, 128, 20), (2, 101, 256, 19), (3, 34, 192, 17),
                                        (2, 40, 128, 20)])
def test_truncated_dft_rows_against_float64(gpu, rows, r, C, m):
    """Both row kernels against float64 matrix products with the same tables, and the forward one against
    torch.fft.rfft on the CPU (network/sp_layer.py:136-141 keeps columns kw < m of the ortho-normalised rfft2)."""
    from spgt_amd.network.truncated_dft import dft_tables
    fw, _, _, fwi = dft_tables(max(r, 2 * m), m, "cpu") if r >= 2 * m else dft_tables(r, m, "cpu")
    fw, fwi = fw[:r].contiguous(), fwi[:r].contiguous()
    x = rnd(rows, r, C, seed=71)
    got = dm.truncated_dft_rows_forward(x.to(gpu), fw.to(gpu)).cpu().double()
    want = torch.matmul(x.double().transpose(1, 2), fw.double())
    assert got.shape == (rows, C, 2 * m)
    assert (got - want).abs().max().item() <= 1e-5 * max(1.0, want.abs().max().item())
    if r >= 2 * m:
        ft = torch.fft.rfft(x.double(), dim=1, norm="ortho")[:, :m]          # [rows, m, C]
        ref = torch.view_as_real(ft.permute(0, 2, 1).contiguous()).reshape(rows, C, 2 * m)
        assert (got - ref).abs().max().item() <= 1e-5 * max(1.0, ref.abs().max().item())
    u = rnd(rows, C, 2 * m, seed=72)
    got = dm.truncated_dft_rows_inverse(u.to(gpu), fwi.to(gpu)).cpu().double()
    want = torch.matmul(fwi.double(), u.double().transpose(1, 2))
    assert got.shape == (rows, r, C)
    assert (got - want).abs().max().item() <= 1e-5 * max(1.0, want.abs().max().item())


def test_truncated_dft_rows_rejects(gpu):
    from spgt_amd._lib import SpgtError
    assert not dm.truncated_dft_rows_supported(211, 48, 12)
    assert dm.truncated_dft_rows_supported(211, 64, 17) and dm.truncated_dft_rows_supported(512, 64, 32)
    assert not dm.truncated_dft_rows_supported(211, 64, 33) and not dm.truncated_dft_rows_supported(513, 64, 17)
    assert dm.truncated_dft_rows_supported(1024, 64, 16) and not dm.truncated_dft_rows_supported(1025, 64, 16)
    with pytest.raises(SpgtError):
        dm.truncated_dft_rows_forward(rnd(2, 9, 48, seed=1).to(gpu), rnd(9, 8, seed=2).to(gpu))


@pytest.mark.parametrize("N,r,cin,cout,m", [(2, 211, 64, 64, 12), (1, 21, 32, 32, 4), (3, 16, 64, 32, 8), (2, 33, 24, 40, 16),
                                            (1, 421, 32, 32, 21), (1, 512, 64, 64, 23), (2, 64, 17, 9, 32),
                                            (1, 1500, 8, 8, 20), (2, 128, 128, 32, 12), (1, 256, 128, 32, 16),
                                            (1, 512, 128, 64, 23), (2, 37, 100, 24, 9), (1, 45, 65, 64, 7)])
def test_spectral_modes_middle_against_float64(gpu, N, r, cin, cout, m):
    """DFT along h onto the kept rows, complex contraction, inverse DFT along h (network/sp_layer.py:136-151
    restricted to the kept modes) against the same three products in float64."""
    from spgt_amd.network.truncated_dft import dft_tables
    _, gh, ghi, _ = dft_tables(r, m, "cpu")
    y = rnd(N, 2 * m, r, cin, seed=81)
    w1, w2 = rnd(m, m, cin, cout, 2, seed=82) / cin ** 0.5, rnd(m, m, cin, cout, 2, seed=83) / cin ** 0.5
    assert dm.spectral_modes_middle_supported(r, cin, cout, m)
    got = dm.spectral_modes_middle(y.to(gpu), gh.to(gpu), ghi.to(gpu), w1.to(gpu), w2.to(gpu)).cpu().double()
    yc = torch.complex(y[:, 0::2].double(), y[:, 1::2].double())               # [N, kw, h, c]
    z = torch.einsum("kh,nwhc->nkcw", gh.to(torch.complex128), yc)             # [N, kh, c, kw]
    wc = torch.cat([torch.view_as_complex(w1.double()), torch.view_as_complex(w2.double())], 0)  # [2m kh, kw, c, o]
    o = torch.einsum("nkcw,kwco->nkow", z, wc)
    u = torch.einsum("hk,nkow->nwho", ghi.to(torch.complex128), o)             # [N, kw, h, o]
    want = torch.stack([u.real, u.imag], 2).reshape(N, 2 * m, r, cout)
    assert got.shape == want.shape
    assert (got - want).abs().max().item() <= 1e-5 * max(1.0, want.abs().max().item())


@pytest.mark.parametrize("r,C,m", [(33, 64, 8), (70, 128, 20), (45, 64, 18), (35, 32, 17), (64, 256, 32)])
def test_truncated_dft_rows_planar_layout(gpu, r, C, m):
    """planar=True is the interleaved result with the mode axis moved ahead of the grid row (also for more than
    16 modes, where the forward kernel folds the grid row and loads several channels per lane)."""
    from spgt_amd.network.truncated_dft import dft_tables
    fw, _, _, fwi = dft_tables(r, m, "cpu")
    x = rnd(2, r, r, C, seed=91).to(gpu)
    a = dm.truncated_dft_rows_forward(x.view(2 * r, r, C), fw.to(gpu)).view(2, r, C, 2 * m)
    b = dm.truncated_dft_rows_forward(x, fw.to(gpu), planar=True)
    assert torch.equal(b, a.permute(0, 3, 1, 2).contiguous())
    u = rnd(2, 2 * m, r, C, seed=92).to(gpu)
    c = dm.truncated_dft_rows_inverse(u, fwi.to(gpu), planar=True)
    d = dm.truncated_dft_rows_inverse(u.permute(0, 2, 3, 1).contiguous().view(2 * r, C, 2 * m), fwi.to(gpu)).view(2, r, r, C)
    assert torch.equal(c, d)


@pytest.mark.parametrize("N,H,W,cin,cout,size", [(2, 21, 21, 1, 128, (15, 15)), (1, 9, 13, 3, 20, (17, 5)), (2, 33, 33, 4, 7, (33, 33)),
                                                 (1, 211, 211, 1, 128, (122, 122)), (1, 5, 5, 2, 3, (1, 1))])
@pytest.mark.parametrize("pre,post", [("silu", "silu"), ("relu", None), (None, None)])
def test_conv3x3_resample(gpu, N, H, W, cin, cout, size, pre, post):
    """conv3x3 (padding 1) + bias + activation + bilinear resampling + activation in one pass
    (network/model.py:30-33 with network/layer.py:7-24) against torch's float64 conv2d and the oracle resampling."""
    x = rnd(N, H, W, cin, seed=101)
    w = rnd(cout, cin, 3, 3, seed=102) / 3.0
    b = rnd(cout, seed=103)
    conv = F.conv2d(x.permute(0, 3, 1, 2).double(), w.double(), b.double(), padding=1)
    want = _act64(O.bilinear_align_corners(_act64(conv, pre), size), post)
    assert dm.conv3x3_resample_supported(cin) and not dm.conv3x3_resample_supported(5)
    got = dm.conv3x3_resample(x.to(gpu), w.to(gpu), b.to(gpu), size, pre, post).cpu().double()
    assert got.shape == want.shape
    # fp32 source coordinates (as torch's own kernel computes them) times the slope of a random convolution
    # output reach 1e-5 of the output scale at 211 -> 122; the bound is 3e-5, far inside the path's 1e-4
    assert (got - want).abs().max().item() <= 3e-5 * max(1.0, want.abs().max().item())


@pytest.mark.parametrize("shape", [(2, 9, 7, 1), (1, 2, 5, 3), (3, 2, 2, 2), (4, 211, 211, 1)])
@pytest.mark.parametrize("per_point", [False, True])
@pytest.mark.parametrize("zero_boundary", [False, True])
def test_denormalize_boundary_matches_tensor_ops(gpu, shape, per_point, zero_boundary):
    """The end of the model's forward (network/sp_model.py:109-111): X * (std + eps) + mean, then the interior
    padded with zeros.  Bit-exact against the tensor operations it replaces."""
    import torch.nn.functional as F
    from spgt_amd.extension.bind.datamove import denormalize_boundary
    g = torch.Generator().manual_seed(sum(shape))
    X = torch.randn(*shape, generator=g).to(gpu)
    if per_point:
        scale = (torch.rand(*shape[1:], generator=g) + 0.5).to(gpu)
        shift = torch.randn(*shape[1:], generator=g).to(gpu)
    else:
        scale = torch.tensor([1.7 + 1e-5], device=gpu)
        shift = torch.tensor([-0.3], device=gpu)
    got = denormalize_boundary(X, scale, shift, zero_boundary)
    want = X * scale + shift
    if zero_boundary:
        want = F.pad(want[:, 1:-1, 1:-1], (0, 0, 1, 1, 1, 1), "constant", 0.0)
    assert got.shape == want.shape and torch.equal(got, want)


def test_denormalize_boundary_rejects_bad_shapes(gpu):
    from spgt_amd.extension.bind.datamove import denormalize_boundary
    X = torch.zeros(2, 4, 4, 1, device=gpu)
    with pytest.raises(ValueError):
        denormalize_boundary(X, torch.ones(3, device=gpu), torch.ones(3, device=gpu), True)
    with pytest.raises(ValueError):
        denormalize_boundary(X[0], torch.ones(1, device=gpu), torch.ones(1, device=gpu), True)



@pytest.mark.parametrize("N,r,m,C", [(1, 33, 4, 64), (2, 64, 12, 64), (4, 211, 12, 64), (2, 141, 16, 64), (1, 32, 16, 64),
                                     (1, 40, 6, 64), (2, 7, 3, 64), (3, 5, 1, 64), (1, 97, 9, 64), (1, 421, 21, 64),
                                     (1, 512, 23, 64), (1, 64, 32, 64), (2, 45, 17, 64), (1, 100, 25, 64),
                                     (2, 141, 12, 32), (1, 421, 21, 32), (1, 512, 23, 32), (2, 7, 3, 32),
                                     (1, 33, 16, 32), (1, 70, 32, 32), (3, 40, 6, 32)])
@pytest.mark.parametrize("act", [None, "relu", "silu"])
def test_spectral_inverse_linear_matches_separate_kernels(gpu, N, r, m, C, act):
    """The fused end of the spectral layer against its parts: truncated_dft_rows_inverse + fused_linear with the
    transform's result as residual (which are tested against the FFT route and a float64 product themselves).
    Tolerance 2e-6 of the output scale: the fused kernel adds the spectral term in the accumulator, the parts
    round it to fp32 in memory first."""
    from spgt_amd.extension.bind.linear import fused_linear
    from spgt_amd.network.truncated_dft import dft_tables
    assert dm.spectral_inverse_linear_supported(r, C, C, m) and not dm.spectral_inverse_linear_supported(r, 96, 96, m)
    assert not dm.spectral_inverse_linear_supported(r, 32, 64, m)
    g = torch.Generator().manual_seed(N * 1000 + r + m)
    x = torch.randn(N, r, r, C, generator=g).to(gpu)
    U = torch.randn(N, 2 * m, r, C, generator=g).to(gpu)
    w = (torch.randn(C, C, generator=g) / 8.0).to(gpu)
    b = torch.randn(C, generator=g).to(gpu)
    _, _, _, fwi = dft_tables(r, m, gpu)
    got = dm.spectral_inverse_linear(U, dm.inverse_table_operand(fwi), x, w, b, act)
    y = dm.truncated_dft_rows_inverse(U, fwi, planar=True)
    activate = {None: lambda t: t, "relu": torch.relu, "silu": torch.nn.functional.silu}[act]
    parts = (lambda bias: fused_linear(x, w, bias, act or "none", y)) if C == 64 else \
        (lambda bias: activate(x @ w + (0 if bias is None else bias) + y))
    want = parts(b)
    assert got.shape == want.shape
    tol = 2e-6 if C == 64 else 1e-5  # the library product behind the 32-channel comparison may not be plain fp32
    assert (got - want).abs().max().item() <= tol * max(1.0, want.abs().max().item())
    # and against float64 arithmetic
    y64 = torch.einsum("wj,njho->nhwo", fwi.double(), U.double())
    z = x.double() @ w.double() + b.double() + y64
    z = torch.relu(z) if act == "relu" else (z * torch.sigmoid(z) if act == "silu" else z)
    assert (got.double() - z).abs().max().item() <= 1e-5 * max(1.0, z.abs().max().item())
    no_bias = dm.spectral_inverse_linear(U, dm.inverse_table_operand(fwi), x, w, None, act)
    want_nb = parts(None)
    assert (no_bias - want_nb).abs().max().item() <= tol * max(1.0, want_nb.abs().max().item())


@pytest.mark.parametrize("N,r,m", [(1, 33, 4), (4, 128, 12), (2, 256, 16), (1, 512, 23), (2, 7, 3), (1, 100, 25), (1, 70, 32)])
@pytest.mark.parametrize("cin,cout", [(128, 32), (128, 64), (64, 32)])
@pytest.mark.parametrize("act", [None, "silu"])
def test_spectral_inverse_linear_unequal_widths(gpu, N, r, m, cin, cout, act):
    """The same kernel with more input than output channels (the reference's own spectral-layer benchmark is
    128 -> 32, evaluate/sp_fno2d.py:12-14) against float64 arithmetic, with and without bias."""
    from spgt_amd.network.truncated_dft import dft_tables
    assert dm.spectral_inverse_linear_supported(r, cin, cout, m)
    assert not dm.spectral_inverse_linear_supported(r, 32, 128, m)
    g = torch.Generator().manual_seed(N * 977 + r + m + cin + cout)
    x = torch.randn(N, r, r, cin, generator=g).to(gpu)
    U = torch.randn(N, 2 * m, r, cout, generator=g).to(gpu)
    w = (torch.randn(cin, cout, generator=g) / cin ** 0.5).to(gpu)
    b = torch.randn(cout, generator=g).to(gpu)
    _, _, _, fwi = dft_tables(r, m, gpu)
    y64 = torch.einsum("wj,njho->nhwo", fwi.double(), U.double())
    for bias in (b, None):
        got = dm.spectral_inverse_linear(U, dm.inverse_table_operand(fwi), x, w, bias, act)
        z = x.double() @ w.double() + (0 if bias is None else bias.double()) + y64
        z = z * torch.sigmoid(z) if act == "silu" else z
        assert got.shape == (N, r, r, cout)
        assert (got.double() - z).abs().max().item() <= 1e-5 * max(1.0, z.abs().max().item())
